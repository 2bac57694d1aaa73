// Host-side declarations shared by the C ABI (ffa_api.cpp, pure host C++), the planner
// and the kernel launchers (ffa_kernels.hip).
#pragma once

#include <stddef.h>
#include <stdint.h>

#include "ffa_c_api.h"

namespace ffa {

constexpr int kTileKeys = 64;            // keys per wave tile (= wavefront size)
constexpr int kMaxSplits = 128;          // upper bound on workgroups per (batch, head)
constexpr int kMaxSplitWorkgroups = 16384;  // upper bound on workgroups of a split launch
constexpr int kMaxDynamicLdsBytes = 160 * 1024 - 20 * 1024;  // gfx950: 160 KiB LDS per CU, minus statics
                                                             // (16 KiB of survivor queues at 16 waves)

// Bytes per element of a precision code (fp16 and bf16: 2, fp32: 4; 0 = unknown).
inline int elem_bytes(int precision) {
    return precision == FFA_PRECISION_F32 ? 4 : (precision == FFA_PRECISION_F16 || precision == FFA_PRECISION_BF16) ? 2 : 0;
}
// The planner and its table know two element sizes: bf16 plans like fp16.
inline int planner_precision(int precision) { return precision == FFA_PRECISION_BF16 ? FFA_PRECISION_F16 : precision; }

// Arguments of one decode step, after validation.
struct DecodeArgs {
    int precision;
    int B, H, Dh, Lmax, t;
    float scale, p;
    const void *q, *k, *v;
    void *k_cache, *v_cache, *out;
    const int* seq_lengths;
    int right_or_no_padding;
    uint32_t* kept_count;
    uint8_t* skip_mask;
    void* stream;
    // Bias and rotary embedding applied to the new token before the step (all optional).
    const void *q_bias = nullptr, *k_bias = nullptr, *v_bias = nullptr;  // [H, Dh]
    int rotary_dim = 0;
    float rotary_base = 10000.f;
    // Beam-search indirection (optional): source beam of every cached key, [B, Lmax].
    const int* cache_indir = nullptr;
    int beam_width = 1;

    // ffa_load_floor: launch the load-only probe of the plan instead of the decode kernel.
    bool floor_probe = false;

    bool transforms_token() const { return q_bias || k_bias || v_bias || rotary_dim > 0; }
};


// Kernel parameters of one decode launch (passed by value).
struct DecodeParams {
    const void* q;
    const void* k;
    const void* v;
    void* k_cache;
    void* v_cache;
    void* out;
    const int* seq_lengths;
    float* ws_acc;         // split launch: [split pairs, n_splits, Dh + kSlotTailFloats]; two-pass: [BH, n_splits, Dh]
    float* ws_ml;          // two-pass: [BH, n_splits, 2]
    unsigned int* ws_cnt;  // [BH] arrival counters, kCounterStride words apart
    float* ws_scores;      // [BH, score_stride] raw q.k of the two-pass path
    int score_stride;      // floats per (b,h) row of ws_scores, a multiple of 64
    unsigned int* kept_count;
    unsigned char* skip_mask;
    int B, H, Lmax, t;
    float scale_log2e;  // softmax_scale * log2(e): scores live in the exp2 domain
    float p;
    int right_or_no_padding;
    int n_splits, tiles_per_split;
    unsigned split_magic;  // floor(2^32 / n_splits) + 1, or 0 for n_splits = 1: quotients without a division
    int n_whole;  // (b,h) pairs [0, n_whole) get one workgroup each; the rest are split
    int bh_total;
    int combine;  // FFA_COMBINE_*
    const int* cache_indir;  // [B, Lmax] source beam of every cached key, or nullptr
    int beam_width;          // samples per beam group (>= 1)
    // Transform of the new token (all optional): biases [H, Dh], rotary embedding of q and k.
    const void *q_bias, *k_bias, *v_bias;
    int rotary_dim;          // 0 = none
    int xform;               // any bias or a rotary embedding present
    double rotary_coef;      // -2 log2(base) / rotary_dim: angle of pair z = pos * 2^(z * coef)
    int floor_probe;         // launch ffa_load_floor_kernel instead of the decode kernel
    int store_through;       // split launch without whole pairs: outputs and appended rows are written through
};

// Carved-up workspace for a given plan.
struct WorkspaceView {
    unsigned int* cnt;  // [B*H] arrival counters, zero between launches
    float* ml;          // two-pass: [B*H, n_splits, 2] piece (max, sum)
    float* acc;         // split: [split pairs, n_splits, Dh + kSlotTailFloats]; two-pass: [B*H, n_splits, Dh]
    float* scores;      // two-pass path: [B*H, score_stride] raw scores
    int score_stride;
};

inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

inline int num_tiles(int t) { return t / kTileKeys + 1; }  // keys 0..t inclusive

// Dynamic LDS of the one-workgroup-per-(b,h) kernel: the larger of the score buffer and
// the cross-wave merge buffer.
inline size_t wg_dynamic_lds_bytes(int t, int waves, int elem_bytes) {
    const size_t scores = (size_t)num_tiles(t) * kTileKeys * sizeof(float);
    const size_t merge = (size_t)waves * 64 * (16 / elem_bytes) * sizeof(float);
    return scores > merge ? scores : merge;
}

// Largest n_splits any plan may carry for this problem.
inline int max_splits_for(int bh, int max_seq_len) {
    int by_len = (max_seq_len + kTileKeys - 1) / kTileKeys;
    int by_grid = kMaxSplitWorkgroups / (bh > 0 ? bh : 1);
    int m = kMaxSplits;
    if (by_len < m) m = by_len;
    if (by_grid < m) m = by_grid;
    return m < 1 ? 1 : m;
}

// Arrival counters sit kCounterStride words apart: one per 256 bytes, so that the read-modify-writes
// of different (batch, head) pairs, which arrive in bursts, do not queue up on one cache line.
constexpr int kCounterStride = 64;
inline size_t workspace_counter_bytes(int bh) { return (size_t)bh * kCounterStride * sizeof(unsigned int); }

// A partial of the exact split launch: accumulator [Dh], then (max, sum), padded to whole 256-byte
// lines so that workgroups never write into each other's lines.
constexpr int kSlotTailFloats = 64;
// bh = all (batch, head) pairs (counter array), split_heads = pairs that are split:
// [counters][split_heads x n_splits slots].
inline size_t workspace_bytes_for(int bh, int split_heads, int head_dim, int n_splits) {
    if (n_splits <= 1 || split_heads <= 0) return workspace_counter_bytes(bh);
    return workspace_counter_bytes(bh) + (size_t)split_heads * n_splits * (head_dim + kSlotTailFloats) * sizeof(float);
}

// Two-pass path: counters, piece (max, sum) [bh, n_splits, 2], partial outputs
// [bh, n_splits, Dh], scores [bh, stride].
inline int score_stride_for(int max_seq_len) { return (max_seq_len / kTileKeys + 1) * kTileKeys; }
inline size_t two_pass_workspace_bytes(int bh, int head_dim, int n_splits, int max_seq_len) {
    return workspace_counter_bytes(bh) + align_up((size_t)bh * n_splits * 2 * sizeof(float), 256) +
           align_up((size_t)bh * n_splits * head_dim * sizeof(float), 256) +
           align_up((size_t)bh * score_stride_for(max_seq_len) * sizeof(float), 256);
}

// Bytes of workspace one given plan needs (0 for plans that use none).
inline size_t plan_workspace_bytes(const ffa_launch_plan& plan, int bh, int head_dim, int max_seq_len) {
    if (plan.kind == FFA_LAUNCH_TWO_PASS) return two_pass_workspace_bytes(bh, head_dim, plan.n_splits, max_seq_len);
    const int split_heads = bh - plan.whole_heads;
    if (plan.kind == FFA_LAUNCH_SPLIT && plan.n_splits > 1 && split_heads > 0)
        return workspace_bytes_for(bh, split_heads, head_dim, plan.n_splits);
    return 0;
}

// Size of the library's own scratch array (one per GPU, held until the process ends), used by
// ffa_attention_static_scratch in place of a caller-owned workspace.
constexpr size_t kStaticScratchBytes = FFA_STATIC_SCRATCH_BYTES;

// planner (ffa_plan.cpp)
int plan_launch(int precision, int B, int H, int Dh, int t, float p, int use_default, int cus,
                ffa_launch_plan* plan);
// use_table = 0: the rules alone (what the sweep compares the table against).
int plan_launch_ex(int precision, int B, int H, int Dh, int t, float p, int use_default, int cus,
                   int use_table, ffa_launch_plan* plan);
int validate_plan(const ffa_launch_plan& plan, int precision, int head_dim, int bh, int t, float p);
// Where the tuned plan of a problem comes from: 0 = the rules, 1 = a row of the table of the
// BASELINE shapes, 2 = the nearest row of the grid.
int plan_source(int precision, int B, int H, int Dh, int t, float p, int cus);
bool tpk_supported(int precision, int head_dim, int tpk);

// launchers (ffa_kernels.hip; the decode kernels of each element type, with and without the
// transform of the new token, are a translation unit of their own: ffa_decode_<type>[_xform].hip)
int launch_decode(const DecodeArgs& a, const ffa_launch_plan& plan, const WorkspaceView& ws);
int launch_decode_f16(const DecodeParams& P, int head_dim, const ffa_launch_plan& plan, void* stream);
int launch_decode_bf16(const DecodeParams& P, int head_dim, const ffa_launch_plan& plan, void* stream);
int launch_decode_f32(const DecodeParams& P, int head_dim, const ffa_launch_plan& plan, void* stream);
int launch_decode_f16_xform(const DecodeParams& P, int head_dim, const ffa_launch_plan& plan, void* stream);
int launch_decode_bf16_xform(const DecodeParams& P, int head_dim, const ffa_launch_plan& plan, void* stream);
int launch_decode_f32_xform(const DecodeParams& P, int head_dim, const ffa_launch_plan& plan, void* stream);
constexpr int kMaxDevices = 64;
int current_device();  // index of the current HIP device, -1 if none or beyond kMaxDevices
int launch_init_cache(int precision, void* k_dst, void* v_dst, const void* k_src,
                      const void* v_src, int B, int H, int L, int Lmax, int Dh, void* stream);
int launch_fill_u32(unsigned int* p, size_t n, unsigned int v, void* stream);
int query_compute_units();
// Device address of the current device's copy of the static scratch array (resolved once per
// device); FFA_ERR_NO_DEVICE if the runtime cannot resolve it.
int static_scratch_address(void** ptr);

}  // namespace ffa
