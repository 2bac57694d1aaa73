// C ABI of the decode-attention engine: argument validation, planning, workspace carving.
// Pure host C++ (no device code, no HIP headers); the launchers live in ffa_kernels.hip.
#include <math.h>
#include <stdint.h>

#include "ffa_c_api.h"
#include "ffa_host.h"

using namespace ffa;

namespace {

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

int validate_decode(const DecodeArgs& a) {
    if (elem_bytes(a.precision) == 0) return FFA_ERR_DTYPE;
    if (a.Dh != 64 && a.Dh != 80 && a.Dh != 128 && a.Dh != 256) return FFA_ERR_HEAD_DIM;
    if (a.B <= 0 || a.H <= 0 || a.Lmax <= 0) return FFA_ERR_SHAPE;
    if ((long long)a.B * a.H > (1ll << 24)) return FFA_ERR_SHAPE;
    if (a.t < 0 || a.t >= a.Lmax) return FFA_ERR_TIMESTEP;
    if (!(a.p >= 0.f) || isinf(a.p)) return FFA_ERR_PROB_THRESH;
    if (!a.q || !a.k || !a.v || !a.k_cache || !a.v_cache || !a.out) return FFA_ERR_NULL_POINTER;
    if (!aligned16(a.q) || !aligned16(a.k) || !aligned16(a.v) || !aligned16(a.k_cache) ||
        !aligned16(a.v_cache) || !aligned16(a.out))
        return FFA_ERR_ALIGNMENT;
    if (a.rotary_dim < 0 || a.rotary_dim > a.Dh || (a.rotary_dim & 1)) return FFA_ERR_TRANSFORM;
    if (!aligned16(a.q_bias) || !aligned16(a.k_bias) || !aligned16(a.v_bias)) return FFA_ERR_TRANSFORM;
    if (a.cache_indir != nullptr) {
        if ((reinterpret_cast<uintptr_t>(a.cache_indir) & 3u) != 0) return FFA_ERR_BEAM;
        if (a.beam_width < 1 || a.B % a.beam_width != 0) return FFA_ERR_BEAM;
        // Rows of a group are numbered beam * H * Lmax + key in 32 bits.
        if ((long long)a.beam_width * a.H * a.Lmax >= (1ll << 31)) return FFA_ERR_BEAM;
    }
    return FFA_OK;
}

int run_decode(const DecodeArgs& args, const ffa_launch_plan* user_plan, void* workspace,
               size_t workspace_bytes) {
    const DecodeArgs& a = args;
    int st = validate_decode(a);
    if (st != FFA_OK) return st;
    const int plan_prec = planner_precision(a.precision);
    const bool diag = a.kept_count != nullptr || a.skip_mask != nullptr;

    ffa_launch_plan plan;
    if (user_plan != nullptr) {
        plan = *user_plan;
    } else {
        // Diagnostics do not exist in the exact split kernel: plan as for a pruned step.
        const int cus = query_compute_units();
        st = plan_launch(plan_prec, a.B, a.H, a.Dh, a.t, a.p, /*use_default=*/0, cus, &plan);
        if (st == FFA_OK && diag && plan.kind == FFA_LAUNCH_SPLIT)
            st = plan_launch(plan_prec, a.B, a.H, a.Dh, a.t, 1.f, 0, cus, &plan);
        if (st != FFA_OK) return st;
    }
    st = validate_plan(plan, plan_prec, a.Dh, a.B * a.H, a.t, a.p);
    if (st != FFA_OK) return st;
    if (diag && plan.kind == FFA_LAUNCH_SPLIT) return FFA_ERR_PLAN;

    // Workspace layout: [arrival counters][what the plan needs].  The counters are the only
    // words that persist from call to call; nothing else is ever placed on them.
    WorkspaceView ws = {nullptr, nullptr, nullptr, nullptr, 0};
    const int bh = a.B * a.H;
    const size_t need = plan_workspace_bytes(plan, bh, a.Dh, a.Lmax);
    if (need > 0) {
        if (workspace == nullptr || workspace_bytes < need) return FFA_ERR_WORKSPACE;
        if (!aligned16(workspace)) return FFA_ERR_ALIGNMENT;
        char* base = static_cast<char*>(workspace);
        ws.cnt = reinterpret_cast<unsigned int*>(base);
        base += workspace_counter_bytes(bh);
        if (plan.kind == FFA_LAUNCH_TWO_PASS) {
            // [piece (max, sum)][partial outputs][scores]
            ws.ml = reinterpret_cast<float*>(base);
            base += align_up((size_t)bh * plan.n_splits * 2 * sizeof(float), 256);
            ws.acc = reinterpret_cast<float*>(base);
            base += align_up((size_t)bh * plan.n_splits * a.Dh * sizeof(float), 256);
            ws.scores = reinterpret_cast<float*>(base);
            ws.score_stride = score_stride_for(a.Lmax);
        } else {
            ws.acc = reinterpret_cast<float*>(base);  // slots: accumulator, (max, sum), padding
        }
    }
    return launch_decode(a, plan, ws);
}

// Optional parts of a decode call: token transform and beam indirection.
int apply_options(DecodeArgs& a, const ffa_token_transform* transform, const ffa_beam_indirection* beams) {
    if (transform != nullptr) {
        a.q_bias = transform->q_bias; a.k_bias = transform->k_bias; a.v_bias = transform->v_bias;
        a.rotary_dim = transform->rotary_embedding_dim;
        a.rotary_base = transform->rotary_base > 0.f ? transform->rotary_base : 10000.f;
    }
    if (beams != nullptr) {
        if (beams->cache_indir == nullptr) return FFA_ERR_BEAM;
        a.cache_indir = beams->cache_indir;
        a.beam_width = beams->beam_width;
    }
    return FFA_OK;
}

int run_init_cache(int precision, void* k_dst, void* v_dst, const void* k_src, const void* v_src,
                   int B, int L, int Lmax, int Dh, int H, void* stream) {
    if (Dh != 64 && Dh != 80 && Dh != 128 && Dh != 256) return FFA_ERR_HEAD_DIM;
    if (B <= 0 || H <= 0 || L < 0 || Lmax <= 0 || L > Lmax) return FFA_ERR_SHAPE;
    if (!k_dst || !v_dst) return FFA_ERR_NULL_POINTER;
    if (L == 0) return FFA_OK;
    if (!k_src || !v_src) return FFA_ERR_NULL_POINTER;
    if (!aligned16(k_dst) || !aligned16(v_dst) || !aligned16(k_src) || !aligned16(v_src))
        return FFA_ERR_ALIGNMENT;
    return launch_init_cache(precision, k_dst, v_dst, k_src, v_src, B, H, L, Lmax, Dh, stream);
}

}  // namespace

extern "C" {

int ffa_api_version(void) { return FFA_API_VERSION; }

const char* ffa_status_string(int status) {
    switch (status) {
        case FFA_OK: return "ok";
        case FFA_ERR_NULL_POINTER: return "a required pointer is NULL";
        case FFA_ERR_DTYPE: return "unsupported precision (expected 16 or 32)";
        case FFA_ERR_HEAD_DIM: return "unsupported head dimension (expected 64, 80, 128 or 256)";
        case FFA_ERR_SHAPE: return "invalid batch, head or sequence size";
        case FFA_ERR_TIMESTEP: return "timestep outside [0, max_seq_len)";
        case FFA_ERR_ALIGNMENT: return "pointer is not 16-byte aligned";
        case FFA_ERR_WORKSPACE: return "workspace missing or too small for the launch plan";
        case FFA_ERR_PLAN: return "malformed launch plan";
        case FFA_ERR_TOO_LONG: return "sequence too long for a one-workgroup launch";
        case FFA_ERR_PROB_THRESH: return "prob_thresh must be a finite number >= 0";
        case FFA_ERR_LAUNCH: return "HIP kernel launch failed";
        case FFA_ERR_NO_DEVICE: return "no usable HIP device";
        case FFA_ERR_BEAM: return "bad beam indirection: table NULL or not 4-byte aligned, beam_width < 1 or not a divisor of batch_size, or beam_width * head_num * max_seq_len >= 2^31";
        case FFA_ERR_TRANSFORM: return "bad token transform: rotary dimension must be even and within [0, head_dim], biases 16-byte aligned";
        case FFA_ERR_SCRATCH_LIMIT: return "the launch plan needs more scratch than the library's static 4 MiB array holds";
        default: return "unknown status";
    }
}

int ffa_device_compute_units(void) { return query_compute_units(); }

static int plan_entry(int precision, int batch_size, int head_num, int head_dim, int t, float prob_thresh,
                      int use_default_kernel_launch, int compute_units, int use_table, ffa_launch_plan* plan) {
    if (compute_units <= 0 && !use_default_kernel_launch) {
        compute_units = query_compute_units();
        if (compute_units <= 0) return FFA_ERR_NO_DEVICE;
    }
    return plan_launch_ex(planner_precision(precision), batch_size, head_num, head_dim, t, prob_thresh,
                          use_default_kernel_launch, compute_units, use_table, plan);
}

int ffa_plan_launch(int precision, int batch_size, int head_num, int head_dim, int t,
                    float prob_thresh, int use_default_kernel_launch, int compute_units,
                    ffa_launch_plan* plan) {
    return plan_entry(precision, batch_size, head_num, head_dim, t, prob_thresh,
                      use_default_kernel_launch, compute_units, /*use_table=*/1, plan);
}

int ffa_plan_launch_rules(int precision, int batch_size, int head_num, int head_dim, int t,
                          float prob_thresh, int use_default_kernel_launch, int compute_units,
                          ffa_launch_plan* plan) {
    return plan_entry(precision, batch_size, head_num, head_dim, t, prob_thresh,
                      use_default_kernel_launch, compute_units, /*use_table=*/0, plan);
}

int ffa_plan_source(int precision, int batch_size, int head_num, int head_dim, int t, float prob_thresh,
                    int compute_units) {
    ffa_launch_plan plan;
    const int st = plan_entry(precision, batch_size, head_num, head_dim, t, prob_thresh, 0, compute_units, 1, &plan);
    if (st != FFA_OK) return -st;
    if (compute_units <= 0) compute_units = query_compute_units();
    return plan_source(planner_precision(precision), batch_size, head_num, head_dim, t, prob_thresh, compute_units);
}

size_t ffa_workspace_bytes(int batch_size, int head_num, int head_dim, int max_seq_len) {
    if (batch_size <= 0 || head_num <= 0 || head_dim <= 0 || max_seq_len <= 0) return 0;
    const int bh = batch_size * head_num;
    const int n_splits = max_splits_for(bh, max_seq_len);
    const size_t exact = workspace_bytes_for(bh, bh, head_dim, n_splits);
    const size_t two_pass = two_pass_workspace_bytes(bh, head_dim, n_splits, max_seq_len);
    return align_up(exact > two_pass ? exact : two_pass, 256);
}

int ffa_workspace_init(void* workspace, size_t workspace_bytes, void* stream) {
    if (workspace == nullptr) return FFA_ERR_NULL_POINTER;
    if (!aligned16(workspace)) return FFA_ERR_ALIGNMENT;
    // Only the arrival counters at the head of the workspace have to start at zero, but how many
    // there are depends on the problem (4 bytes per (batch, head) pair), which this call does not
    // know, and a caller may hand over a buffer sized for one plan rather than
    // ffa_workspace_bytes().  The call is made once per workspace: clear all of it.
    const size_t bytes = workspace_bytes & ~(size_t)3;
    return launch_fill_u32(static_cast<unsigned int*>(workspace), bytes / 4, 0u, stream);
}

int ffa_init_cache_f16(uint16_t* k_dst, uint16_t* v_dst, const uint16_t* k_src,
                       const uint16_t* v_src, int batch_size, int seq_len, int max_seq_len,
                       int head_dim, int head_num, void* stream) {
    return run_init_cache(FFA_PRECISION_F16, k_dst, v_dst, k_src, v_src, batch_size, seq_len,
                          max_seq_len, head_dim, head_num, stream);
}

int ffa_init_cache_f32(float* k_dst, float* v_dst, const float* k_src, const float* v_src,
                       int batch_size, int seq_len, int max_seq_len, int head_dim, int head_num,
                       void* stream) {
    return run_init_cache(FFA_PRECISION_F32, k_dst, v_dst, k_src, v_src, batch_size, seq_len,
                          max_seq_len, head_dim, head_num, stream);
}

int ffa_attention_diag(int precision, int batch_size, int head_num, int head_dim, int max_seq_len,
                       float softmax_scale, int t, const void* q, const void* k, const void* v,
                       void* k_cache, void* v_cache, void* out, const int* seq_lengths,
                       float prob_thresh, const ffa_launch_plan* plan, int right_or_no_padding,
                       void* workspace, size_t workspace_bytes, uint32_t* kept_count,
                       uint8_t* skip_mask, void* stream) {
    DecodeArgs a;
    a.precision = precision;
    a.B = batch_size; a.H = head_num; a.Dh = head_dim; a.Lmax = max_seq_len; a.t = t;
    a.scale = softmax_scale; a.p = prob_thresh;
    a.q = q; a.k = k; a.v = v;
    a.k_cache = k_cache; a.v_cache = v_cache; a.out = out;
    a.seq_lengths = seq_lengths;
    a.right_or_no_padding = right_or_no_padding;
    a.kept_count = kept_count; a.skip_mask = skip_mask;
    a.stream = stream;
    return run_decode(a, plan, workspace, workspace_bytes);
}

int ffa_attention_ex(int precision, int batch_size, int head_num, int head_dim, int max_seq_len,
                     float softmax_scale, int t, const void* q, const void* k, const void* v,
                     void* k_cache, void* v_cache, void* out, const int* seq_lengths,
                     float prob_thresh, const ffa_launch_plan* plan, int right_or_no_padding,
                     const ffa_token_transform* transform, const ffa_beam_indirection* beams,
                     void* workspace, size_t workspace_bytes, void* stream) {
    DecodeArgs a;
    a.precision = precision;
    a.B = batch_size; a.H = head_num; a.Dh = head_dim; a.Lmax = max_seq_len; a.t = t;
    a.scale = softmax_scale; a.p = prob_thresh;
    a.q = q; a.k = k; a.v = v;
    a.k_cache = k_cache; a.v_cache = v_cache; a.out = out;
    a.seq_lengths = seq_lengths;
    a.right_or_no_padding = right_or_no_padding;
    a.kept_count = nullptr; a.skip_mask = nullptr;
    a.stream = stream;
    const int st = apply_options(a, transform, beams);
    if (st != FFA_OK) return st;
    return run_decode(a, plan, workspace, workspace_bytes);
}

int ffa_load_floor(int precision, int batch_size, int head_num, int head_dim, int max_seq_len, int t,
                   const void* k_cache, const void* v_cache, const int* seq_lengths, int right_or_no_padding,
                   const ffa_launch_plan* plan, void* sink, void* stream) {
    if (plan == nullptr || sink == nullptr) return FFA_ERR_NULL_POINTER;
    if (plan->kind != FFA_LAUNCH_SPLIT || plan->threads_per_key != 1 ||
        (plan->waves_per_wg != 2 && plan->waves_per_wg != 4 && plan->waves_per_wg != 8))
        return FFA_ERR_PLAN;
    DecodeArgs a;
    a.precision = precision;
    a.B = batch_size; a.H = head_num; a.Dh = head_dim; a.Lmax = max_seq_len; a.t = t;
    a.scale = 1.f; a.p = 0.f;
    // The probe reads the caches only; q, k, v stand in as non-null, aligned addresses that it never touches.
    a.q = a.k = a.v = sink;
    a.k_cache = const_cast<void*>(k_cache); a.v_cache = const_cast<void*>(v_cache); a.out = sink;
    a.seq_lengths = seq_lengths;
    a.right_or_no_padding = right_or_no_padding;
    a.kept_count = nullptr; a.skip_mask = nullptr;
    a.stream = stream;
    a.floor_probe = true;
    int st = validate_decode(a);
    if (st != FFA_OK) return st;
    st = validate_plan(*plan, planner_precision(precision), head_dim, batch_size * head_num, t, 0.f);
    if (st != FFA_OK) return st;
    const WorkspaceView none = {nullptr, nullptr, nullptr, nullptr, 0};
    return launch_decode(a, *plan, none);
}

int ffa_attention_static_scratch(int precision, int batch_size, int head_num, int head_dim,
                                  int max_seq_len, float softmax_scale, int t, const void* q,
                                  const void* k, const void* v, void* k_cache, void* v_cache,
                                  void* out, const int* seq_lengths, float prob_thresh,
                                  const ffa_launch_plan* plan, int right_or_no_padding,
                                  const ffa_token_transform* transform,
                                  const ffa_beam_indirection* beams, void* stream) {
    DecodeArgs a;
    a.precision = precision;
    a.B = batch_size; a.H = head_num; a.Dh = head_dim; a.Lmax = max_seq_len; a.t = t;
    a.scale = softmax_scale; a.p = prob_thresh;
    a.q = q; a.k = k; a.v = v;
    a.k_cache = k_cache; a.v_cache = v_cache; a.out = out;
    a.seq_lengths = seq_lengths;
    a.right_or_no_padding = right_or_no_padding;
    a.kept_count = nullptr; a.skip_mask = nullptr;
    a.stream = stream;
    int st = apply_options(a, transform, beams);
    if (st != FFA_OK) return st;
    st = validate_decode(a);
    if (st != FFA_OK) return st;
    ffa_launch_plan chosen;
    if (plan != nullptr) {
        chosen = *plan;
    } else {
        st = plan_launch(planner_precision(precision), a.B, a.H, a.Dh, a.t, a.p, /*use_default=*/0,
                         query_compute_units(), &chosen);
        if (st != FFA_OK) return st;
    }
    st = validate_plan(chosen, planner_precision(precision), a.Dh, a.B * a.H, a.t, a.p);
    if (st != FFA_OK) return st;
    const size_t need = plan_workspace_bytes(chosen, a.B * a.H, a.Dh, a.Lmax);
    if (need > kStaticScratchBytes) return FFA_ERR_SCRATCH_LIMIT;
    void* scratch_ptr = nullptr;
    if (need > 0) {
        st = static_scratch_address(&scratch_ptr);
        if (st != FFA_OK) return st;
        // The array keeps whatever the previous call on this GPU left behind: the arrival
        // counters of this call's pairs are cleared first (a small kernel, not a memset node,
        // so the call may be recorded into a HIP graph).
        st = launch_fill_u32(static_cast<unsigned int*>(scratch_ptr), (size_t)a.B * a.H * kCounterStride, 0u, stream);
        if (st != FFA_OK) return st;
    }
    return run_decode(a, &chosen, scratch_ptr, need > 0 ? kStaticScratchBytes : 0);
}

int ffa_attention_f16(int batch_size, int head_num, int head_dim, int max_seq_len,
                      float softmax_scale, int t, const uint16_t* q, const uint16_t* k,
                      const uint16_t* v, uint16_t* k_cache, uint16_t* v_cache, uint16_t* out,
                      const int* seq_lengths, float prob_thresh, const ffa_launch_plan* plan,
                      int right_or_no_padding, void* workspace, size_t workspace_bytes,
                      void* stream) {
    return ffa_attention_diag(FFA_PRECISION_F16, batch_size, head_num, head_dim, max_seq_len,
                              softmax_scale, t, q, k, v, k_cache, v_cache, out, seq_lengths,
                              prob_thresh, plan, right_or_no_padding, workspace, workspace_bytes,
                              nullptr, nullptr, stream);
}

int ffa_attention_f32(int batch_size, int head_num, int head_dim, int max_seq_len,
                      float softmax_scale, int t, const float* q, const float* k, const float* v,
                      float* k_cache, float* v_cache, float* out, const int* seq_lengths,
                      float prob_thresh, const ffa_launch_plan* plan, int right_or_no_padding,
                      void* workspace, size_t workspace_bytes, void* stream) {
    return ffa_attention_diag(FFA_PRECISION_F32, batch_size, head_num, head_dim, max_seq_len,
                              softmax_scale, t, q, k, v, k_cache, v_cache, out, seq_lengths,
                              prob_thresh, plan, right_or_no_padding, workspace, workspace_bytes,
                              nullptr, nullptr, stream);
}

}  // extern "C"
