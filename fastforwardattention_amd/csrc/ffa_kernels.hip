// gfx950 (MI355X, wave64) kernels and launchers that do not depend on the element type of the
// decode step: cache construction, the fill kernel, per-device state, and the entry that turns
// validated arguments into kernel parameters.  The decode kernels themselves are templates in
// ffa_decode_kernels.h, instantiated per element type in ffa_decode_{f16,bf16,f32}.hip.
#include <hip/hip_runtime.h>
#include <math.h>
#include <stdint.h>

#include <mutex>

#include "ffa_c_api.h"
#include "ffa_device.h"
#include "ffa_host.h"

namespace ffa {

// Scratch of the entry point that takes no workspace (ffa_attention_static_scratch): arrival
// counters, split partials and two-pass scores live here instead of in caller-owned memory.
// Every GPU the library runs on holds its own copy at its own address; host code never uses
// this name as an address, only what hipGetSymbolAddress returned for the current device
// (static_scratch_address below).
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

// ---------------------------------------------------------------------------------------
// Cache construction (attention.cu:1556-1609).  One workgroup moves a tile of TK keys of
// one (b,h), TK*NCH 16-byte chunks each of K and V: coalesced row reads [TK keys x Dh] -> LDS
// -> coalesced chunk-row writes (TK x 16 B contiguous) for K; V is a straight copy.  All
// loads of a thread are issued before anything is stored (indices past the end are clamped,
// so no load sits under a branch).
template <int NCH, int TK>
__global__ void __launch_bounds__(256) ffa_init_cache_kernel(uint4* __restrict__ k_dst,
                                                             uint4* __restrict__ v_dst,
                                                             const uint4* __restrict__ k_src,
                                                             const uint4* __restrict__ v_src,
                                                             int L, int Lmax, int tiles) {
    constexpr int PER = (TK * NCH + 255) / 256;  // chunks per thread, of K and of V
    __shared__ uint4 s_tile[NCH * (TK + 1)];  // [chunk][key], one chunk of padding per row
    // One-dimensional grid, the tiles of a (b,h) pair adjacent: no 65535 limit on B*H.
    const int bh = blockIdx.x / tiles;
    const int l0 = (blockIdx.x % tiles) * TK;
    const int n = min(TK, L - l0) * NCH;  // chunks of this tile, >= NCH
    const uint4* ks = k_src + ((size_t)bh * L + l0) * NCH;
    const uint4* vs = v_src + ((size_t)bh * L + l0) * NCH;
    uint4* kd = k_dst + (size_t)bh * Lmax * NCH + l0;
    uint4* vd = v_dst + ((size_t)bh * Lmax + l0) * NCH;
    uint4 kv[PER], vv[PER];
#pragma unroll
    for (int j = 0; j < PER; ++j) {
        const int i = min((int)threadIdx.x + j * 256, n - 1);
        kv[j] = ld16(&ks[i]);
        vv[j] = ld16(&vs[i]);
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int j = 0; j < PER; ++j) {
        const int i = threadIdx.x + j * 256;
        if (i < n) st16_stream(&vd[i], vv[j]);                               // V: contiguous copy
        if (i < TK * NCH) s_tile[(i % NCH) * (TK + 1) + i / NCH] = kv[j];   // K: [key][chunk] -> [chunk][key]
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < PER; ++j) {
        const int i = threadIdx.x + j * 256;
        const int c = i / TK, key = i % TK;
        if (c < NCH && key * NCH < n) st16_stream(&kd[(size_t)c * Lmax + key], s_tile[c * (TK + 1) + key]);
    }
}

__global__ void ffa_fill_u32_kernel(unsigned int* p, size_t n, unsigned int v) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = v;
}

// ---------------------------------------------------------------------------------------
// Host side.
static int check_launch() {
    return hipGetLastError() == hipSuccess ? FFA_OK : FFA_ERR_LAUNCH;
}

// Per-device facts, resolved once per device under a lock (several host threads may drive
// several GPUs of one process).
struct DeviceState {
    int compute_units = 0;
    void* scratch = nullptr;
};
static std::mutex g_dev_mutex;
static DeviceState g_dev[kMaxDevices];

int current_device() {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) { (void)hipGetLastError(); return -1; }
    return (dev >= 0 && dev < kMaxDevices) ? dev : -1;
}

int static_scratch_address(void** ptr) {
    const int dev = current_device();
    if (dev < 0 || ptr == nullptr) return FFA_ERR_NO_DEVICE;
    std::lock_guard<std::mutex> lock(g_dev_mutex);
    if (g_dev[dev].scratch == nullptr) {
        void* p = nullptr;
        if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || p == nullptr) {
            (void)hipGetLastError();
            return FFA_ERR_NO_DEVICE;
        }
        g_dev[dev].scratch = p;
    }
    *ptr = g_dev[dev].scratch;
    return FFA_OK;
}

int launch_decode(const DecodeArgs& a, const ffa_launch_plan& plan, const WorkspaceView& ws) {
    DecodeParams P;
    P.q = a.q; P.k = a.k; P.v = a.v;
    P.k_cache = a.k_cache; P.v_cache = a.v_cache; P.out = a.out;
    P.seq_lengths = a.seq_lengths;
    P.ws_acc = ws.acc; P.ws_ml = ws.ml; P.ws_cnt = ws.cnt;
    P.ws_scores = ws.scores; P.score_stride = ws.score_stride;
    P.kept_count = a.kept_count; P.skip_mask = a.skip_mask;
    P.B = a.B; P.H = a.H; P.Lmax = a.Lmax; P.t = a.t;
    P.scale_log2e = a.scale * kLog2e;
    P.p = a.p;
    P.right_or_no_padding = a.right_or_no_padding;
    P.n_splits = plan.n_splits; P.tiles_per_split = plan.tiles_per_split;
    P.split_magic = plan.n_splits > 1 ? (unsigned)(0x100000000ull / (unsigned)plan.n_splits) + 1u : 0u;
    P.bh_total = a.B * a.H;
    // Pieces of an unsplit pair are whole pairs.
    P.n_whole = plan.kind == FFA_LAUNCH_SPLIT ? (plan.n_splits > 1 ? plan.whole_heads : P.bh_total) : 0;
    P.combine = plan.combine;
    P.cache_indir = a.cache_indir;
    P.beam_width = a.cache_indir != nullptr ? a.beam_width : 1;
    P.q_bias = a.q_bias; P.k_bias = a.k_bias; P.v_bias = a.v_bias;
    P.rotary_dim = a.rotary_dim;
    P.xform = a.transforms_token() ? 1 : 0;
    P.floor_probe = a.floor_probe ? 1 : 0;
    P.store_through = (plan.kind == FFA_LAUNCH_SPLIT && plan.n_splits > 1 && plan.whole_heads == 0) ? 1 : 0;
    P.rotary_coef = a.rotary_dim > 0 ? -2.0 * log2((double)a.rotary_base) / (double)a.rotary_dim : 0.0;
    // The transform is a compile-time switch of the kernels: the plain step carries none of its code.
    if (P.xform) {
        if (a.precision == FFA_PRECISION_F16) return launch_decode_f16_xform(P, a.Dh, plan, a.stream);
        if (a.precision == FFA_PRECISION_BF16) return launch_decode_bf16_xform(P, a.Dh, plan, a.stream);
        return launch_decode_f32_xform(P, a.Dh, plan, a.stream);
    }
    if (a.precision == FFA_PRECISION_F16) return launch_decode_f16(P, a.Dh, plan, a.stream);
    if (a.precision == FFA_PRECISION_BF16) return launch_decode_bf16(P, a.Dh, plan, a.stream);
    return launch_decode_f32(P, a.Dh, plan, a.stream);
}

int launch_init_cache(int precision, void* k_dst, void* v_dst, const void* k_src,
                      const void* v_src, int B, int H, int L, int Lmax, int Dh, void* stream) {
    const int nch = Dh * (precision / 8) / 16;
    if (nch != 8 && nch != 10 && nch != 16 && nch != 20 && nch != 32 && nch != 64) return FFA_ERR_HEAD_DIM;
    if (L <= 0) return FFA_OK;
    // 512 chunks (8 KiB of K, 8 KiB of V) per workgroup: measured against 1024 / 2048 / 4096,
    // the small tile wins at every shape -- many resident workgroups hide the latency better
    // than more loads per thread do.
    constexpr int kIc = 512;
    const int tk = nch == 10 ? 64 : nch == 20 ? 32 : kIc / nch;  // Dh = 80: 640 chunks
    const int tiles = (L + tk - 1) / tk;
    if ((long long)tiles * B * H > 0x7fffffffll) return FFA_ERR_SHAPE;
    const dim3 grid((unsigned)(tiles * B * H));
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    auto kd = reinterpret_cast<uint4*>(k_dst);
    auto vd = reinterpret_cast<uint4*>(v_dst);
    auto ks = reinterpret_cast<const uint4*>(k_src);
    auto vs = reinterpret_cast<const uint4*>(v_src);
    switch (nch) {
        case 8: hipLaunchKernelGGL((ffa_init_cache_kernel<8, kIc / 8>), grid, dim3(256), 0, st, kd, vd, ks, vs, L, Lmax, tiles); break;
        case 16: hipLaunchKernelGGL((ffa_init_cache_kernel<16, kIc / 16>), grid, dim3(256), 0, st, kd, vd, ks, vs, L, Lmax, tiles); break;
        case 32: hipLaunchKernelGGL((ffa_init_cache_kernel<32, kIc / 32>), grid, dim3(256), 0, st, kd, vd, ks, vs, L, Lmax, tiles); break;
        case 64: hipLaunchKernelGGL((ffa_init_cache_kernel<64, kIc / 64>), grid, dim3(256), 0, st, kd, vd, ks, vs, L, Lmax, tiles); break;
        case 10: hipLaunchKernelGGL((ffa_init_cache_kernel<10, 64>), grid, dim3(256), 0, st, kd, vd, ks, vs, L, Lmax, tiles); break;
        case 20: hipLaunchKernelGGL((ffa_init_cache_kernel<20, 32>), grid, dim3(256), 0, st, kd, vd, ks, vs, L, Lmax, tiles); break;
        default: return FFA_ERR_HEAD_DIM;
    }
    return check_launch();
}

int launch_fill_u32(unsigned int* p, size_t n, unsigned int v, void* stream) {
    if (n == 0) return FFA_OK;
    const unsigned blocks = (unsigned)((n + 255) / 256);
    hipLaunchKernelGGL(ffa_fill_u32_kernel, dim3(blocks), dim3(256), 0,
                       reinterpret_cast<hipStream_t>(stream), p, n, v);
    return check_launch();
}

int query_compute_units() {
    const int dev = current_device();
    if (dev < 0) return -1;
    std::lock_guard<std::mutex> lock(g_dev_mutex);
    if (g_dev[dev].compute_units > 0) return g_dev[dev].compute_units;
    int cus = 0;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) {
        (void)hipGetLastError();
        return -1;
    }
    g_dev[dev].compute_units = cus;
    return cus;
}

}  // namespace ffa
