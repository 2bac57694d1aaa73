// PyTorch-ROCm extension `ff_attention`: the Python-visible class FastForwardAttn with the
// constructor, get_cache() and the three positional attention(...) overloads of the
// reference extension (torch_ffa_api.cpp:161-214), implemented on the C ABI of
// include/ffa_c_api.h.  torch is used for device memory and the current stream only.
//
// Differences from the reference, all on the side of refusing bad input:
//   - arguments are checked (device, dtype, element count, t < max_len) and C-ABI status
//     codes become Python exceptions; the reference prints and continues
//     (torch_ffa_api.cpp:101, :129, :154; attention.cu:1444-1451);
//   - kernels run on torch's current HIP stream instead of the legacy default stream
//     (attention.cu:1504);
//   - the launch plan is recomputed from t at every call instead of once from the prompt
//     length (torch_ffa_api.cpp:176).
#include <torch/extension.h>

// PyTorch-ROCm presents HIP devices under the device type "cuda"; these are the guard and
// stream accessors that understand that.
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>

#include <tuple>
#include <utility>

#include "ffa_c_api.h"

namespace {

void check_status(int st, const char* what) {
    TORCH_CHECK(st == FFA_OK, "ff_attention: ", what, " failed: ", ffa_status_string(st),
                " (status ", st, ")");
}

int precision_of(const torch::Tensor& x) {
    if (x.scalar_type() == torch::kHalf) return FFA_PRECISION_F16;
    if (x.scalar_type() == torch::kFloat) return FFA_PRECISION_F32;
    if (x.scalar_type() == torch::kBFloat16) return FFA_PRECISION_BF16;
    TORCH_CHECK(false, "ff_attention: unsupported tensor type ", x.scalar_type(),
                " (float16, bfloat16 and float32 are supported)");
}

// The planner knows two element sizes: bf16 plans like fp16.
int plan_precision(int precision) { return precision == FFA_PRECISION_BF16 ? FFA_PRECISION_F16 : precision; }

void* stream_of(const torch::Tensor& x) {
    return static_cast<void*>(c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(x.device().index()).stream());
}

struct CacheDims {
    int B, H, Lmax, Dh;
};

// Every dimension is recovered from the K cache's 5-D shape, as the reference does
// (torch_ffa_api.cpp:112-115, :137-140).
CacheDims dims_of(const torch::Tensor& k_cache, const torch::Tensor& v_cache) {
    TORCH_CHECK(k_cache.dim() == 5, "ff_attention: k_cache must be [B,H,Dh/x,Lmax,x]");
    TORCH_CHECK(v_cache.dim() == 4, "ff_attention: v_cache must be [B,H,Lmax,Dh]");
    CacheDims d;
    d.B = (int)k_cache.size(0);
    d.H = (int)k_cache.size(1);
    d.Lmax = (int)k_cache.size(3);
    d.Dh = (int)(k_cache.size(2) * k_cache.size(4));
    TORCH_CHECK(k_cache.size(4) * k_cache.element_size() == 16,
                "ff_attention: last k_cache dimension must span 16 bytes");
    TORCH_CHECK(v_cache.size(0) == d.B && v_cache.size(1) == d.H && v_cache.size(2) == d.Lmax &&
                    v_cache.size(3) == d.Dh,
                "ff_attention: k_cache and v_cache shapes disagree");
    TORCH_CHECK(k_cache.is_contiguous() && v_cache.is_contiguous(),
                "ff_attention: caches must be contiguous");
    return d;
}

torch::Tensor token_input(const torch::Tensor& x, const torch::Tensor& like, int64_t numel,
                          const char* name) {
    TORCH_CHECK(x.device() == like.device(), "ff_attention: ", name, " is on ", x.device(),
                " but the cache is on ", like.device());
    TORCH_CHECK(x.scalar_type() == like.scalar_type(), "ff_attention: ", name,
                " dtype differs from the cache dtype");
    TORCH_CHECK(x.numel() == numel, "ff_attention: ", name, " must hold B*H*Dh = ", numel,
                " elements, got ", x.numel());
    return x.contiguous();  // storage order [B,H,Dh]; no copy when already contiguous
}

}  // namespace

struct FastForwardAttn {
    FastForwardAttn(torch::Tensor K, torch::Tensor V, int max_timesteps, bool _ft_kernel_launch) {
        TORCH_CHECK(K.is_cuda() && V.is_cuda(), "ff_attention: K and V must be GPU tensors");
        TORCH_CHECK(K.dim() == 4 && V.sizes() == K.sizes(),
                    "ff_attention: K and V must both be [B,H,L,Dh]");
        TORCH_CHECK(K.scalar_type() == V.scalar_type() && K.device() == V.device(),
                    "ff_attention: K and V must share dtype and device");
        const int precision = precision_of(K);
        const int B = (int)K.size(0), H = (int)K.size(1), L = (int)K.size(2), Dh = (int)K.size(3);
        TORCH_CHECK(max_timesteps >= L && max_timesteps > 0,
                    "ff_attention: max_timesteps (", max_timesteps, ") < prompt length (", L, ")");
        const int x = 16 / (int)K.element_size();
        TORCH_CHECK(Dh % x == 0, "ff_attention: head dim must be a multiple of ", x);

        c10::hip::HIPGuardMasqueradingAsCUDA guard(K.device());
        K = K.contiguous();
        V = V.contiguous();
        k_cache = torch::empty({B, H, Dh / x, max_timesteps, x}, K.options());
        v_cache = torch::empty({B, H, max_timesteps, Dh}, K.options());
        void* st = stream_of(K);
        int rc;
        if (precision != FFA_PRECISION_F32)  // fp16 and bf16 alike: cache construction moves 16-byte chunks
            rc = ffa_init_cache_f16((uint16_t*)k_cache.data_ptr(), (uint16_t*)v_cache.data_ptr(),
                                    (const uint16_t*)K.data_ptr(), (const uint16_t*)V.data_ptr(), B, L,
                                    max_timesteps, Dh, H, st);
        else
            rc = ffa_init_cache_f32((float*)k_cache.data_ptr(), (float*)v_cache.data_ptr(),
                                    (const float*)K.data_ptr(), (const float*)V.data_ptr(), B, L,
                                    max_timesteps, Dh, H, st);
        check_status(rc, "cache construction");
        ft_kernel_launch = _ft_kernel_launch;
        ensure_workspace(B, H, Dh, max_timesteps, K.device());
    }

    // attention(q, k, v, k_cache, v_cache, softmax_scale, t, p)      torch_ffa_api.cpp:179-182
    torch::Tensor attention(torch::Tensor q, torch::Tensor k, torch::Tensor v, torch::Tensor k_cache,
                            torch::Tensor v_cache, float softmax_scale, int curr_timestep,
                            float prob_thresh = 0) {
        return run(q, k, v, k_cache, v_cache, softmax_scale, curr_timestep, nullptr, prob_thresh, true,
                   nullptr, nullptr);
    }

    // attention(q, k, v, k_cache, v_cache, softmax_scale, t, seq_lengths, p): left-padded
    // batch, seq_lengths[b] = first real key (torch_ffa_api.cpp:184-187, :122).
    torch::Tensor attention(torch::Tensor q, torch::Tensor k, torch::Tensor v, torch::Tensor k_cache,
                            torch::Tensor v_cache, float softmax_scale, int curr_timestep,
                            torch::Tensor seq_lengths, float prob_thresh = 0) {
        return run(q, k, v, k_cache, v_cache, softmax_scale, curr_timestep, &seq_lengths, prob_thresh,
                   false, nullptr, nullptr);
    }

    // attention(q, k, v, softmax_scale, t, p)                         torch_ffa_api.cpp:189-192
    torch::Tensor attention(torch::Tensor q, torch::Tensor k, torch::Tensor v, float softmax_scale,
                            int curr_timestep, float prob_thresh = 0) {
        return run(q, k, v, k_cache, v_cache, softmax_scale, curr_timestep, nullptr, prob_thresh, true,
                   nullptr, nullptr);
    }

    std::pair<torch::Tensor, torch::Tensor> get_cache() { return std::make_pair(k_cache, v_cache); }

    // Not in the reference's Python surface: the step with the FasterTransformer features its host
    // code switches off (attention.cu:1472-1483) -- q/k/v bias [H,Dh] and the rotary embedding of
    // q and k over the first rotary_dim elements (GPT-J's pairing), applied to the new token
    // before it is attended and appended.  seq_lengths = None, or int32 [B] first real keys of
    // a left-padded batch; biases may be None.
    torch::Tensor attention_ex(torch::Tensor q, torch::Tensor k, torch::Tensor v, torch::Tensor k_cache,
                               torch::Tensor v_cache, float softmax_scale, int curr_timestep,
                               c10::optional<torch::Tensor> seq_lengths, float prob_thresh, int rotary_dim,
                               c10::optional<torch::Tensor> q_bias, c10::optional<torch::Tensor> k_bias,
                               c10::optional<torch::Tensor> v_bias, c10::optional<torch::Tensor> cache_indir,
                               int beam_width) {
        const CacheDims d = dims_of(k_cache, v_cache);
        torch::Tensor bias[3];
        const c10::optional<torch::Tensor>* in[3] = {&q_bias, &k_bias, &v_bias};
        ffa_token_transform tt = {nullptr, nullptr, nullptr, rotary_dim, 0.f};
        const void** slot[3] = {&tt.q_bias, &tt.k_bias, &tt.v_bias};
        for (int i = 0; i < 3; ++i) {
            if (!in[i]->has_value()) continue;
            bias[i] = token_input(in[i]->value(), k_cache, (int64_t)d.H * d.Dh, "bias");
            *slot[i] = bias[i].data_ptr();
        }
        torch::Tensor sl, indir;
        if (seq_lengths.has_value()) sl = seq_lengths.value();
        ffa_beam_indirection beams = {nullptr, beam_width};
        if (cache_indir.has_value()) {
            indir = cache_indir.value();
            TORCH_CHECK(indir.device() == k_cache.device() && indir.scalar_type() == torch::kInt &&
                            indir.is_contiguous() && indir.dim() == 2 && indir.size(0) == d.B &&
                            indir.size(1) == d.Lmax,
                        "ff_attention: cache_indir must be a contiguous int32 tensor [B, max_len] on the cache's device");
            beams.cache_indir = indir.data_ptr<int>();
        }
        return run(q, k, v, k_cache, v_cache, softmax_scale, curr_timestep, seq_lengths.has_value() ? &sl : nullptr,
                   prob_thresh, !seq_lengths.has_value(), nullptr, nullptr, &tt,
                   cache_indir.has_value() ? &beams : nullptr);
    }

    // Not in the reference: the same step plus what pruning dropped.
    // Returns (out [B,H,Dh], kept_count int32 [B,H], skip_mask uint8 [B,H,Lmax]).
    std::tuple<torch::Tensor, torch::Tensor, torch::Tensor> attention_diag(
        torch::Tensor q, torch::Tensor k, torch::Tensor v, float softmax_scale, int curr_timestep,
        float prob_thresh) {
        const CacheDims d = dims_of(k_cache, v_cache);
        auto kept = torch::zeros({d.B, d.H}, k_cache.options().dtype(torch::kInt32));
        auto mask = torch::zeros({d.B, d.H, d.Lmax}, k_cache.options().dtype(torch::kUInt8));
        auto out = run(q, k, v, k_cache, v_cache, softmax_scale, curr_timestep, nullptr, prob_thresh,
                       true, &kept, &mask);
        return std::make_tuple(out, kept, mask);
    }

    // Not in the reference: the plan the next call at (t, p) would use, as
    // (kind, waves_per_wg, threads_per_key, keys_per_wave, n_splits, tiles_per_split, combine,
    //  whole_heads).
    std::vector<int> launch_plan(int curr_timestep, float prob_thresh) {
        const CacheDims d = dims_of(k_cache, v_cache);
        ffa_launch_plan plan;
        check_status(ffa_plan_launch(plan_precision(precision_of(k_cache)), d.B, d.H, d.Dh, curr_timestep, prob_thresh,
                                     ft_kernel_launch ? 1 : 0, 0, &plan),
                     "launch planning");
        return {plan.kind, plan.waves_per_wg, plan.threads_per_key, plan.keys_per_wave, plan.n_splits,
                plan.tiles_per_split, plan.combine, plan.whole_heads};
    }

    torch::Tensor k_cache;
    torch::Tensor v_cache;
    torch::Tensor workspace;
    bool ft_kernel_launch;

private:
    void ensure_workspace(int B, int H, int Dh, int Lmax, const torch::Device& dev) {
        const size_t need = ffa_workspace_bytes(B, H, Dh, Lmax);
        if (workspace.defined() && workspace.device() == dev && (size_t)workspace.numel() >= need) return;
        // zeros(): the arrival counters must start at zero; the kernels restore that.
        workspace = torch::zeros({(int64_t)need}, torch::TensorOptions().dtype(torch::kUInt8).device(dev));
    }

    torch::Tensor run(const torch::Tensor& q_in, const torch::Tensor& k_in, const torch::Tensor& v_in,
                      torch::Tensor& kc, torch::Tensor& vc, float softmax_scale, int t,
                      const torch::Tensor* seq_lengths, float prob_thresh, bool right_or_no_padding,
                      torch::Tensor* kept, torch::Tensor* mask, const ffa_token_transform* transform = nullptr,
                      const ffa_beam_indirection* beams = nullptr) {
        TORCH_CHECK(kc.is_cuda() && vc.is_cuda() && kc.device() == vc.device() &&
                        kc.scalar_type() == vc.scalar_type(),
                    "ff_attention: caches must be GPU tensors of one dtype on one device");
        const CacheDims d = dims_of(kc, vc);
        const int precision = precision_of(kc);
        TORCH_CHECK(t >= 0 && t < d.Lmax, "ff_attention: timestep ", t, " outside the cache [0, ",
                    d.Lmax, ")");
        const int64_t numel = (int64_t)d.B * d.H * d.Dh;
        c10::hip::HIPGuardMasqueradingAsCUDA guard(kc.device());
        torch::Tensor q = token_input(q_in, kc, numel, "q");
        torch::Tensor k = token_input(k_in, kc, numel, "k");
        torch::Tensor v = token_input(v_in, kc, numel, "v");

        torch::Tensor sl;
        const int* sl_ptr = nullptr;
        if (seq_lengths != nullptr) {
            TORCH_CHECK(seq_lengths->device() == kc.device() && seq_lengths->scalar_type() == torch::kInt &&
                            seq_lengths->numel() == d.B,
                        "ff_attention: seq_lengths must be an int32 tensor of B entries on the cache's device");
            sl = seq_lengths->contiguous();
            sl_ptr = sl.data_ptr<int>();
        }

        ensure_workspace(d.B, d.H, d.Dh, d.Lmax, kc.device());
        torch::Tensor out = torch::empty({d.B, d.H, d.Dh}, q.options());

        ffa_launch_plan plan;
        const bool diag = kept != nullptr || mask != nullptr;
        // The default launch keeps diagnostics at any length; the exact split kernel has none.
        check_status(ffa_plan_launch(plan_precision(precision), d.B, d.H, d.Dh, t, prob_thresh,
                                     (ft_kernel_launch || diag) ? 1 : 0, 0, &plan),
                     "launch planning");
        if (transform != nullptr || beams != nullptr) {
            TORCH_CHECK(!diag, "ff_attention: diagnostics cannot be combined with a token transform or beams");
            check_status(ffa_attention_ex(precision, d.B, d.H, d.Dh, d.Lmax, softmax_scale, t, q.data_ptr(),
                                          k.data_ptr(), v.data_ptr(), kc.data_ptr(), vc.data_ptr(), out.data_ptr(),
                                          sl_ptr, prob_thresh, &plan, right_or_no_padding ? 1 : 0, transform, beams,
                                          workspace.data_ptr(), (size_t)workspace.numel(), stream_of(kc)),
                         "attention");
            return out;
        }
        const int rc = ffa_attention_diag(
            precision, d.B, d.H, d.Dh, d.Lmax, softmax_scale, t, q.data_ptr(), k.data_ptr(), v.data_ptr(),
            kc.data_ptr(), vc.data_ptr(), out.data_ptr(), sl_ptr, prob_thresh, &plan,
            right_or_no_padding ? 1 : 0, workspace.data_ptr(), (size_t)workspace.numel(),
            kept ? (uint32_t*)kept->data_ptr() : nullptr, mask ? (uint8_t*)mask->data_ptr() : nullptr,
            stream_of(kc));
        check_status(rc, "attention");
        return out;
    }
};

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
    m.doc() = "MI355X-native FastForwardAttention decode step (drop-in for ff_attention)";
    py::class_<FastForwardAttn>(m, "FastForwardAttn")
        .def(py::init<torch::Tensor, torch::Tensor, int, bool>())
        .def("get_cache", &FastForwardAttn::get_cache, "Get KV_cache")
        .def("attention",
             py::overload_cast<torch::Tensor, torch::Tensor, torch::Tensor, float, int, float>(
                 &FastForwardAttn::attention),
             "Attention forward, fixed timestep, cache held by the object")
        .def("attention",
             py::overload_cast<torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor,
                               float, int, float>(&FastForwardAttn::attention),
             "Attention forward, fixed timestep")
        .def("attention",
             py::overload_cast<torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor,
                               float, int, torch::Tensor, float>(&FastForwardAttn::attention),
             "Attention forward, left-padded batch")
        .def("attention_ex", &FastForwardAttn::attention_ex,
             "Attention forward with q/k/v bias and rotary embedding of the new token and, optionally, "
             "beam-search cache indirection (cache_indir int32 [B, max_len], beam_width)",
             py::arg("q"), py::arg("k"), py::arg("v"), py::arg("k_cache"), py::arg("v_cache"),
             py::arg("softmax_scale"), py::arg("curr_timestep"), py::arg("seq_lengths"), py::arg("prob_thresh"),
             py::arg("rotary_dim"), py::arg("q_bias"), py::arg("k_bias"), py::arg("v_bias"),
             py::arg("cache_indir") = py::none(), py::arg("beam_width") = 1)
        .def("attention_diag", &FastForwardAttn::attention_diag,
             "Attention forward plus (kept_count, skip_mask) of the pruning rule")
        .def("launch_plan", &FastForwardAttn::launch_plan, "Launch plan for (t, p)");
}
