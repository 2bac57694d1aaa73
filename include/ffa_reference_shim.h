/*
 * ffa_reference_shim.h -- the reference's C++ entry points on top of the MI355X engine's C ABI.
 *
 * A program written against the reference's c_ffa_api.h (:5-20: call_attention<T>,
 * do_attention<T>) compiles unchanged with this header included in its place (or installed
 * under that name) and links libffa_hip.so instead of libffa.so.  Same template names, same parameter order and
 * meaning; what differs:
 *   - tpv / tpk / tpb (threads per value, per key, per block of the CUDA launch,
 *     kernel_launch_utils.h:135) are accepted and ignored: the engine plans its own launch
 *     from the step's shape at every call;
 *   - the step goes through ffa_attention_static_scratch, the entry point that needs no
 *     workspace and allocates nothing, because the reference's signature has no place for one;
 *     calls therefore must not overlap on one GPU (the reference's own calls all run on the
 *     default stream and never do);
 *   - the reference prints and carries on when something is wrong (attention.cu:1444-1451,
 *     :1529); here the status of the last call is kept per thread, ffa_last_status() returns
 *     it, and a failed call prints one line to stderr.
 * Kernels are launched on the default stream, like the reference's (attention.cu:1504).
 */
#ifndef FFA_REFERENCE_SHIM_C_FFA_API_H
#define FFA_REFERENCE_SHIM_C_FFA_API_H

#include <stdint.h>
#include <stdio.h>

#include "ffa_c_api.h"

namespace ffa_shim {

inline int& last_status() {
    static thread_local int status = FFA_OK;
    return status;
}

inline void step(int precision, int batch_size, int head_num, int size_per_head, int seq_length,
                 float softmax_scale, int curr_timestep, const void* q, const void* k, const void* v,
                 void* k_cache, void* v_cache, void* out, const int* seq_lengths, float prob_thresh,
                 bool right_or_no_padding) {
    const int rc = ffa_attention_static_scratch(precision, batch_size, head_num, size_per_head, seq_length,
                                                softmax_scale, curr_timestep, q, k, v, k_cache, v_cache, out,
                                                seq_lengths, prob_thresh, /*plan=*/nullptr,
                                                right_or_no_padding ? 1 : 0, /*transform=*/nullptr,
                                                /*beams=*/nullptr, /*stream=*/nullptr);
    last_status() = rc;
    if (rc != FFA_OK) fprintf(stderr, "call_attention: %s\n", ffa_status_string(rc));
}

}  // namespace ffa_shim

/* Status of the calling thread's most recent call_attention / do_attention (FFA_OK = 0). */
inline int ffa_last_status() { return ffa_shim::last_status(); }

/* c_ffa_api.h:5-8: the primary template covers the element types the engine does not know. */
template <typename T>
void call_attention(int batch_size, int head_num, int size_per_head, int seq_length, float softmax_scale,
                    int curr_timestep, T* q, T* k, T* v, T* k_cache, T* v_cache, T* out, int* seq_lengths,
                    float prob_thresh, int tpv, int tpk, int tpb, bool right_or_no_padding) {
    (void)batch_size; (void)head_num; (void)size_per_head; (void)seq_length; (void)softmax_scale;
    (void)curr_timestep; (void)q; (void)k; (void)v; (void)k_cache; (void)v_cache; (void)out;
    (void)seq_lengths; (void)prob_thresh; (void)tpv; (void)tpk; (void)tpb; (void)right_or_no_padding;
    ffa_shim::last_status() = FFA_ERR_DTYPE;
    fprintf(stderr, "call_attention: %s\n", ffa_status_string(FFA_ERR_DTYPE));
}

/* c_ffa_api.h:10-11 (defined in attention.cu:1512-1531). */
template <>
inline void call_attention<float>(int batch_size, int head_num, int size_per_head, int seq_length,
                                  float softmax_scale, int curr_timestep, float* q, float* k, float* v,
                                  float* k_cache, float* v_cache, float* out, int* seq_lengths,
                                  float prob_thresh, int tpv, int tpk, int tpb, bool right_or_no_padding) {
    (void)tpv; (void)tpk; (void)tpb;
    ffa_shim::step(FFA_PRECISION_F32, batch_size, head_num, size_per_head, seq_length, softmax_scale,
                   curr_timestep, q, k, v, k_cache, v_cache, out, seq_lengths, prob_thresh, right_or_no_padding);
}

/* c_ffa_api.h:13-14 (defined in attention.cu:1533-1554): fp16 travels as uint16_t bit patterns. */
template <>
inline void call_attention<uint16_t>(int batch_size, int head_num, int size_per_head, int seq_length,
                                     float softmax_scale, int curr_timestep, uint16_t* q, uint16_t* k,
                                     uint16_t* v, uint16_t* k_cache, uint16_t* v_cache, uint16_t* out,
                                     int* seq_lengths, float prob_thresh, int tpv, int tpk, int tpb,
                                     bool right_or_no_padding) {
    (void)tpv; (void)tpk; (void)tpb;
    ffa_shim::step(FFA_PRECISION_F16, batch_size, head_num, size_per_head, seq_length, softmax_scale,
                   curr_timestep, q, k, v, k_cache, v_cache, out, seq_lengths, prob_thresh, right_or_no_padding);
}

/* c_ffa_api.h:17-20: the reference's order of arguments (scale and timestep after the pointers,
 * tpb before tpv and tpk), right_or_no_padding fixed to true. */
template <typename T>
void do_attention(int batch_size, int head_num, int head_dim, int max_seq_length, T* q, T* k, T* v, T* k_cache,
                  T* v_cache, T* out, float softmax_scale, int curr_timestep, int* seq_lengths,
                  float prob_thresh, int tpb, int tpv, int tpk) {
    call_attention<T>(batch_size, head_num, head_dim, max_seq_length, softmax_scale, curr_timestep, q, k, v,
                      k_cache, v_cache, out, seq_lengths, prob_thresh, tpv, tpk, tpb, true);
}

#endif /* FFA_REFERENCE_SHIM_C_FFA_API_H */
