// A translation unit written the way a user of the reference's c_ffa_api.h writes one: it calls
// do_attention<T> and call_attention<T> with the reference's argument lists.  Compiled (and, when
// the library is built, linked) by tests/test_host_cpp.py; never run.
#include "ffa_reference_shim.h"

int use_f16(uint16_t* q, uint16_t* k, uint16_t* v, uint16_t* kc, uint16_t* vc, uint16_t* out, int* seq_lengths) {
    do_attention<uint16_t>(/*batch_size=*/10, /*head_num=*/32, /*head_dim=*/64, /*max_seq_length=*/1128, q, k, v, kc,
                           vc, out, /*softmax_scale=*/0.125f, /*curr_timestep=*/1000, seq_lengths,
                           /*prob_thresh=*/0.f, /*tpb=*/256, /*tpv=*/8, /*tpk=*/4);
    return ffa_last_status();
}

int use_f32(float* q, float* k, float* v, float* kc, float* vc, float* out) {
    call_attention<float>(1, 32, 64, 1128, 0.125f, 1000, q, k, v, kc, vc, out, nullptr, 0.001f, 4, 4, 128, false);
    return ffa_last_status();
}

int use_unsupported(double* p) {
    do_attention<double>(1, 1, 64, 8, p, p, p, p, p, p, 1.f, 0, nullptr, 0.f, 64, 1, 1);
    return ffa_last_status();  // FFA_ERR_DTYPE
}

int main() { return 0; }
