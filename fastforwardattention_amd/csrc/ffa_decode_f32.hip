// Decode kernels of the engine instantiated for one element type (float): one translation unit
// per type, so that the three compile in parallel.
#include "ffa_decode_kernels.h"

namespace ffa {

int launch_decode_f32(const DecodeParams& P, int head_dim, const ffa_launch_plan& plan, void* stream) {
    return dispatch_head_dim<float>(P, head_dim, plan, reinterpret_cast<hipStream_t>(stream));
}

}  // namespace ffa
