// Decode kernels of the engine instantiated for one element type (float), without a transform of the new token:
// one translation unit per element type and transform switch, so that the six compile in parallel.
#include "ffa_decode_kernels.h"

namespace ffa {

int launch_decode_f32(const DecodeParams& P, int head_dim, const ffa_launch_plan& plan, void* stream) {
    return dispatch_head_dim<float, false>(P, head_dim, plan, reinterpret_cast<hipStream_t>(stream));
}

}  // namespace ffa
