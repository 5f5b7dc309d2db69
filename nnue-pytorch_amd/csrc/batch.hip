// The device side of the loader hand-off.  A batch arrives as ONE block of 32-bit words (the
// loader's float block followed by its int block, copied by one DMA); most tensors the model wants
// are views of that block.  The two that are not (them = 1 - us, piece_count as int64) are written
// here in one pass, in place of two elementwise launches per batch.
#include "common.h"

namespace {

__global__ __launch_bounds__(256) void k_batch_unpack(const float* __restrict__ us,
                                                      const int32_t* __restrict__ piece_count32,
                                                      float* __restrict__ them, int64_t* __restrict__ piece_count,
                                                      int B) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i >= B) return;
    them[i] = 1.0f - us[i];
    piece_count[i] = (int64_t)piece_count32[i];
}

}  // namespace

extern "C" int nnueft_batch_unpack(const float* us, const int32_t* piece_count32, float* them, int64_t* piece_count,
                                   int B, void* stream) {
    if (B <= 0 || !us || !piece_count32 || !them || !piece_count) return NNUEFT_E_ARG;
    hipLaunchKernelGGL(k_batch_unpack, dim3((B + 255) / 256), dim3(256), 0, (hipStream_t)stream, us, piece_count32,
                       them, piece_count, B);
    NNUEFT_LAUNCH_CHECK();
    return 0;
}
