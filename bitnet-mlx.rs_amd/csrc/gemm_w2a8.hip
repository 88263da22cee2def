// Prefill GEMM: int8 activations [m, k] x 2-bit ternary weights [n, k] -> int32 [m, n] on the int8 MFMA
// units of gfx950, with the fp32 scale epilogue fused into the store.
//
//   acc[t, n] = sum_k a[t, k] * w[n, k]      bitnet-quant/src/simd/matrix.rs:256-282 (ternary_gemm_scalar),
//                                            front door bitnet-quant/src/bitlinear/forward.rs:179-214
//   out[t, n] = (float(acc) * w_scale) / a_scale[t] (+ bias[n]) (+ residual[t, n])
#include "kernels.hpp"

namespace bitnet {

int launch_gemm_tiled(const uint8_t *tiled, const int8_t *a, size_t m, size_t n, size_t k, int32_t *acc,
                      const float *w_scale, const float *a_scale, const float *bias, const float *residual,
                      float *out, hipStream_t stream)
{
    // Until the MFMA kernel is in place every token count goes through the decode GEMV in blocks.
    return launch_gemv_tiled(tiled, a, m, n, k, acc, w_scale, a_scale, bias, residual, out, stream);
}

}  // namespace bitnet
