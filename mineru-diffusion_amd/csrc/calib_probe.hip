// Calibration helper for the benchmark (no counterpart in the reference): a register-only loop of
// back-to-back bf16 MFMAs, 32x32x16 or 16x16x32, on operands taken from memory once.  It measures what the
// matrix pipe itself sustains on a given kind of data under the board's power limit -- the ceiling that any
// kernel feeding the same data through the same instructions shares -- so that the attention kernel's
// fraction of the published peak can be read against it.  One wavefront per SIMD with 256 blocks, two with 512.
#include "mdx_common.h"

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;

template <int SHAPE>
__global__ __launch_bounds__(256) void mfma_loop_kernel(const uint32_t* __restrict__ operands, float* __restrict__ out, int iters)
{
    bf16x8 a[8], b[8];
    const uint32_t* s = operands + (size_t)(blockIdx.x * 256 + threadIdx.x) * 64;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        union { uint32_t u[4]; bf16x8 v; } x, y;
#pragma unroll
        for (int k = 0; k < 4; ++k) { x.u[k] = s[i * 8 + k]; y.u[k] = s[i * 8 + 4 + k]; }
        a[i] = x.v; b[i] = y.v;
    }
    float sum = 0.f;
    if (SHAPE == 32) {
        f32x16 acc[8];
#pragma unroll
        for (int i = 0; i < 8; ++i)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][e] = 0.f;
        for (int it = 0; it < iters; it += 8) {
#pragma unroll
            for (int r = 0; r < 8; ++r)
#pragma unroll
                for (int i = 0; i < 8; ++i) acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i], b[(i + r) & 7], acc[i], 0, 0, 0);
        }
#pragma unroll
        for (int i = 0; i < 8; ++i)
#pragma unroll
            for (int e = 0; e < 16; ++e) sum += acc[i][e];
    } else {
        f32x4 acc[16];
#pragma unroll
        for (int i = 0; i < 16; ++i)
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[i][e] = 0.f;
        for (int it = 0; it < iters; it += 8) {
#pragma unroll
            for (int r = 0; r < 8; ++r)
#pragma unroll
                for (int i = 0; i < 16; ++i) acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[i & 7], b[(i + r) & 7], acc[i], 0, 0, 0);
        }
#pragma unroll
        for (int i = 0; i < 16; ++i)
#pragma unroll
            for (int e = 0; e < 4; ++e) sum += acc[i][e];
    }
    out[blockIdx.x * 256 + threadIdx.x] = sum;
}

}  // namespace

extern "C" int64_t mdx_calib_mfma_loop_flops(int32_t shape, int32_t blocks, int32_t iters)
{
    if (blocks <= 0 || iters <= 0) return 0;
    const int64_t per_wave_iter = shape == 32 ? 8ll * 32 * 32 * 16 * 2 : 16ll * 16 * 16 * 32 * 2;
    return (int64_t)blocks * 4 * ((iters + 7) / 8 * 8) * per_wave_iter;
}

extern "C" int mdx_calib_mfma_loop(int32_t shape, const void* operands, float* out, int32_t blocks, int32_t iters, mdx_stream_t stream)
{
    MDX_REQUIRE(shape == 32 || shape == 16, MDX_EINVAL, "calib_mfma_loop: shape %d (32 = 32x32x16, 16 = 16x16x32)", shape);
    MDX_REQUIRE(blocks >= 0 && iters >= 0, MDX_EINVAL, "calib_mfma_loop: negative size");
    if (blocks == 0 || iters == 0) return MDX_OK;
    MDX_REQUIRE(operands && out, MDX_EINVAL, "calib_mfma_loop: null pointer");
    if (shape == 32) mfma_loop_kernel<32><<<(unsigned)blocks, 256, 0, static_cast<hipStream_t>(stream)>>>((const uint32_t*)operands, out, iters);
    else             mfma_loop_kernel<16><<<(unsigned)blocks, 256, 0, static_cast<hipStream_t>(stream)>>>((const uint32_t*)operands, out, iters);
    return mdx::check_launch("calib_mfma_loop");
}
