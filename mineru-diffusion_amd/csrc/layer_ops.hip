// The two element-wise steps that sit between the GEMMs of a decoder layer, each as one pass
// over its rows:
//
//   add_rms_norm   hidden, residual = norm(hidden, residual)
//                  nanovllm/layers/layernorm.py:16-26 (rms_forward) and :28-41 (add_rms_forward),
//                  called at nanovllm/models/sdar.py:147-152,180
//   silu_and_mul   x = act_fn(gate_up)
//                  nanovllm/layers/activation.py:7-16, called at nanovllm/models/sdar.py:110-111
//
// In the stock engine these are five to six element-wise launches per layer (add, norm, add,
// norm, SiLU on a strided half, multiply); here they are two, and every byte is read once.
// Both are pure bandwidth ops.
//
// Rounding follows the reference line by line: the sum x + residual is formed in fp32 and
// rounded once into the new residual; the mean of squares uses the unrounded fp32 sum; the
// normalised value is rounded to the storage type and then multiplied by the weight in the
// storage type (layernorm.py:37-40).  SiLU is evaluated in fp32, rounded to the storage type,
// and the product with the other half is rounded again (the reference's activation is the
// third-party liger-kernel 0.6.4 SwiGLU forward, which computes silu(a).cast(b.dtype) * b).
#include "mdx_common.h"

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;

constexpr int kNormThreads = 256;
constexpr int kNormMaxVecs = 4;                  // 16-byte vectors per thread: rows up to 8192 elements

struct NormParams {
    const __bf16* x; int64_t x_stride;                     // [rows][hidden]
    const __bf16* residual_in; int64_t res_in_stride;      // null: plain rms_forward
    __bf16* residual_out; int64_t res_out_stride;          // null when residual_in is null
    const __bf16* weight; float eps;
    __bf16* out; int64_t out_stride;
    int64_t rows; int hidden;
};

// One workgroup per row; thread t holds vectors t, t + 256, ... of the row in registers, so the
// row is read once.  In-place use (out == x, residual_out == residual_in) is safe: a thread
// writes only the elements it has read.
template <int VECS>
__global__ __launch_bounds__(kNormThreads) void add_rms_norm_kernel(const NormParams P)
{
    __shared__ float wave_sums[kNormThreads / 64];
    const int64_t row = blockIdx.x;
    const int tid = threadIdx.x;
    const int n_vec = P.hidden / 8;
    float s[VECS][8];
    float sq = 0.f;
#pragma unroll
    for (int i = 0; i < VECS; ++i) {
        const int v = tid + i * kNormThreads;
        if (v < n_vec) {
            const bf16x8 a = *reinterpret_cast<const bf16x8*>(P.x + row * P.x_stride + 8 * v);
#pragma unroll
            for (int e = 0; e < 8; ++e) s[i][e] = (float)a[e];
            if (P.residual_in) {
                const bf16x8 r = *reinterpret_cast<const bf16x8*>(P.residual_in + row * P.res_in_stride + 8 * v);
                bf16x8 nr;
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    s[i][e] += (float)r[e];
                    nr[e] = (__bf16)s[i][e];
                }
                *reinterpret_cast<bf16x8*>(P.residual_out + row * P.res_out_stride + 8 * v) = nr;
            }
#pragma unroll
            for (int e = 0; e < 8; ++e) sq += s[i][e] * s[i][e];
        }
    }
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) sq += __shfl_xor(sq, o);
    if ((tid & 63) == 0) wave_sums[tid >> 6] = sq;
    __syncthreads();
    float total = 0.f;
#pragma unroll
    for (int w = 0; w < kNormThreads / 64; ++w) total += wave_sums[w];
    const float inv = 1.0f / sqrtf(total / (float)P.hidden + P.eps);
#pragma unroll
    for (int i = 0; i < VECS; ++i) {
        const int v = tid + i * kNormThreads;
        if (v < n_vec) {
            const bf16x8 w = *reinterpret_cast<const bf16x8*>(P.weight + 8 * v);
            bf16x8 y;
#pragma unroll
            for (int e = 0; e < 8; ++e) y[e] = (__bf16)((float)(__bf16)(s[i][e] * inv) * (float)w[e]);
            *reinterpret_cast<bf16x8*>(P.out + row * P.out_stride + 8 * v) = y;
        }
    }
}

// One thread per 16-byte vector of the output: reads the matching vectors of the two halves.
__global__ __launch_bounds__(256) void silu_and_mul_kernel(const __bf16* x, int64_t x_stride, __bf16* out, int64_t out_stride,
                                                            int64_t rows, int inter)
{
    const int vecs_per_row = inter / 8;
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= rows * vecs_per_row) return;
    const int64_t row = idx / vecs_per_row;
    const int v = (int)(idx - row * vecs_per_row);
    const __bf16* src = x + row * x_stride + 8 * v;
    const bf16x8 g = __builtin_nontemporal_load(reinterpret_cast<const bf16x8*>(src));
    const bf16x8 u = __builtin_nontemporal_load(reinterpret_cast<const bf16x8*>(src + inter));
    bf16x8 y;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        const float a = (float)g[e];
        const float act = a / (1.0f + __expf(-a));
        y[e] = (__bf16)((float)(__bf16)act * (float)u[e]);
    }
    *reinterpret_cast<bf16x8*>(out + row * out_stride + 8 * v) = y;
}

}  // namespace

extern "C" int mdx_add_rms_norm(const void* x, int64_t x_row_stride,
                                const void* residual_in, int64_t residual_in_row_stride,
                                void* residual_out, int64_t residual_out_row_stride,
                                const void* weight, float eps,
                                void* out, int64_t out_row_stride,
                                int64_t rows, int32_t hidden, int32_t dtype, mdx_stream_t stream_)
{
    const char* what = "add_rms_norm";
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    MDX_REQUIRE(rows >= 0 && hidden > 0, MDX_EINVAL, "%s: bad size (rows %lld, hidden %d)", what, (long long)rows, hidden);
    MDX_REQUIRE(dtype == MDX_BF16, MDX_EUNSUPPORTED, "%s: dtype %d (only bf16)", what, dtype);
    MDX_REQUIRE(hidden % 8 == 0 && hidden <= 8 * kNormThreads * kNormMaxVecs, MDX_EUNSUPPORTED,
                "%s: hidden %d (multiples of 8 up to %d)", what, hidden, 8 * kNormThreads * kNormMaxVecs);
    MDX_REQUIRE(eps >= 0.f, MDX_EINVAL, "%s: negative eps", what);
    if (rows == 0) return MDX_OK;
    MDX_REQUIRE(x && weight && out, MDX_EINVAL, "%s: null pointer", what);
    MDX_REQUIRE((residual_in == nullptr) == (residual_out == nullptr), MDX_EINVAL,
                "%s: residual_in and residual_out go together", what);
    MDX_REQUIRE(rows <= 0x7fffffffLL, MDX_EUNSUPPORTED, "%s: %lld rows", what, (long long)rows);
    MDX_REQUIRE(mdx::aligned16(x) && mdx::aligned16(out) && mdx::aligned16(weight) && mdx::aligned16(residual_in) && mdx::aligned16(residual_out) &&
                x_row_stride % 8 == 0 && out_row_stride % 8 == 0 &&
                (!residual_in || (residual_in_row_stride % 8 == 0 && residual_out_row_stride % 8 == 0)),
                MDX_EUNSUPPORTED, "%s: rows must be 16-byte aligned", what);
    MDX_REQUIRE(x_row_stride >= hidden && out_row_stride >= hidden &&
                (!residual_in || (residual_in_row_stride >= hidden && residual_out_row_stride >= hidden)),
                MDX_EINVAL, "%s: row stride smaller than the row", what);
    NormParams P;
    P.x = (const __bf16*)x; P.x_stride = x_row_stride;
    P.residual_in = (const __bf16*)residual_in; P.res_in_stride = residual_in_row_stride;
    P.residual_out = (__bf16*)residual_out; P.res_out_stride = residual_out_row_stride;
    P.weight = (const __bf16*)weight; P.eps = eps;
    P.out = (__bf16*)out; P.out_stride = out_row_stride;
    P.rows = rows; P.hidden = hidden;
    const int vecs = (hidden / 8 + kNormThreads - 1) / kNormThreads;
    const dim3 grid((unsigned)rows);
    if (vecs <= 1) add_rms_norm_kernel<1><<<grid, kNormThreads, 0, stream>>>(P);
    else if (vecs == 2) add_rms_norm_kernel<2><<<grid, kNormThreads, 0, stream>>>(P);
    else add_rms_norm_kernel<4><<<grid, kNormThreads, 0, stream>>>(P);
    return mdx::check_launch(what);
}

extern "C" int mdx_silu_and_mul(const void* x, int64_t x_row_stride, void* out, int64_t out_row_stride,
                                int64_t rows, int32_t intermediate, int32_t dtype, mdx_stream_t stream_)
{
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    MDX_REQUIRE(rows >= 0 && intermediate > 0, MDX_EINVAL, "silu_and_mul: bad size (rows %lld, width %d)", (long long)rows, intermediate);
    MDX_REQUIRE(dtype == MDX_BF16, MDX_EUNSUPPORTED, "silu_and_mul: dtype %d (only bf16)", dtype);
    MDX_REQUIRE(intermediate % 8 == 0, MDX_EUNSUPPORTED, "silu_and_mul: width %d not a multiple of 8", intermediate);
    if (rows == 0) return MDX_OK;
    MDX_REQUIRE(x && out, MDX_EINVAL, "silu_and_mul: null pointer");
    MDX_REQUIRE(mdx::aligned16(x) && mdx::aligned16(out) && x_row_stride % 8 == 0 && out_row_stride % 8 == 0,
                MDX_EUNSUPPORTED, "silu_and_mul: rows must be 16-byte aligned");
    MDX_REQUIRE(x_row_stride >= 2 * (int64_t)intermediate && out_row_stride >= intermediate, MDX_EINVAL,
                "silu_and_mul: row stride smaller than the row");
    const int64_t n_vec = rows * (intermediate / 8);
    MDX_REQUIRE((n_vec + 255) / 256 <= 0x7fffffffLL, MDX_EUNSUPPORTED, "silu_and_mul: %lld rows", (long long)rows);
    silu_and_mul_kernel<<<(unsigned)((n_vec + 255) / 256), 256, 0, stream>>>(
        (const __bf16*)x, x_row_stride, (__bf16*)out, out_row_stride, rows, intermediate);
    return mdx::check_launch("silu_and_mul");
}
