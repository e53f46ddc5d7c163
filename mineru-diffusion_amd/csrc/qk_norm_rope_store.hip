// Fused producer of the attention inputs: per-head q/k RMSNorm, rotary embedding and the
// KV-cache store in one pass over the fused QKV projection output.
//
// Replaces, for one token, the chain
//   q = q_norm(q); k = k_norm(k)          nanovllm/models/sdar.py:79-81, layers/layernorm.py:16-26
//   q, k = rotary_emb(positions, q, k)    nanovllm/layers/rotary_embedding.py:6-14,37-48
//   store_kvcache(k, v, ...)              nanovllm/layers/sdar_attention.py:37-38, layers/attention.py:10-40
// which in the engine is about a dozen element-wise launches per layer.  It is a pure
// bandwidth op (reads 8 KiB of QKV per token, writes q, k and the two cache rows), so: one
// workgroup per token, 8 lanes per head row, each lane holding elements [8j, 8j+8) and
// [64+8j, 64+8j+8) of the row, which are exactly the pairs the rotation mixes, so no data
// crosses lanes except the 8-lane sum of squares.
//
// Rounding follows the reference: the normalised value is rounded to the storage type, then
// multiplied by the weight in the storage type (layernorm.py:24-25); the rotation is done in
// fp32 and rounded once (rotary_embedding.py:11-14).
#include "mdx_common.h"

namespace {

constexpr int kHeadDim = 128;
constexpr int kLanesPerHead = 8;

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;

struct FusedParams {
    const __bf16* qkv; int64_t qkv_stride;
    const __bf16* q_w; const __bf16* k_w; float eps;
    const float* cos_t; const float* sin_t; int64_t max_pos; const int64_t* positions;
    __bf16* q_out; int64_t q_out_stride;
    __bf16* k_out; int64_t k_out_stride;          // k_out may be null
    __bf16* k_cache; __bf16* v_cache;             // both may be null
    const int32_t* slot_mapping; int64_t num_slots;
    int64_t n_tokens; int hq, hkv;
};

__global__ __launch_bounds__(256) void qk_norm_rope_store_kernel(const FusedParams P)
{
    const int64_t tok = blockIdx.x;
    const int n_rows = P.hq + 2 * P.hkv;                       // head rows of this token: q | k | v
    const int j = threadIdx.x % kLanesPerHead;
    const int64_t pos = P.positions[tok];
    int64_t slot = -1;
    if (P.k_cache && P.slot_mapping) {
        const int64_t s = P.slot_mapping[tok];
        if (s >= 0 && s < P.num_slots) slot = s;
    }
    float cs[8], sn[8];
    const bool pos_ok = pos >= 0 && pos < P.max_pos;            // out-of-table positions rotate by 0
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        cs[e] = pos_ok ? P.cos_t[pos * (kHeadDim / 2) + 8 * j + e] : 1.0f;
        sn[e] = pos_ok ? P.sin_t[pos * (kHeadDim / 2) + 8 * j + e] : 0.0f;
    }
    for (int row = threadIdx.x / kLanesPerHead; row < n_rows; row += 256 / kLanesPerHead) {
        const __bf16* src = P.qkv + tok * P.qkv_stride + (int64_t)row * kHeadDim;
        bf16x8 a = *reinterpret_cast<const bf16x8*>(src + 8 * j);
        bf16x8 b = *reinterpret_cast<const bf16x8*>(src + 64 + 8 * j);
        const bool is_q = row < P.hq, is_k = !is_q && row < P.hq + P.hkv;
        if (is_q || is_k) {
            float ss = 0.f;
#pragma unroll
            for (int e = 0; e < 8; ++e) { const float x = (float)a[e], y = (float)b[e]; ss += x * x + y * y; }
            ss += __shfl_xor(ss, 1);
            ss += __shfl_xor(ss, 2);
            ss += __shfl_xor(ss, 4);
            const float inv = rsqrtf(ss * (1.0f / kHeadDim) + P.eps);
            const __bf16* w = is_q ? P.q_w : P.k_w;
            const bf16x8 wa = *reinterpret_cast<const bf16x8*>(w + 8 * j);
            const bf16x8 wb = *reinterpret_cast<const bf16x8*>(w + 64 + 8 * j);
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float x1 = (float)(__bf16)((float)(__bf16)((float)a[e] * inv) * (float)wa[e]);
                const float x2 = (float)(__bf16)((float)(__bf16)((float)b[e] * inv) * (float)wb[e]);
                a[e] = (__bf16)(x1 * cs[e] - x2 * sn[e]);
                b[e] = (__bf16)(x2 * cs[e] + x1 * sn[e]);
            }
        }
        if (is_q) {
            __bf16* dst = P.q_out + tok * P.q_out_stride + (int64_t)row * kHeadDim;
            *reinterpret_cast<bf16x8*>(dst + 8 * j) = a;
            *reinterpret_cast<bf16x8*>(dst + 64 + 8 * j) = b;
        } else {
            const int kvrow = is_k ? row - P.hq : row - P.hq - P.hkv;
            if (is_k && P.k_out) {
                __bf16* dst = P.k_out + tok * P.k_out_stride + (int64_t)kvrow * kHeadDim;
                *reinterpret_cast<bf16x8*>(dst + 8 * j) = a;
                *reinterpret_cast<bf16x8*>(dst + 64 + 8 * j) = b;
            }
            if (slot >= 0) {
                __bf16* dst = (is_k ? P.k_cache : P.v_cache) + (slot * P.hkv + kvrow) * kHeadDim;
                *reinterpret_cast<bf16x8*>(dst + 8 * j) = a;
                *reinterpret_cast<bf16x8*>(dst + 64 + 8 * j) = b;
            }
        }
    }
}

}  // namespace

extern "C" int mdx_qk_norm_rope_store(const void* qkv, int64_t qkv_row_stride,
                                      const void* q_weight, const void* k_weight, float eps,
                                      const float* cos_table, const float* sin_table, int64_t max_positions,
                                      const int64_t* positions,
                                      void* q_out, int64_t q_out_row_stride,
                                      void* k_out, int64_t k_out_row_stride,
                                      void* k_cache, void* v_cache, const int32_t* slot_mapping, int64_t num_slots,
                                      int64_t n_tokens, int32_t num_q_heads, int32_t num_kv_heads, int32_t head_dim,
                                      int32_t dtype, mdx_stream_t stream_)
{
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    MDX_REQUIRE(n_tokens >= 0 && num_q_heads > 0 && num_kv_heads > 0, MDX_EINVAL, "qk_norm_rope_store: bad size");
    MDX_REQUIRE(dtype == MDX_BF16, MDX_EUNSUPPORTED, "qk_norm_rope_store: dtype %d (only bf16)", dtype);
    MDX_REQUIRE(head_dim == kHeadDim, MDX_EUNSUPPORTED, "qk_norm_rope_store: head_dim %d (only 128)", head_dim);
    if (n_tokens == 0) return MDX_OK;
    MDX_REQUIRE(qkv && q_weight && k_weight && cos_table && sin_table && positions && q_out, MDX_EINVAL,
                "qk_norm_rope_store: null pointer");
    MDX_REQUIRE((k_cache == nullptr) == (v_cache == nullptr), MDX_EINVAL, "qk_norm_rope_store: give both caches or neither");
    MDX_REQUIRE(!k_cache || slot_mapping, MDX_EINVAL, "qk_norm_rope_store: caches without slot_mapping");
    MDX_REQUIRE(n_tokens < ((int64_t)1 << 31), MDX_EUNSUPPORTED, "qk_norm_rope_store: too many tokens");
    MDX_REQUIRE(mdx::aligned16(qkv) && mdx::aligned16(q_out) && mdx::aligned16(q_weight) && mdx::aligned16(k_weight) &&
                (!k_out || mdx::aligned16(k_out)) && (!k_cache || (mdx::aligned16(k_cache) && mdx::aligned16(v_cache))) &&
                qkv_row_stride % 8 == 0 && q_out_row_stride % 8 == 0 && k_out_row_stride % 8 == 0,
                MDX_EUNSUPPORTED, "qk_norm_rope_store: tensors must be 16-byte aligned with row strides that are multiples of 8");
    MDX_REQUIRE(qkv_row_stride >= (int64_t)(num_q_heads + 2 * num_kv_heads) * kHeadDim, MDX_EINVAL,
                "qk_norm_rope_store: qkv row stride shorter than a QKV row");
    FusedParams P;
    P.qkv = (const __bf16*)qkv; P.qkv_stride = qkv_row_stride;
    P.q_w = (const __bf16*)q_weight; P.k_w = (const __bf16*)k_weight; P.eps = eps;
    P.cos_t = cos_table; P.sin_t = sin_table; P.max_pos = max_positions; P.positions = positions;
    P.q_out = (__bf16*)q_out; P.q_out_stride = q_out_row_stride;
    P.k_out = (__bf16*)k_out; P.k_out_stride = k_out_row_stride;
    P.k_cache = (__bf16*)k_cache; P.v_cache = (__bf16*)v_cache;
    P.slot_mapping = slot_mapping; P.num_slots = num_slots;
    P.n_tokens = n_tokens; P.hq = num_q_heads; P.hkv = num_kv_heads;
    qk_norm_rope_store_kernel<<<(unsigned)n_tokens, 256, 0, stream>>>(P);
    return mdx::check_launch("qk_norm_rope_store");
}
