// Staircase block-prefill attention in fp32 arithmetic: the form of mdx_staircase_attn_varlen for fp32
// q/k/v/o and for heads that the 16-bit kernels of staircase_attn.hip do not take (wider than 128 columns,
// up to 256, or not a multiple of 16).  The reference's kernel accepts any q.dtype and any head_dim
// (engines/nano_dvlm/nanovllm/kernels/triton/attention/block_prefill_attention_v2.py:16-199:
// BLOCK_DMODEL = head_dim, o = empty_like(q)); the model itself runs bf16 with d = 128, so this is the path
// for callers outside the model's own configuration.  Arithmetic and layout: attn_f32_tile.h.
//
// Same decomposition as the 16-bit kernels: a workgroup of 4 wavefronts owns 128 padded query rows of one
// (sequence, head), a wavefront 32 of them; K and V tiles of 32 keys are staged through LDS as fp32, one at a time.
//
// The mask is the reference's (:98-102,137-139): with nb = ceil(L / S) blocks right-aligned, pad = nb S - L,
// query row i sees key j iff j <= ((i + pad) / S + 1) S - 1 - pad.
#include "attn_f32_tile.h"
#include <atomic>

namespace {

using namespace mdx_attn_f32;

constexpr int kThreads = 256;
constexpr int kRowsPerWg = 128;

struct WideParams {
    const void* q; const void* k; const void* v; void* o;
    int64_t q_st, q_sh, k_st, k_sh, v_st, v_sh, o_st, o_sh;    // strides in elements
    const int32_t* cu_seqlens;
    int batch, total_tokens, n_row_groups, num_q_heads, num_kv_heads, head_dim, log2_s;
    float c;                                                   // scale * log2(e)
};

// T: element type of q/k/v/o.  D: 128 or 256, the head width that registers and LDS are laid out for.
template <typename T, int D>
__global__ __launch_bounds__(kThreads, D <= 128 ? 2 : 1) void staircase_attn_f32_kernel(const WideParams P)
{
    extern __shared__ __attribute__((aligned(16))) float lds[];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int H = lane >> 5, r = lane & 31;
    const int head = blockIdx.x;
    const int rg = P.n_row_groups - 1 - (int)blockIdx.y;       // the heaviest row groups start first
    const int b = blockIdx.z;

    // bounds that do not describe a range inside the packed tensors (decreasing, negative, past total_tokens) are clipped
    // to one, so that no row outside q/k/v/o is ever touched
    const int seq0 = min(max(P.cu_seqlens[b], 0), P.total_tokens);
    const int L = min(max(P.cu_seqlens[b + 1], seq0), P.total_tokens) - seq0;
    if (L <= 0) return;
    const int S = 1 << P.log2_s;
    const int Lp = ((L + S - 1) >> P.log2_s) << P.log2_s;      // padded length
    const int pad = Lp - L;
    const int row_g0 = rg * kRowsPerWg;                        // first padded row of the workgroup
    if (row_g0 >= Lp) return;
    const int kvh = head / (P.num_q_heads / P.num_kv_heads);
    const int width = P.head_dim;

    const T* kb = static_cast<const T*>(P.k) + (int64_t)kvh * P.k_sh;
    const T* vb = static_cast<const T*>(P.v) + (int64_t)kvh * P.v_sh;

    // ---- this lane's query ----
    const int row_w0 = row_g0 + wave * 32;
    const int ip = row_w0 + r;                                 // padded query row
    const bool row_ok = ip >= pad && ip < Lp;
    const int64_t tok = (int64_t)seq0 + (ip - pad);
    float q[D / 2];
    load_q<T, D>(q, row_ok ? static_cast<const T*>(P.q) + tok * P.q_st + (int64_t)head * P.q_sh : nullptr, H, width);

    // exclusive key limit (padded coordinates) of a row
    auto limit_of = [&](int row) { return min(Lp, ((row >> P.log2_s) + 1) << P.log2_s); };
    const int key_hi = limit_of(ip);
    const int wave_hi = (row_w0 < Lp) ? limit_of(min(row_w0 + 31, Lp - 1)) : 0;    // 0: idle wavefront
    const int wg_hi = limit_of(min(row_g0 + kRowsPerWg - 1, Lp - 1));
    const int n_tiles = (wg_hi + kTileKeys - 1) / kTileKeys;

    State<D> st;
    st.init();
    for (int t = 0; t < n_tiles; ++t) {
        const int key0 = t * kTileKeys;
        __syncthreads();                                       // the previous tile has been read by everybody
        // ---- K and V rows key0 .. key0 + 31 into LDS as fp32 (rows outside the sequence and padding columns: zeros) ----
#pragma unroll
        for (int p = 0; p < kTileKeys * (D / 4) / kThreads; ++p) {
            const int u = tid + kThreads * p;
            const int row = u / (D / 4), c4 = u % (D / 4);
            const int jp = key0 + row;
            const bool real = jp >= pad && jp < Lp && 4 * c4 < width;
            const int64_t ktok = (int64_t)seq0 + (jp - pad);
            stage4<T, D>(lds, row, c4, real ? kb + ktok * P.k_st + 4 * c4 : nullptr, real ? vb + ktok * P.v_st + 4 * c4 : nullptr);
        }
        __syncthreads();
        if (key0 >= wave_hi || key0 + kTileKeys <= pad) continue;        // nothing of this tile is visible to this wavefront
        tile_step<D>(lds, q, st, P.c, width, lane, [&](int key) { const int kj = key0 + key; return kj >= pad && kj < key_hi; });
    }
    store_o<T, D>(row_ok ? static_cast<T*>(P.o) + tok * P.o_st + (int64_t)head * P.o_sh : nullptr, st, H, width);
}

template <typename T, int D>
int launch(const WideParams& P, hipStream_t stream)
{
    // the kernel's LDS limit is raised once per device
    static std::atomic<bool> raised[64];
    int device = 0;
    hipError_t e = hipGetDevice(&device);
    MDX_REQUIRE(e == hipSuccess && device >= 0 && device < 64, MDX_ELAUNCH, "staircase_attn: no current device (%s)", hipGetErrorString(e));
    if (!raised[device].load(std::memory_order_acquire)) {
        e = hipFuncSetAttribute(reinterpret_cast<const void*>(staircase_attn_f32_kernel<T, D>), hipFuncAttributeMaxDynamicSharedMemorySize, Lds<D>::kBytes);
        MDX_REQUIRE(e == hipSuccess, MDX_ELAUNCH, "staircase_attn: cannot reserve %d bytes of LDS (%s)", Lds<D>::kBytes, hipGetErrorString(e));
        raised[device].store(true, std::memory_order_release);
    }
    const dim3 grid((unsigned)P.num_q_heads, (unsigned)P.n_row_groups, (unsigned)P.batch);
    staircase_attn_f32_kernel<T, D><<<grid, kThreads, Lds<D>::kBytes, stream>>>(P);
    return mdx::check_launch("staircase_attn (fp32 arithmetic)");
}

}  // namespace

namespace mdx {

// Called by mdx_staircase_attn_varlen, which has checked sizes, head counts, staircase size and scale, for
// dtype MDX_F32 and for head widths outside the 16-bit kernels'.
int launch_staircase_f32(const void* q, const void* k, const void* v, void* o,
                         int64_t q_stride_t, int64_t q_stride_h, int64_t k_stride_t, int64_t k_stride_h,
                         int64_t v_stride_t, int64_t v_stride_h, int64_t o_stride_t, int64_t o_stride_h,
                         const int32_t* cu_seqlens, int32_t batch, int64_t max_l, int64_t total_tokens,
                         int32_t num_q_heads, int32_t num_kv_heads, int32_t head_dim,
                         int32_t log2_s, float scale, int32_t dtype, hipStream_t stream)
{
    MDX_REQUIRE(head_dim >= 4 && head_dim <= 256 && head_dim % 4 == 0, MDX_EUNSUPPORTED,
                "staircase_attn: head_dim %d (fp32 arithmetic: multiples of 4 up to 256)", head_dim);
    const uintptr_t align = dtype == MDX_F32 ? 15u : 7u;       // four elements per access
    MDX_REQUIRE((((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)o) & align) == 0 &&
                q_stride_t % 4 == 0 && q_stride_h % 4 == 0 && k_stride_t % 4 == 0 && k_stride_h % 4 == 0 &&
                v_stride_t % 4 == 0 && v_stride_h % 4 == 0 && o_stride_t % 4 == 0 && o_stride_h % 4 == 0,
                MDX_EUNSUPPORTED, "staircase_attn: q/k/v/o must be aligned to four elements with strides that are multiples of 4 elements");
    WideParams P;
    P.q = q; P.k = k; P.v = v; P.o = o;
    P.q_st = q_stride_t; P.q_sh = q_stride_h; P.k_st = k_stride_t; P.k_sh = k_stride_h;
    P.v_st = v_stride_t; P.v_sh = v_stride_h; P.o_st = o_stride_t; P.o_sh = o_stride_h;
    P.cu_seqlens = cu_seqlens;
    P.batch = batch;
    P.total_tokens = (int)total_tokens;
    P.n_row_groups = (int)((max_l + (1 << log2_s) - 1 + kRowsPerWg - 1) / kRowsPerWg);
    P.num_q_heads = num_q_heads; P.num_kv_heads = num_kv_heads; P.head_dim = head_dim; P.log2_s = log2_s;
    P.c = scale * kLog2e;
    MDX_REQUIRE(batch <= 65535 && P.n_row_groups <= 65535, MDX_EUNSUPPORTED,
                "staircase_attn: fp32 arithmetic takes up to 65535 sequences of up to 8 M tokens");
    const bool wide = head_dim > 128;
    switch (dtype) {
    case MDX_F32:  return wide ? launch<float, 256>(P, stream) : launch<float, 128>(P, stream);
    case MDX_F16:  return wide ? launch<_Float16, 256>(P, stream) : launch<_Float16, 128>(P, stream);
    case MDX_BF16: return wide ? launch<__bf16, 256>(P, stream) : launch<__bf16, 128>(P, stream);
    }
    return mdx::fail(MDX_EUNSUPPORTED, "staircase_attn: dtype %d", dtype);
}

}  // namespace mdx
