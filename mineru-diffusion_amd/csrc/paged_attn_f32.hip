// Paged single-block ("decode") attention in fp32 arithmetic: the form of mdx_paged_block_attn for fp32
// tensors and for heads that the 16-bit kernel of paged_attn.hip does not take (wider than 128 columns,
// up to 256, or not a multiple of 16).  flash_attn_with_kvcache, which this call replaces
// (engines/nano_dvlm/nanovllm/layers/sdar_attention.py:48-56), takes heads of up to 256 columns; the model
// itself runs bf16 with d = 128, so this is the path for callers outside the model's own configuration.
// Arithmetic and layout: attn_f32_tile.h.
//
// A workgroup serves one (sequence, query head, tile of 32 queries).  Its NW wavefronts (4 for heads of up to 128
// columns, 2 for wider ones: what fits in LDS) take consecutive tiles of 32 keys, NW tiles staged at a time, each
// wavefront with its own running softmax state; at the end the states are merged through LDS and every wavefront
// writes its share of the head's columns.  No split over workgroups and no workspace.
// The semantics are those of the 16-bit kernel: non-causal, the first min(context_lens[b], max_pages x
// page_size) keys through block_table[b]; keys on a page id outside [0, num_pages) are left out; a sequence
// without any key yields zeros.
#include "attn_f32_tile.h"
#include <atomic>

namespace {

using namespace mdx_attn_f32;

struct PagedWideParams {
    const void* q; void* o; const void* k_cache; const void* v_cache;
    int64_t q_sb, q_ss, q_sh, o_sb, o_ss, o_sh;     // element strides
    int64_t c_sp, c_st, c_sh;                       // cache strides: page, token, head
    const int32_t* block_table; int64_t bt_stride;
    const int32_t* context_lens;
    int sq, heads_per_kv, page_size, max_pages, head_dim;
    int64_t num_pages;
    float c;                                        // scale * log2(e)
};

template <typename T, int D, int NW>
__global__ __launch_bounds__(64 * NW, 1) void paged_attn_f32_kernel(const PagedWideParams P)
{
    constexpr int kThreads = 64 * NW;
    constexpr int kTileFloats = Lds<D>::kFloats;
    extern __shared__ __attribute__((aligned(16))) float lds[];          // NW tiles (K and V of 32 keys each)

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int H = lane >> 5, r = lane & 31;
    const int head = blockIdx.x, qt = blockIdx.y, b = blockIdx.z;
    const int kvh = head / P.heads_per_kv;
    const int width = P.head_dim;

    const int64_t room = (int64_t)P.max_pages * P.page_size;
    const int ctx_raw = P.context_lens[b];
    const int ctx = (int)(ctx_raw < room ? ctx_raw : room);
    const int32_t* bt = P.block_table + (int64_t)b * P.bt_stride;
    const int n_tiles = ctx > 0 ? (ctx + kTileKeys - 1) / kTileKeys : 0;

    const int qrow = qt * 32 + r;                   // this lane's query of the sequence's block
    const bool row_ok = qrow < P.sq;
    const T* kc = static_cast<const T*>(P.k_cache) + (int64_t)kvh * P.c_sh;
    const T* vc = static_cast<const T*>(P.v_cache) + (int64_t)kvh * P.c_sh;

    float q[D / 2];
    load_q<T, D>(q, row_ok ? static_cast<const T*>(P.q) + (int64_t)b * P.q_sb + (int64_t)qrow * P.q_ss + (int64_t)head * P.q_sh : nullptr, H, width);
    State<D> st;
    st.init();
    for (int t0 = 0; t0 < n_tiles; t0 += NW) {
        __syncthreads();                                       // the previous tiles have been read by everybody
        // ---- tiles t0 .. t0 + NW - 1 into LDS, all threads on each (a tile never straddles a page: page_size % 32 == 0) ----
        unsigned tile_ok = 0;                                  // bit i: tile t0 + i exists and lies on a valid page (uniform)
#pragma unroll
        for (int i = 0; i < NW; ++i) {
            const int key0 = (t0 + i) * kTileKeys;
            if (key0 >= ctx) break;
            const int64_t page = bt[key0 / P.page_size];
            if (page < 0 || page >= P.num_pages) continue;
            tile_ok |= 1u << i;
            const int64_t base = page * P.c_sp + (int64_t)(key0 % P.page_size) * P.c_st;
#pragma unroll
            for (int p = 0; p < kTileKeys * (D / 4) / kThreads; ++p) {
                const int u = tid + kThreads * p;
                const int row = u / (D / 4), c4 = u % (D / 4);
                const bool real = key0 + row < ctx && 4 * c4 < width;
                const int64_t off = base + (int64_t)row * P.c_st + 4 * c4;
                stage4<T, D>(lds + i * kTileFloats, row, c4, real ? kc + off : nullptr, real ? vc + off : nullptr);
            }
        }
        __syncthreads();
        if ((tile_ok >> wave) & 1u) {
            const int key0 = (t0 + wave) * kTileKeys;
            tile_step<D>(lds + wave * kTileFloats, q, st, P.c, width, lane, [&](int key) { return key0 + key < ctx; });
        }
    }

    // ---- merge the NW states through LDS: every wavefront folds, and stores, the column tiles dt = wave, wave + NW, ... ----
    constexpr int kStateFloats = (D / 32) * 16 * 64 + 2 * 64;                  // O as [dt][register][lane], then m, l
    static_assert(NW * kStateFloats <= NW * kTileFloats, "merge buffer exceeds the tile region");
    st.l += __shfl_xor(st.l, 32);                                              // a state is now (m, l, O) per query
    __syncthreads();                                                           // the last tiles have been read by everybody
    {
        float* dst = lds + wave * kStateFloats;
#pragma unroll
        for (int dt = 0; dt < D / 32; ++dt)
#pragma unroll
            for (int i = 0; i < 16; ++i) dst[(dt * 16 + i) * 64 + lane] = st.o[dt][i];
        dst[(D / 32) * 16 * 64 + lane] = st.m;
        dst[(D / 32) * 16 * 64 + 64 + lane] = st.l;
    }
    __syncthreads();
    float w[NW];
    float M = kMinusBig, l_all = 0.f;
#pragma unroll
    for (int s = 0; s < NW; ++s) { w[s] = lds[s * kStateFloats + (D / 32) * 16 * 64 + lane]; M = fmaxf(M, w[s]); }
#pragma unroll
    for (int s = 0; s < NW; ++s) {
        w[s] = __builtin_amdgcn_exp2f(w[s] - M);
        l_all += lds[s * kStateFloats + (D / 32) * 16 * 64 + 64 + lane] * w[s];
    }
    if (!row_ok) return;
    const float inv = l_all > 0.f ? 1.0f / l_all : 0.f;                        // no key at all: zeros
    T* orow = static_cast<T*>(P.o) + (int64_t)b * P.o_sb + (int64_t)qrow * P.o_ss + (int64_t)head * P.o_sh;
#pragma unroll
    for (int dt = 0; dt < D / 32; ++dt) {
        if (dt % NW != wave || dt * 32 >= width) continue;                     // (uniform per wavefront)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int s = 0; s < NW; ++s)
#pragma unroll
                for (int e = 0; e < 4; ++e) acc[e] += lds[s * kStateFloats + (dt * 16 + 4 * g + e) * 64 + lane] * w[s];
            const int d = dt * 32 + 8 * g + 4 * H;
            if (d < width) store4(orow + d, f32x4{acc[0] * inv, acc[1] * inv, acc[2] * inv, acc[3] * inv});
        }
    }
}

template <typename T, int D>
int launch(const PagedWideParams& P, int bs, int num_q_heads, hipStream_t stream)
{
    constexpr int NW = D <= 128 ? 4 : 2;            // tiles of 32 keys that fit in LDS side by side
    constexpr int kLdsBytes = NW * Lds<D>::kBytes;
    // the kernel's LDS limit is raised once per device
    static std::atomic<bool> raised[64];
    int device = 0;
    hipError_t e = hipGetDevice(&device);
    MDX_REQUIRE(e == hipSuccess && device >= 0 && device < 64, MDX_ELAUNCH, "paged_block_attn: no current device (%s)", hipGetErrorString(e));
    if (!raised[device].load(std::memory_order_acquire)) {
        e = hipFuncSetAttribute(reinterpret_cast<const void*>(paged_attn_f32_kernel<T, D, NW>), hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes);
        MDX_REQUIRE(e == hipSuccess, MDX_ELAUNCH, "paged_block_attn: cannot reserve %d bytes of LDS (%s)", kLdsBytes, hipGetErrorString(e));
        raised[device].store(true, std::memory_order_release);
    }
    const dim3 grid((unsigned)num_q_heads, (unsigned)((P.sq + 31) / 32), (unsigned)bs);
    paged_attn_f32_kernel<T, D, NW><<<grid, 64 * NW, kLdsBytes, stream>>>(P);
    return mdx::check_launch("paged_block_attn (fp32 arithmetic)");
}

}  // namespace

namespace mdx {

// Called by the launch behind every paged entry point, which has checked sizes, head counts, the page size
// (a multiple of 32), the scale and the pointers, for dtype MDX_F32 and for head widths outside the 16-bit kernel's.
int launch_paged_f32(const void* q, void* o, const void* k_cache, const void* v_cache,
                     int64_t q_stride_b, int64_t q_stride_s, int64_t q_stride_h,
                     int64_t o_stride_b, int64_t o_stride_s, int64_t o_stride_h,
                     int64_t cache_stride_page, int64_t cache_stride_tok, int64_t cache_stride_head,
                     const int32_t* block_table, int64_t bt_stride, const int32_t* context_lens,
                     int32_t bs, int32_t sq, int32_t num_q_heads, int32_t num_kv_heads,
                     int32_t head_dim, int32_t max_pages, int32_t page_size, int64_t num_pages,
                     float scale, int32_t dtype, hipStream_t stream)
{
    MDX_REQUIRE(head_dim >= 4 && head_dim <= 256 && head_dim % 4 == 0, MDX_EUNSUPPORTED,
                "paged_block_attn: head_dim %d (fp32 arithmetic: multiples of 4 up to 256)", head_dim);
    const uintptr_t align = dtype == MDX_F32 ? 15u : 7u;       // four elements per access
    MDX_REQUIRE((((uintptr_t)q | (uintptr_t)o | (uintptr_t)k_cache | (uintptr_t)v_cache) & align) == 0 &&
                q_stride_b % 4 == 0 && q_stride_s % 4 == 0 && q_stride_h % 4 == 0 &&
                o_stride_b % 4 == 0 && o_stride_s % 4 == 0 && o_stride_h % 4 == 0 &&
                cache_stride_page % 4 == 0 && cache_stride_tok % 4 == 0 && cache_stride_head % 4 == 0,
                MDX_EUNSUPPORTED, "paged_block_attn: tensors must be aligned to four elements with strides that are multiples of 4 elements");
    MDX_REQUIRE(bs <= 65535 && num_q_heads <= 65535, MDX_EUNSUPPORTED, "paged_block_attn: fp32 arithmetic takes up to 65535 sequences");
    PagedWideParams P;
    P.q = q; P.o = o; P.k_cache = k_cache; P.v_cache = v_cache;
    P.q_sb = q_stride_b; P.q_ss = q_stride_s; P.q_sh = q_stride_h;
    P.o_sb = o_stride_b; P.o_ss = o_stride_s; P.o_sh = o_stride_h;
    P.c_sp = cache_stride_page; P.c_st = cache_stride_tok; P.c_sh = cache_stride_head;
    P.block_table = block_table; P.bt_stride = bt_stride; P.context_lens = context_lens;
    P.sq = sq; P.heads_per_kv = num_q_heads / num_kv_heads; P.page_size = page_size; P.max_pages = max_pages; P.head_dim = head_dim;
    P.num_pages = num_pages;
    P.c = scale * kLog2e;
    const bool wide = head_dim > 128;
    switch (dtype) {
    case MDX_F32:  return wide ? launch<float, 256>(P, bs, num_q_heads, stream) : launch<float, 128>(P, bs, num_q_heads, stream);
    case MDX_F16:  return wide ? launch<_Float16, 256>(P, bs, num_q_heads, stream) : launch<_Float16, 128>(P, bs, num_q_heads, stream);
    case MDX_BF16: return wide ? launch<__bf16, 256>(P, bs, num_q_heads, stream) : launch<__bf16, 128>(P, bs, num_q_heads, stream);
    }
    return mdx::fail(MDX_EUNSUPPORTED, "paged_block_attn: dtype %d", dtype);
}

}  // namespace mdx
