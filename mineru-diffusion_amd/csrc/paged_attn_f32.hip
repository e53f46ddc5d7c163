// Paged single-block ("decode") attention in fp32 arithmetic: the form of mdx_paged_block_attn for fp32
// tensors and for heads that the 16-bit kernel of paged_attn.hip does not take (wider than 128 columns,
// up to 256, or not a multiple of 16).  flash_attn_with_kvcache, which this call replaces
// (engines/nano_dvlm/nanovllm/layers/sdar_attention.py:48-56), takes heads of up to 256 columns; the model
// itself runs bf16 with d = 128, so this is the path for callers outside the model's own configuration.
// Arithmetic and layout: attn_f32_tile.h.
//
// A workgroup of 4 wavefronts serves one (sequence, KV head, tile of 32 queries): it walks the sequence's
// context once per round of four query heads of that KV head, a wavefront per head, all of them on the same
// K / V tile in LDS.  No split over the keys and no workspace: every output row is written once, by its wavefront.
// The semantics are those of the 16-bit kernel: non-causal, the first min(context_lens[b], max_pages x
// page_size) keys through block_table[b]; keys on a page id outside [0, num_pages) are left out; a sequence
// without any key yields zeros.
#include "attn_f32_tile.h"
#include <atomic>

namespace {

using namespace mdx_attn_f32;

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / 64;

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

template <typename T, int D>
__global__ __launch_bounds__(kThreads, 1) void paged_attn_f32_kernel(const PagedWideParams P)
{
    extern __shared__ __attribute__((aligned(16))) float lds[];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int H = lane >> 5, r = lane & 31;
    const int kvh = blockIdx.x, qt = blockIdx.y, b = blockIdx.z;
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

    for (int h0 = 0; h0 < P.heads_per_kv; h0 += kWaves) {
        const bool active = h0 + wave < P.heads_per_kv;       // uniform per wavefront
        const int head = kvh * P.heads_per_kv + h0 + wave;
        float q[D / 2];
        load_q<T, D>(q, (active && row_ok) ? static_cast<const T*>(P.q) + (int64_t)b * P.q_sb + (int64_t)qrow * P.q_ss + (int64_t)head * P.q_sh : nullptr, H, width);
        State<D> st;
        st.init();
        for (int t = 0; t < n_tiles; ++t) {
            const int key0 = t * kTileKeys;
            // a tile never straddles a page (page_size % 32 == 0): one look-up, uniform
            const int64_t page = bt[key0 / P.page_size];
            const bool page_ok = page >= 0 && page < P.num_pages;
            __syncthreads();                                   // the previous tile has been read by everybody
            if (page_ok) {
                const int64_t base = page * P.c_sp + (int64_t)(key0 % P.page_size) * P.c_st;
#pragma unroll
                for (int p = 0; p < kTileKeys * (D / 4) / kThreads; ++p) {
                    const int u = tid + kThreads * p;
                    const int row = u / (D / 4), c4 = u % (D / 4);
                    const bool real = key0 + row < ctx && 4 * c4 < width;
                    const int64_t off = base + (int64_t)row * P.c_st + 4 * c4;
                    stage4<T, D>(lds, row, c4, real ? kc + off : nullptr, real ? vc + off : nullptr);
                }
            }
            __syncthreads();
            if (page_ok && active)
                tile_step<D>(lds, q, st, P.c, width, lane, [&](int key) { return key0 + key < ctx; });
        }
        if (active)
            store_o<T, D>(row_ok ? static_cast<T*>(P.o) + (int64_t)b * P.o_sb + (int64_t)qrow * P.o_ss + (int64_t)head * P.o_sh : nullptr, st, H, width);
    }
}

template <typename T, int D>
int launch(const PagedWideParams& P, int bs, int num_kv_heads, hipStream_t stream)
{
    // the kernel's LDS limit is raised once per device
    static std::atomic<bool> raised[64];
    int device = 0;
    hipError_t e = hipGetDevice(&device);
    MDX_REQUIRE(e == hipSuccess && device >= 0 && device < 64, MDX_ELAUNCH, "paged_block_attn: no current device (%s)", hipGetErrorString(e));
    if (!raised[device].load(std::memory_order_acquire)) {
        e = hipFuncSetAttribute(reinterpret_cast<const void*>(paged_attn_f32_kernel<T, D>), hipFuncAttributeMaxDynamicSharedMemorySize, Lds<D>::kBytes);
        MDX_REQUIRE(e == hipSuccess, MDX_ELAUNCH, "paged_block_attn: cannot reserve %d bytes of LDS (%s)", Lds<D>::kBytes, hipGetErrorString(e));
        raised[device].store(true, std::memory_order_release);
    }
    const dim3 grid((unsigned)num_kv_heads, (unsigned)((P.sq + 31) / 32), (unsigned)bs);
    paged_attn_f32_kernel<T, D><<<grid, kThreads, Lds<D>::kBytes, stream>>>(P);
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
    MDX_REQUIRE(bs <= 65535 && num_kv_heads <= 65535, MDX_EUNSUPPORTED, "paged_block_attn: fp32 arithmetic takes up to 65535 sequences");
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
    case MDX_F32:  return wide ? launch<float, 256>(P, bs, num_kv_heads, stream) : launch<float, 128>(P, bs, num_kv_heads, stream);
    case MDX_F16:  return wide ? launch<_Float16, 256>(P, bs, num_kv_heads, stream) : launch<_Float16, 128>(P, bs, num_kv_heads, stream);
    case MDX_BF16: return wide ? launch<__bf16, 256>(P, bs, num_kv_heads, stream) : launch<__bf16, 128>(P, bs, num_kv_heads, stream);
    }
    return mdx::fail(MDX_EUNSUPPORTED, "paged_block_attn: dtype %d", dtype);
}

}  // namespace mdx
