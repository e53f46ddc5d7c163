// Paged single-block ("decode") attention: the Sq <= 32 queries of the current
// denoising block of every sequence attend, non-causally, to the first
// context_lens[b] keys of that sequence's paged KV cache.
//
// Replaces flash_attn_with_kvcache(..., causal=False) at
// engines/nano_dvlm/nanovllm/layers/sdar_attention.py:48-56.
//
// The op is HBM-bound (each K/V byte is used by only Sq * Hq/Hkv = 64 query
// rows), so the design goal is to keep the whole chip streaming pages:
//  * split-KV: workgroup (split, head group, sequence) owns `chunk` consecutive
//    keys; there are far more workgroups than the bs*Hkv (sequence, KV head)
//    pairs.  Splits past the context length exit at once.
//  * a workgroup has 8 wavefronts, each owning 32 queries of ONE query head:
//    HPW heads that share a KV head (2 for grouped-query attention) times
//    KW = 8/HPW key slices.  Every tile of 32*KW keys is staged in LDS by one
//    pass of coalesced 16-byte loads and split between the key slices (32 keys
//    per wavefront); the next tile's loads are in flight (in registers) while
//    the current one is consumed.
//  * the KW wavefront states of a head are merged through LDS (a tree), then
//    either written as the final output (single split) or as an fp32 partial
//    (m, l, O) that a second, small kernel combines.
#include "mdx_common.h"
#include "attn_tile.h"
#include <cstdlib>

namespace {

using namespace mdx_attn;

constexpr int kMaxSq = 32;
constexpr int kThreads = 512;      // 8 wavefronts
constexpr int kChunkAlign = 256;   // split boundaries are multiples of this many keys

struct PagedParams {
    const __bf16* q; __bf16* o; const __bf16* k_cache; const __bf16* v_cache;
    int64_t q_sb, q_ss, q_sh, o_sb, o_ss, o_sh;     // element strides
    int64_t c_sp, c_st, c_sh;                       // cache strides: page, token, head
    const int32_t* block_table; int64_t bt_stride;
    const int32_t* context_lens;
    int sq, heads_per_kv, page_size, max_pages;
    int64_t num_pages;
    int chunk, nsplit;                              // keys per split, splits per sequence (grid.x)
    int num_q_heads;
    float c;                                        // scale * log2(e)
    float* part_o; float* part_ml;                  // [bs, Hq, nsplit, 32, 128] and [bs, Hq, nsplit, 2, 32]
};

template <int HPW>
__global__ __launch_bounds__(kThreads) void paged_block_attn_kernel(const PagedParams P)
{
    constexpr int KW = 8 / HPW;                     // key slices (wavefronts per head)
    constexpr int kTileKeys = 32 * KW;
    constexpr int kTileBytes = kTileKeys * kLdsPitch;
    // K and V tiles; the region is reused for the cross-wavefront merge at the end.
    __shared__ __attribute__((aligned(16))) char lds[2 * kTileBytes];
    char* lds_k = lds;
    char* lds_v = lds + kTileBytes;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int H = lane >> 5, r = lane & 31;
    const int split = blockIdx.x, hg = blockIdx.y, b = blockIdx.z;
    const int kw = wave % KW;                       // this wavefront's key slice
    const int head = hg * HPW + wave / KW;          // and query head

    const int ctx = P.context_lens[b];
    const int n_valid_splits = (ctx + P.chunk - 1) / P.chunk;

    if (ctx <= 0) {
        // graph-padding row: defined output (zeros), written by split 0
        if (split == 0) {
            for (int e = tid; e < P.sq * HPW * (kHeadDim / 8); e += kThreads) {
                const int d8 = e % (kHeadDim / 8), h = (e / (kHeadDim / 8)) % HPW, s = e / (kHeadDim / 8) / HPW;
                *reinterpret_cast<u32x4*>(P.o + (int64_t)b * P.o_sb + (int64_t)s * P.o_ss + (int64_t)(hg * HPW + h) * P.o_sh + d8 * 8) = u32x4{0, 0, 0, 0};
            }
        }
        return;
    }
    const int key_begin = split * P.chunk;
    if (key_begin >= ctx) return;
    const int key_end = min(ctx, key_begin + P.chunk);
    const int kvh = (hg * HPW) / P.heads_per_kv;

    const bool row_ok = r < P.sq;
    bf16x8 q[8];
    load_q(q, row_ok ? P.q + (int64_t)b * P.q_sb + (int64_t)r * P.q_ss + (int64_t)head * P.q_sh : nullptr, H);

    WaveState st;
    st.init();

    const int32_t* bt = P.block_table + (int64_t)b * P.bt_stride;
    const int chunk = tid & 15, trow = tid >> 4;    // 512 threads: one pass stages 32 rows
    const int n_tiles = (key_end - key_begin + kTileKeys - 1) / kTileKeys;
    TileRegs<kTileKeys, kThreads> regs;
    // Pass p of a tile holds keys key0 + 32p .. +31: 32 consecutive keys never straddle a page
    // (page_size % 32 == 0, key_begin % 32 == 0), so each pass looks its page up once.
    auto fetch = [&](int t) {
        const int key0 = key_begin + t * kTileKeys;
#pragma unroll
        for (int p = 0; p < KW; ++p) {
            const int kp = key0 + 32 * p;
            bool ok = kp < key_end;
            int64_t page = -1;
            if (ok) {
                const int page_slot = kp / P.page_size;
                page = page_slot < P.max_pages ? (int64_t)bt[page_slot] : -1;
                ok = page >= 0 && page < P.num_pages;
            }
            if (ok && kp + trow < key_end) {
                const int64_t off = page * P.c_sp + (int64_t)(kp % P.page_size + trow) * P.c_st + (int64_t)kvh * P.c_sh + chunk * 8;
                regs.k[p] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(P.k_cache + off));
                regs.v[p] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(P.v_cache + off));
            } else {                                // past the context or an invalid page id: zero rows
                regs.k[p] = u32x4{0, 0, 0, 0};
                regs.v[p] = u32x4{0, 0, 0, 0};
            }
        }
    };
    // Keys of an invalid page are excluded (not merely zeroed): the owning wavefront skips them.
    auto slice_ok = [&](int kp) {
        if (kp >= key_end) return false;
        const int page_slot = kp / P.page_size;
        const int64_t page = page_slot < P.max_pages ? (int64_t)bt[page_slot] : -1;
        return page >= 0 && page < P.num_pages;
    };

    fetch(0);
    for (int t = 0; t < n_tiles; ++t) {
        __syncthreads();
        store_tile<kTileKeys, kThreads>(lds_k, lds_v, regs, tid);
        __syncthreads();
        if (t + 1 < n_tiles) fetch(t + 1);

        const int key0 = key_begin + t * kTileKeys + kw * 32;        // this wavefront's 32 keys
        if (slice_ok(key0)) {
            if (key0 + 32 <= key_end)
                attn_step<1, false>(lds_k, lds_v, kw * 32, q, st, P.c, lane, key0, 0, key_end);
            else
                attn_step<1, true>(lds_k, lds_v, kw * 32, q, st, P.c, lane, key0, 0, key_end);
        }
    }

    // ---- merge the KW key-slice states of each head (tree through LDS) ----------------------
    st.l = both_halves_sum(st.l);          // a state is now (m, l, O) per query
    // Exchange layout per sending wavefront: O as [4][16][64 lanes] floats, then m, l as [64].
    constexpr int kStateFloats = 4 * 16 * 64 + 2 * 64;
    static_assert(4 * kStateFloats * 4 <= (int)sizeof(lds), "merge buffer exceeds the tile region");
    float* xch = reinterpret_cast<float*>(lds);
    auto send = [&](int slot) {
        float* dst = xch + slot * kStateFloats;
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
            for (int i = 0; i < 16; ++i) dst[(t * 16 + i) * 64 + lane] = st.o[t][i];
        dst[4 * 16 * 64 + lane] = st.m;
        dst[4 * 16 * 64 + 64 + lane] = st.l;
    };
    auto recv = [&](int slot) {
        const float* src = xch + slot * kStateFloats;
        const float m2 = src[4 * 16 * 64 + lane];
        const float l2 = src[4 * 16 * 64 + 64 + lane];
        const float M = fmaxf(st.m, m2);
        const float a1 = __builtin_amdgcn_exp2f(st.m - M), a2 = __builtin_amdgcn_exp2f(m2 - M);
        st.l = st.l * a1 + l2 * a2;
        st.m = M;
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
            for (int i = 0; i < 16; ++i)
                st.o[t][i] = st.o[t][i] * a1 + src[(t * 16 + i) * 64 + lane] * a2;
    };
    __syncthreads();                         // tiles no longer needed
#pragma unroll
    for (int stride = KW / 2; stride >= 1; stride >>= 1) {
        const int slot = (wave / KW) * stride + (kw - stride);     // 4 slots at most (HPW * KW/2)
        if (kw >= stride && kw < 2 * stride) send(slot);
        __syncthreads();
        if (kw < stride) recv((wave / KW) * stride + kw);
        __syncthreads();
    }
    if (kw != 0 || !row_ok) return;

    // ---- output ---------------------------------------------------------------
    if (n_valid_splits == 1) {
        const float inv = 1.0f / st.l;
        __bf16* orow = P.o + (int64_t)b * P.o_sb + (int64_t)r * P.o_ss + (int64_t)head * P.o_sh;
#pragma unroll
        for (int dt = 0; dt < 4; ++dt)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
                bf16x4 out;
#pragma unroll
                for (int e = 0; e < 4; ++e) out[e] = (__bf16)(st.o[dt][4 * g + e] * inv);
                *reinterpret_cast<bf16x4*>(orow + d_of_reg(dt, 4 * g, H)) = out;
            }
    } else {
        const int64_t slot = ((int64_t)b * P.num_q_heads + head) * P.nsplit + split;
        float* po = P.part_o + (slot * kMaxSq + r) * kHeadDim;
#pragma unroll
        for (int dt = 0; dt < 4; ++dt)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                float4 out = make_float4(st.o[dt][4 * g], st.o[dt][4 * g + 1], st.o[dt][4 * g + 2], st.o[dt][4 * g + 3]);
                *reinterpret_cast<float4*>(po + d_of_reg(dt, 4 * g, H)) = out;
            }
        if (H == 0) {
            P.part_ml[(slot * 2 + 0) * kMaxSq + r] = st.m;
            P.part_ml[(slot * 2 + 1) * kMaxSq + r] = st.l;
        }
    }
}

// One wavefront per (sequence, head, query): merges the split partials.
__global__ __launch_bounds__(256) void paged_combine_kernel(const PagedParams P, int bs)
{
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int64_t n_rows = (int64_t)bs * P.num_q_heads * P.sq;
    if (row >= n_rows) return;
    const int s = (int)(row % P.sq);
    const int hq = (int)((row / P.sq) % P.num_q_heads);
    const int b = (int)(row / P.sq / P.num_q_heads);
    const int ctx = P.context_lens[b];
    const int nv = (ctx + P.chunk - 1) / P.chunk;
    if (nv <= 1) return;                                   // written directly by the attention kernel
    const int64_t slot0 = ((int64_t)b * P.num_q_heads + hq) * P.nsplit;
    float M = kMinusBig;
    for (int i = 0; i < nv; ++i) M = fmaxf(M, P.part_ml[((slot0 + i) * 2 + 0) * kMaxSq + s]);
    float Lsum = 0.f;
    float2 acc = make_float2(0.f, 0.f);
    for (int i = 0; i < nv; ++i) {
        const float w = __builtin_amdgcn_exp2f(P.part_ml[((slot0 + i) * 2 + 0) * kMaxSq + s] - M);
        Lsum += w * P.part_ml[((slot0 + i) * 2 + 1) * kMaxSq + s];
        const float2 po = *reinterpret_cast<const float2*>(P.part_o + ((slot0 + i) * kMaxSq + s) * kHeadDim + lane * 2);
        acc.x += w * po.x;
        acc.y += w * po.y;
    }
    const float inv = 1.0f / Lsum;
    typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
    bf16x2 out;
    out[0] = (__bf16)(acc.x * inv);
    out[1] = (__bf16)(acc.y * inv);
    *reinterpret_cast<bf16x2*>(P.o + (int64_t)b * P.o_sb + (int64_t)s * P.o_ss + (int64_t)hq * P.o_sh + lane * 2) = out;
}

// Keys per split: enough workgroups to fill 256 CUs a few times over, but no smaller than one page.
int pick_chunk(int bs, int head_groups, int max_pages, int page_size) {
    static const int forced = [] { const char* e = getenv("MDX_PAGED_CHUNK"); return e ? atoi(e) : 0; }();
    if (forced >= kChunkAlign && forced % kChunkAlign == 0) return forced;
    const int64_t max_keys = (int64_t)max_pages * page_size;
    const int64_t target_wgs = 1024;
    int64_t chunk = (int64_t)bs * head_groups * max_keys / target_wgs;
    chunk = (chunk + kChunkAlign - 1) / kChunkAlign * kChunkAlign;
    if (chunk < kChunkAlign) chunk = kChunkAlign;
    if (chunk > max_keys) chunk = (max_keys + kChunkAlign - 1) / kChunkAlign * kChunkAlign;
    return (int)chunk;
}

int nsplit_of(int max_pages, int page_size, int chunk) {
    const int64_t max_keys = (int64_t)max_pages * page_size;
    return (int)((max_keys + chunk - 1) / chunk);
}

}  // namespace

extern "C" int64_t mdx_paged_block_attn_workspace_bytes(int32_t bs, int32_t sq, int32_t num_q_heads,
                                                        int32_t num_kv_heads, int32_t head_dim,
                                                        int32_t max_pages, int32_t page_size)
{
    if (bs <= 0 || num_q_heads <= 0 || num_kv_heads <= 0 || max_pages <= 0 || page_size <= 0) return 0;
    const int G = num_q_heads / num_kv_heads;
    const int HPW = (G % 2 == 0) ? 2 : 1;
    const int chunk = pick_chunk(bs, num_q_heads / HPW, max_pages, page_size);
    const int nsplit = nsplit_of(max_pages, page_size, chunk);
    if (nsplit <= 1) return 0;
    return (int64_t)bs * num_q_heads * nsplit * kMaxSq * (kHeadDim + 2) * (int64_t)sizeof(float);
}

extern "C" int mdx_paged_block_attn(const void* q, void* o, const void* k_cache, const void* v_cache,
                                    int64_t q_stride_b, int64_t q_stride_s, int64_t q_stride_h,
                                    int64_t o_stride_b, int64_t o_stride_s, int64_t o_stride_h,
                                    int64_t cache_stride_page, int64_t cache_stride_tok, int64_t cache_stride_head,
                                    const int32_t* block_table, int64_t bt_stride, const int32_t* context_lens,
                                    int32_t bs, int32_t sq, int32_t num_q_heads, int32_t num_kv_heads,
                                    int32_t head_dim, int32_t max_pages, int32_t page_size, int64_t num_pages,
                                    float scale, int32_t dtype,
                                    void* workspace, int64_t workspace_bytes, mdx_stream_t stream_)
{
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    MDX_REQUIRE(bs >= 0 && sq >= 0 && max_pages >= 0 && num_pages >= 0, MDX_EINVAL, "paged_block_attn: negative size");
    MDX_REQUIRE(dtype == MDX_BF16, MDX_EUNSUPPORTED, "paged_block_attn: dtype %d (only bf16)", dtype);
    MDX_REQUIRE(head_dim == kHeadDim, MDX_EUNSUPPORTED, "paged_block_attn: head_dim %d (only 128)", head_dim);
    MDX_REQUIRE(num_q_heads > 0 && num_kv_heads > 0 && num_q_heads % num_kv_heads == 0, MDX_EINVAL,
                "paged_block_attn: Hq %d not a multiple of Hkv %d", num_q_heads, num_kv_heads);
    MDX_REQUIRE(sq <= kMaxSq, MDX_EUNSUPPORTED, "paged_block_attn: %d queries per sequence (max %d)", sq, kMaxSq);
    MDX_REQUIRE(page_size > 0 && page_size % 32 == 0, MDX_EUNSUPPORTED,
                "paged_block_attn: page_size %d not a multiple of 32", page_size);
    MDX_REQUIRE(scale > 0.f, MDX_EINVAL, "paged_block_attn: scale must be positive");
    if (bs == 0 || sq == 0) return MDX_OK;
    MDX_REQUIRE(max_pages > 0, MDX_EINVAL, "paged_block_attn: empty block table");
    MDX_REQUIRE(q && o && k_cache && v_cache && block_table && context_lens, MDX_EINVAL, "paged_block_attn: null pointer");
    MDX_REQUIRE(bs <= 65535, MDX_EUNSUPPORTED, "paged_block_attn: bs %d > 65535", bs);
    MDX_REQUIRE(bt_stride >= max_pages, MDX_EINVAL, "paged_block_attn: bt_stride < max_pages");
    MDX_REQUIRE(mdx::aligned16(q) && mdx::aligned16(o) && mdx::aligned16(k_cache) && mdx::aligned16(v_cache) &&
                q_stride_b % 8 == 0 && q_stride_s % 8 == 0 && q_stride_h % 8 == 0 &&
                o_stride_b % 8 == 0 && o_stride_s % 8 == 0 && o_stride_h % 8 == 0 &&
                cache_stride_page % 8 == 0 && cache_stride_tok % 8 == 0 && cache_stride_head % 8 == 0,
                MDX_EUNSUPPORTED, "paged_block_attn: tensors must be 16-byte aligned with strides that are multiples of 8 elements");

    const int G = num_q_heads / num_kv_heads;
    const int HPW = (G % 2 == 0) ? 2 : 1;
    PagedParams P;
    P.q = (const __bf16*)q; P.o = (__bf16*)o; P.k_cache = (const __bf16*)k_cache; P.v_cache = (const __bf16*)v_cache;
    P.q_sb = q_stride_b; P.q_ss = q_stride_s; P.q_sh = q_stride_h;
    P.o_sb = o_stride_b; P.o_ss = o_stride_s; P.o_sh = o_stride_h;
    P.c_sp = cache_stride_page; P.c_st = cache_stride_tok; P.c_sh = cache_stride_head;
    P.block_table = block_table; P.bt_stride = bt_stride; P.context_lens = context_lens;
    P.sq = sq; P.heads_per_kv = G; P.page_size = page_size; P.max_pages = max_pages; P.num_pages = num_pages;
    P.chunk = pick_chunk(bs, num_q_heads / HPW, max_pages, page_size);
    P.nsplit = nsplit_of(max_pages, page_size, P.chunk);
    P.num_q_heads = num_q_heads;
    P.c = scale * kLog2e;
    P.part_o = nullptr; P.part_ml = nullptr;
    if (P.nsplit > 1) {
        const int64_t n_slots = (int64_t)bs * num_q_heads * P.nsplit;
        const int64_t need = n_slots * kMaxSq * (kHeadDim + 2) * (int64_t)sizeof(float);
        MDX_REQUIRE(workspace && workspace_bytes >= need, MDX_EWORKSPACE,
                    "paged_block_attn: workspace of %lld bytes needed, %lld given", (long long)need, (long long)workspace_bytes);
        MDX_REQUIRE(mdx::aligned16(workspace), MDX_EWORKSPACE, "paged_block_attn: workspace not 16-byte aligned");
        P.part_o = static_cast<float*>(workspace);
        P.part_ml = P.part_o + n_slots * kMaxSq * kHeadDim;
    }
    const dim3 grid((unsigned)P.nsplit, (unsigned)(num_q_heads / HPW), (unsigned)bs);
    if (HPW == 2) paged_block_attn_kernel<2><<<grid, kThreads, 0, stream>>>(P);
    else          paged_block_attn_kernel<1><<<grid, kThreads, 0, stream>>>(P);
    int rc = mdx::check_launch("paged_block_attn");
    if (rc != MDX_OK || P.nsplit == 1) return rc;
    const int64_t n_rows = (int64_t)bs * num_q_heads * sq;
    paged_combine_kernel<<<(unsigned)((n_rows + 3) / 4), 256, 0, stream>>>(P, bs);
    return mdx::check_launch("paged_combine");
}
