// Paged single-block ("decode") attention: the Sq <= 128 queries of the current
// denoising block of every sequence attend, non-causally, to the first
// context_lens[b] keys of that sequence's paged KV cache.  A workgroup serves one
// tile of 32 queries; blocks of 64 or 128 positions (the reference's block length
// is a configuration field, nanovllm/config.py:48) run as 2 or 4 query tiles,
// each a workgroup with its own partials and arrival counter; they stream the
// same keys and are launched next to each other, 8 workgroups apart, so that
// they run on one XCD and the later ones find in its L2 what the first fetched.
//
// Replaces flash_attn_with_kvcache(..., causal=False) at
// engines/nano_dvlm/nanovllm/layers/sdar_attention.py:48-56.
//
// The op is HBM-bound (each K/V byte is used by only Sq * Hq/Hkv = 64 query
// rows), so the design goal is to keep the whole chip streaming pages:
//  * split-KV: a workgroup owns one split of consecutive keys of one sequence
//    for one group of query heads; the split size is chosen so that there are
//    1.5 to 1.8 workgroups per CU (pick_chunk), and with a (sequence, KV head)
//    pair per CU sequences stay whole unless the kernel finds one far longer
//    than the mean.  Workgroups are numbered densely over the
//    (sequence, split) pairs that exist (lane b of each wavefront holds the
//    split count of sequence b), so the launch order has no holes: the
//    dispatcher deals consecutive workgroups round-robin to XCDs and shader
//    engines and stalls on a full one, which punishes interleaved no-op groups.
//  * a workgroup has 4 wavefronts, each owning 32 queries of ONE query head:
//    HPW heads that share a KV head (2 for grouped-query attention) times
//    KW = 4/HPW key slices of 32 keys.  Two workgroups share a CU.
//  * K/V tiles of 32*KW keys travel global -> registers -> LDS with 16-byte
//    coalesced loads into two register sets while a third tile is consumed from
//    the double-buffered LDS.  (As compiled, a stage waits for every load the
//    wavefront has outstanding, because the fetch of the younger tile sits under
//    a condition; making all fetches unconditional, so that the wait leaves the
//    younger tile in flight, was measured and changes nothing: the depth of the
//    load queue is not what bounds this kernel.)
//  * the KW wavefront states of a head are merged through LDS, then either
//    written as the final output (single split) or as an fp32 partial
//    (m, l, O) that a second, small kernel combines.
#include "mdx_common.h"
#include "attn_tile.h"
#include <atomic>

namespace {

using namespace mdx_attn;

constexpr int kQTile = 32;          // queries per workgroup (one per lane pair of a wavefront)
constexpr int kMaxSq = 128;         // queries per sequence: up to four query tiles
constexpr int kChunkAlign = 256;   // the host's split sizes are multiples of this many keys

// Sum over the 64 lanes: DPP shifts inside the rows of 16 lanes, the two row broadcasts, the total from lane 63
// (six additions, no LDS traffic: the butterfly of cross-lane LDS permutes it replaces sat in every workgroup's start).
__device__ __forceinline__ int wave_sum(int x) {
    int v = x;
    v += __builtin_amdgcn_update_dpp(0, v, 0x111, 0xf, 0xf, false);   // row_shr:1
    v += __builtin_amdgcn_update_dpp(0, v, 0x112, 0xf, 0xf, false);   // row_shr:2
    v += __builtin_amdgcn_update_dpp(0, v, 0x114, 0xf, 0xf, false);   // row_shr:4
    v += __builtin_amdgcn_update_dpp(0, v, 0x118, 0xf, 0xf, false);   // row_shr:8
    v += __builtin_amdgcn_update_dpp(0, v, 0x142, 0xa, 0xf, false);   // row_bcast:15 into rows 1 and 3
    v += __builtin_amdgcn_update_dpp(0, v, 0x143, 0xc, 0xf, false);   // row_bcast:31 into rows 2 and 3
    return __builtin_amdgcn_readlane(v, 63);
}

__device__ __forceinline__ int wave_max(int x) {                         // same pattern; x >= 0
    int v = x;
    v = max(v, __builtin_amdgcn_update_dpp(0, v, 0x111, 0xf, 0xf, false));
    v = max(v, __builtin_amdgcn_update_dpp(0, v, 0x112, 0xf, 0xf, false));
    v = max(v, __builtin_amdgcn_update_dpp(0, v, 0x114, 0xf, 0xf, false));
    v = max(v, __builtin_amdgcn_update_dpp(0, v, 0x118, 0xf, 0xf, false));
    v = max(v, __builtin_amdgcn_update_dpp(0, v, 0x142, 0xa, 0xf, false));
    v = max(v, __builtin_amdgcn_update_dpp(0, v, 0x143, 0xc, 0xf, false));
    return __builtin_amdgcn_readlane(v, 63);
}

// Partials that another workgroup of the same launch reads (single-launch merge) travel with
// agent-scope accesses: such a store is written through to memory and such a load does not take a line
// that this XCD's L2 may still hold from an earlier launch.  That makes them visible across the XCDs'
// L2 caches without the release fence (a write-back walk of the whole L2) that ordinary stores would need.
typedef __attribute__((ext_vector_type(4))) float f32x4;
__device__ __forceinline__ void store_agent(float* p, f32x4 v) {
    asm volatile("global_store_dwordx4 %0, %1, off sc1" :: "v"(p), "v"(v) : "memory");
}
__device__ __forceinline__ f32x4 load_agent(const float* p) {
    f32x4 v;
    asm volatile("global_load_dwordx4 %0, %1, off sc1" : "=v"(v) : "v"(p) : "memory");
    return v;
}
__device__ __forceinline__ void wait_vector_memory() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

struct PagedParams {
    const __bf16* q; __bf16* o; const __bf16* k_cache; const __bf16* v_cache;
    int64_t q_sb, q_ss, q_sh, o_sb, o_ss, o_sh;     // element strides
    int64_t c_sp, c_st, c_sh;                       // cache strides: page, token, head
    const int32_t* block_table; int64_t bt_stride;
    const int32_t* context_lens;
    int bs, sq, heads_per_kv, page_size, page_shift, max_pages;   // page_shift: log2(page_size) or -1
    int64_t num_pages;
    int chunk, nsplit;                              // keys per split, max splits per sequence
    int nqt;                                        // query tiles of 32 per sequence (grid z)
    int num_q_heads;
    int head_dim;                                   // <= 128, a multiple of 16: columns beyond it are zeros in LDS and never stored
    float c;                                        // scale * log2(e)
    float* part_o; float* part_ml;                  // [bs, Hq, nqt, nsplit, 32, 128] and [bs, Hq, nqt, nsplit, 2, 32]
    // non-null: the attention kernel picks the split size (>= chunk) from the lengths and leaves it
    // here for the combine kernel.  A float on purpose: an int store in the attention kernel could
    // alias the int page table and lengths for the compiler, which would then stop fetching those
    // through the scalar cache and wait on the vector-memory counter for them, draining the K/V
    // prefetch queue (measured: 78 -> 120 us).  Split sizes are far below 2^24, so the value is exact.
    float* span_out;
    // > 0: every sequence is cut (fewer (sequence, head group) pairs than the chip holds workgroups) and the host's
    // split assumes page tables that are 65 % full.  The attention kernel, which sees the lengths, starts from the
    // split that fills the chip when the tables are emptier, grows it by a tile at a time until the launch fits this
    // many resident workgroups -- one round, nobody starts late -- and leaves the split it settled on in span_out.  (Full tables: 16 sequences of 4128 keys 69 -> 60 us, 16 of
    // 1000 to 3000 keys in a table 12 pages wide 51 -> 42 us; no shape of the sweep slower.  Cutting each sequence
    // into equal pieces instead of full splits and a short remainder was measured too and loses: the remainders
    // start last and fill the tail.)
    int fit_slots;
    // Single-launch mode: one arrival counter per (sequence, head group), zero between launches.  The
    // last split of a pair to arrive merges the pair's partials itself.  float for the same reason.
    float* arrive;
};

// Merges the nv split partials of query s of (sequence b, head hq); the caller's 8 threads c = 0..7
// of a query take 16 consecutive d values each.  nv comes from `count()`, which is asked only after the
// loads of the first four slots are on their way: where those slots lie does not depend on it (slots
// beyond nv hold leftovers and are masked out), so a caller whose split count is still in flight from
// memory overlaps that latency with the partials'.
template <typename E, bool AGENT, typename Count>
__device__ __forceinline__ void combine_query(const PagedParams& P, int b, int hq, int qt, int s, int c, Count count)
{
    if (c * 16 >= P.head_dim) return;
    const int64_t slot0 = (((int64_t)b * P.num_q_heads + hq) * P.nqt + qt) * P.nsplit;
    int nv = P.nsplit;                         // until count() is in: every slot that exists
    float M = kMinusBig, Lsum = 0.f;
    float acc[16];
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[e] = 0.f;
    for (int i0 = 0; i0 < nv; i0 += 4) {
        float m[4], l[4];
        f32x4 po[4][4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int64_t slot = slot0 + min(i0 + i, P.nsplit - 1);
            const float* ml = P.part_ml + (slot * 2 + 0) * kQTile + s;
            const float* src = P.part_o + (slot * kQTile + s) * kHeadDim + c * 16;
            if (AGENT) {
                m[i] = __hip_atomic_load(ml, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                l[i] = __hip_atomic_load(ml + kQTile, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
                for (int k = 0; k < 4; ++k) po[i][k] = load_agent(src + 4 * k);
            } else {
                m[i] = ml[0];
                l[i] = ml[kQTile];
#pragma unroll
                for (int k = 0; k < 4; ++k) po[i][k] = *reinterpret_cast<const f32x4*>(src + 4 * k);
            }
        }
        if (AGENT) {
            // the asm loads are invisible to the compiler's own counting: wait here, and tie every loaded
            // value to the wait so that no use of it can be scheduled above it
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int k = 0; k < 4; ++k) asm volatile("s_waitcnt vmcnt(0)" : "+v"(po[i][k]) :: "memory");
        }
        if (i0 == 0) {
            nv = count();
            if (nv <= 1) return;               // written directly by the attention kernel
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) m[i] = i0 + i < nv ? m[i] : kMinusBig;
        const float Mn = fmaxf(fmaxf(fmaxf(m[0], m[1]), fmaxf(m[2], m[3])), M);
        const float keep = __builtin_amdgcn_exp2f(M - Mn);
        Lsum *= keep;
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[e] *= keep;
        M = Mn;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const bool on = i0 + i < nv;
            const float w = on ? __builtin_amdgcn_exp2f(m[i] - M) : 0.f;
            Lsum += on ? w * l[i] : 0.f;
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                acc[4 * k + 0] += on ? w * po[i][k].x : 0.f;
                acc[4 * k + 1] += on ? w * po[i][k].y : 0.f;
                acc[4 * k + 2] += on ? w * po[i][k].z : 0.f;
                acc[4 * k + 3] += on ? w * po[i][k].w : 0.f;
            }
        }
    }
    const float inv = Lsum > 0.f ? 1.0f / Lsum : 0.f;   // no valid key at all (every page id invalid): zeros, like a context of 0
    typedef typename Elem16<E>::vec8 vec8;
    __bf16* dst = P.o + (int64_t)b * P.o_sb + (int64_t)(qt * kQTile + s) * P.o_ss + (int64_t)hq * P.o_sh + c * 16;
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        vec8 out;
#pragma unroll
        for (int e = 0; e < 8; ++e) out[e] = (E)(acc[8 * h + e] * inv);
        *reinterpret_cast<vec8*>(dst + 8 * h) = out;
    }
}

// WAVES = 4 (two workgroups per CU) or 8 (one workgroup per CU, 128-key tiles: for launches with about
// one workgroup per CU, where a CU would otherwise hold four wavefronts only).  Tiles hold 32 keys per
// key slice (WAVES / HPW slices); two 64-key tile buffers fit a CU twice, two 128-key ones once.
template <typename E, int HPW, int DEPTH, int WAVES>
__global__ __launch_bounds__(64 * WAVES, (WAVES / HPW == 2) ? 2 : 1) void paged_block_attn_kernel(const PagedParams P)
{
    constexpr int kThreads = 64 * WAVES;
    constexpr int kRowsPerPass = kThreads / 16;     // LDS rows one pass of the workgroup stages
    constexpr int kPassesPerSlice = 32 / kRowsPerPass;
    constexpr int KW = WAVES / HPW;                 // key slices (wavefronts per head)
    constexpr int kTileKeys = 32 * KW;
    constexpr int kTileBytes = kTileKeys * kLdsPitch;
    constexpr int kPasses = TileRegs<kTileKeys, kThreads>::kPasses;   // 16 rows per pass
    // [buffer][K tile, V tile]; the region is reused for the cross-wavefront merge at the end.
    __shared__ __attribute__((aligned(16))) char lds[2][2 * kTileBytes];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int H = lane >> 5, r = lane & 31;
    // launch order: head group fastest, then the query tiles of a (sequence, split), then the pairs -- the tiles of a
    // block longer than 32 queries stream the same keys, so they start next to each other and on the same XCD
    const int n_groups = P.num_q_heads / HPW;
    const int hg = blockIdx.x % n_groups;
    const int qt = blockIdx.x / n_groups;           // this workgroup's tile of 32 queries
    const int kw = wave % KW;                       // this wavefront's key slice
    const int head = hg * HPW + wave / KW;          // and query head

    // ---- workgroup -> (sequence b, split) ------------------------------------------------------
    int b, split, span = P.chunk;
    int ctx_all = 0;                                // (up to 64 sequences) the clipped length of sequence `lane`
    if (P.bs <= 64) {
        // lengths beyond the page table name keys that do not exist: clipped here and below
        const int ctx_l = lane < P.bs ? min(max(0, P.context_lens[lane]), P.max_pages * P.page_size) : 0;
        ctx_all = ctx_l;
        auto splits_of_lane = [&]() { return lane < P.bs ? max(1, (ctx_l + span - 1) / span) : 0; };   // (padding rows get one)
        int n;
        if (P.fit_slots > 0) {
            // Tables emptier than assumed: start from the split that would fill the chip, total / (resident workgroups
            // per head group - a remainder of half a split per sequence) -- at least 512 keys (256 where even pieces
            // that short leave half of the chip's workgroup slots empty: a launch that small is a chain of
            // latencies, and the chain is as long as its longest workgroup), no more pieces per sequence than the
            // launch has room for, and not so many that the combine pass, which walks a sequence's pieces four at a
            // time, costs more than shorter pieces save (0.6 us per piece against 0.022 us per key of the longest
            // workgroup: pieces of sqrt(27.6 x longest) keys balance the two; a sequence of tens of thousands of
            // keys grows its split by the same rule).  A sequence that the host's split leaves whole is only cut
            // if that takes 256 keys or more off the longest workgroup (what the combine pass and the partials cost).
            // (Quotients by reciprocal: an estimate is all that is needed, and every workgroup makes the same one;
            // the "+ 1" keeps the longest sequence within nsplit pieces whatever the rounding.)
            const int total = wave_sum(ctx_l), longest = wave_max(ctx_l), live = wave_sum(ctx_l > 0 ? 1 : 0);
            const float per_group = (float)P.fit_slots * __builtin_amdgcn_rcpf((float)gridDim.x);      // resident workgroups per head group and query tile
            const float room = fmaxf(1.f, per_group - 0.5f * (float)live);
            const float least = (float)total * (1.f / 256.f) + (float)live <= 0.5f * per_group ? 256.f : 512.f;
            const float depth = __builtin_amdgcn_sqrtf(27.6f * (float)longest);
            const float want = fmaxf(fmaxf(least, (float)total * __builtin_amdgcn_rcpf(room)),
                                     fmaxf((float)longest * __builtin_amdgcn_rcpf((float)P.nsplit) + 1.f, depth));
            const int fill = ((int)want + 63) & ~63;
            if (min(longest, span) - fill >= (longest > span ? 64 : 256)) span = fill;
            span = max(span, ((int)depth + 63) & ~63);
            n = splits_of_lane();
            // a tile more per step (24 steps double the smallest split); a few workgroups beyond what is resident
            // may stay: the last to start are remainders, which fill the tail
            for (int it = 0; it < 24 && wave_sum(n) * (int)gridDim.x > P.fit_slots + P.fit_slots / 32; ++it) {
                span += 64;
                n = splits_of_lane();
            }
            if (blockIdx.x == 0 && blockIdx.y == 0 && tid == 0) *P.span_out = (float)span;
        } else {
            if (P.span_out) {
                // With a (sequence, head group) pair per CU the sequences are best left whole (no partials,
                // nothing to combine) -- unless one of them is much longer than the rest and would keep
                // its CU busy long after the others are done.  Only the device knows the lengths: the
                // split grows from the host's size to 1.25 x the mean length, so that only sequences
                // well above the mean are cut, into pieces of about the mean.
                const int live = wave_sum(ctx_l > 0 ? 1 : 0);
                const int mean = wave_sum(ctx_l) / max(live, 1);
                span = max(span, (mean + mean / 4 + kChunkAlign - 1) / kChunkAlign * kChunkAlign);
                if (blockIdx.x == 0 && blockIdx.y == 0 && tid == 0) *P.span_out = (float)span;
            }
            n = splits_of_lane();
        }
        // Launch order: the first split of every sequence, then the second of those that have one, ...
        // The last split of a sequence is its short remainder, so the workgroups that start late
        // (when there are more of them than the chip holds at once) are the short ones.
        int j = blockIdx.y, level = 0;
        b = -1;
        for (; level < P.nsplit; ++level) {
            const unsigned long long has = __ballot(n > level);
            const int c = __popcll(has);
            if (j < c) {
                const int before = __popcll(has & ((1ull << lane) - 1ull));
                const unsigned long long hit = __ballot(((has >> lane) & 1ull) != 0 && before == j);
                b = __ffsll((long long)hit) - 1;
                break;
            }
            j -= c;
        }
        if (b < 0) return;                          // past the last (sequence, split) pair
        split = level;
    } else {
        b = blockIdx.y / P.nsplit;
        split = blockIdx.y % P.nsplit;
    }
    const int ctx = P.bs <= 64 ? __builtin_amdgcn_readlane(ctx_all, b)       // lane b read it above: no second trip to memory
                               : min(P.context_lens[b], P.max_pages * P.page_size);
    const int n_valid_splits = (ctx + span - 1) / span;
    if (ctx <= 0) {
        // graph-padding row: defined output (zeros), written by its split 0
        if (split == 0 && qt == 0) {
            for (int e = tid; e < P.sq * HPW * (kHeadDim / 8); e += kThreads) {
                const int d8 = e % (kHeadDim / 8), h = (e / (kHeadDim / 8)) % HPW, s = e / (kHeadDim / 8) / HPW;
                if (d8 * 8 < P.head_dim) *reinterpret_cast<u32x4*>(P.o + (int64_t)b * P.o_sb + (int64_t)s * P.o_ss + (int64_t)(hg * HPW + h) * P.o_sh + d8 * 8) = u32x4{0, 0, 0, 0};
            }
        }
        return;
    }
    const int key_begin = split * span;
    if (key_begin >= ctx) return;
    const int key_end = min(ctx, key_begin + span);
    const int kvh = (hg * HPW) / P.heads_per_kv;

    const int qrow = qt * kQTile + r;               // this lane's query of the sequence's block
    const bool row_ok = qrow < P.sq;
    typename Elem16<E>::vec8 q[1][8];
    load_q(q[0], row_ok ? P.q + (int64_t)b * P.q_sb + (int64_t)qrow * P.q_ss + (int64_t)head * P.q_sh : nullptr, H, P.head_dim);

    WaveState<1> st;
    st.init();

    const int32_t* bt = P.block_table + (int64_t)b * P.bt_stride;
    const int chunk = tid & 15, trow = tid >> 4;    // one pass stages kRowsPerPass rows
    const int n_tiles = (key_end - key_begin + kTileKeys - 1) / kTileKeys;
    // kRowsPerPass (16 or 32) consecutive keys starting at a multiple of that never straddle a page (page_size % 32 == 0):
    // each pass looks its page up once.  The loads of a fetch are unconditional (rows past the context
    // or on an invalid page id read row `trow` of page 0 instead and are zeroed when they reach LDS).
    struct Staged {
        TileRegs<kTileKeys, kThreads> regs;
        unsigned row_ok;       // bit p: this thread's row of pass p holds a real key
        unsigned pass_ok;      // bit p (uniform): pass p lies on a valid page inside the context
    };
    // (a thread whose 16-byte chunk lies beyond a narrow head reads the head's last chunk instead; zeroed like a row past the end)
    const bool col_ok = chunk * 8 < P.head_dim;
    const int64_t safe_off = (int64_t)trow * P.c_st + (int64_t)kvh * P.c_sh + min(chunk * 8, P.head_dim - 8);
    auto fetch = [&](Staged& sg, int t) {
        const int key0 = key_begin + t * kTileKeys;
        sg.row_ok = 0;
        sg.pass_ok = 0;
#pragma unroll
        for (int p = 0; p < kPasses; ++p) {
            const int kp = key0 + kRowsPerPass * p;
            const int page_slot = P.page_shift >= 0 ? kp >> P.page_shift : kp / P.page_size;
            const int in_page = P.page_shift >= 0 ? kp & (P.page_size - 1) : kp % P.page_size;
            const bool inside = kp < key_end && page_slot < P.max_pages;
            const int64_t page = bt[inside ? page_slot : 0];
            const bool ok = inside && page >= 0 && page < P.num_pages;             // uniform
            const int64_t off = ok ? page * P.c_sp + (int64_t)in_page * P.c_st + safe_off : safe_off;
            sg.regs.k[p] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(P.k_cache + off));
            sg.regs.v[p] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(P.v_cache + off));
            sg.pass_ok |= (ok ? 1u : 0u) << p;
            sg.row_ok |= ((ok && col_ok && kp + trow < key_end) ? 1u : 0u) << p;
        }
    };
    unsigned tile_pass_ok[2] = {0, 0};                 // pass_ok of the tile sitting in LDS buffer 0 / 1
    auto stage = [&](int buf, Staged& sg) {
#pragma unroll
        for (int p = 0; p < kPasses; ++p)
            if (!((sg.row_ok >> p) & 1u)) { sg.regs.k[p] = u32x4{0, 0, 0, 0}; sg.regs.v[p] = u32x4{0, 0, 0, 0}; }
        store_tile<kTileKeys, kThreads>(lds[buf], lds[buf] + kTileBytes, sg.regs, tid);
        tile_pass_ok[buf] = sg.pass_ok;
    };
    auto compute = [&](int t) {
        const char* lk = lds[t & 1];
        const int key0 = key_begin + t * kTileKeys + kw * 32;        // this wavefront's 32 keys = passes 2kw, 2kw+1
        // keys of an invalid page are excluded (not merely zeroed): the owning wavefront skips them
        if ((tile_pass_ok[t & 1] >> (kPassesPerSlice * kw)) & 1u) {
            if (key0 + 32 <= key_end)
                attn_step<E, 1, 1, false>(lk, lk + kTileBytes, kw * 32, q, st, P.c, lane, key0, 0, key_end);
            else
                attn_step<E, 1, 1, true>(lk, lk + kTileBytes, kw * 32, q, st, P.c, lane, key0, 0, key_end);
        }
    };

    // Register sets ra / rb hold the tiles after the one in LDS; tile t+1 sits in set (t+1)%2.
    Staged ra, rb;
    fetch(ra, 0);
    if (DEPTH == 2 && n_tiles > 1) fetch(rb, 1);
    stage(0, ra);
    if (DEPTH == 2) { if (n_tiles > 2) fetch(ra, 2); } else { if (n_tiles > 1) fetch(ra, 1); }
    __syncthreads();
    for (int t = 0; t < n_tiles; t += 2) {
        // even tile t from buffer 0; stage tile t+1 into buffer 1
        compute(t);
        if (t + 1 < n_tiles) {
            if (DEPTH == 2) {
                stage(1, rb);
                if (t + 3 < n_tiles) fetch(rb, t + 3);
            } else {
                stage(1, ra);
                if (t + 2 < n_tiles) fetch(ra, t + 2);
            }
        }
        __syncthreads();
        if (t + 1 >= n_tiles) break;
        // odd tile t+1 from buffer 1; stage tile t+2 into buffer 0
        compute(t + 1);
        if (t + 2 < n_tiles) {
            stage(0, ra);
            if (DEPTH == 2) { if (t + 4 < n_tiles) fetch(ra, t + 4); } else { if (t + 3 < n_tiles) fetch(ra, t + 3); }
        }
        __syncthreads();
    }

    // ---- merge the KW key-slice states of each head through LDS ---------------------------------
    // Every slice leaves its state in LDS (register quads as 16-byte lanes: 16 stores of 1 KB per wavefront); after one
    // barrier slice kw folds the d tiles kw, kw + KW, ... of all KW states -- every slice a quarter (half) of the head,
    // and every slice stores what it folded.  (A tree of pairwise merges with 4-byte LDS accesses and three barriers,
    // all output from one wavefront, took 2.7 us of every workgroup's end.)  All slices sum in the same order, so they
    // agree on the head's m and l bit for bit.
    st.l[0] = both_halves_sum(st.l[0]);          // a state is now (m, l, O) per query
    // Exchange layout per wavefront: O as [d tile][group][64 lanes][4] floats, then m, l as [64].
    constexpr int kStateFloats = 4 * 16 * 64 + 2 * 64;
    static_assert(HPW * KW * kStateFloats * 4 <= (int)sizeof(lds), "merge buffer exceeds the tile region");
    float* xch = reinterpret_cast<float*>(&lds[0][0]) + (wave / KW) * KW * kStateFloats;   // this head's slots
    // (the loop's last barrier already separates the tile reads from these writes)
    {
        float* dst = xch + kw * kStateFloats;
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
            for (int g = 0; g < 4; ++g)
                *reinterpret_cast<f32x4*>(dst + ((t * 4 + g) * 64 + lane) * 4) =
                    f32x4{st.o[0][t][4 * g], st.o[0][t][4 * g + 1], st.o[0][t][4 * g + 2], st.o[0][t][4 * g + 3]};
        dst[4 * 16 * 64 + lane] = st.m[0];
        dst[4 * 16 * 64 + 64 + lane] = st.l[0];
    }
    __syncthreads();
    {
        float w[KW];                                // weights of the KW states: 2^(m_s - M)
        float M = kMinusBig;
#pragma unroll
        for (int s = 0; s < KW; ++s) { w[s] = xch[s * kStateFloats + 4 * 16 * 64 + lane]; M = fmaxf(M, w[s]); }
        float l = 0.f;
#pragma unroll
        for (int s = 0; s < KW; ++s) {
            w[s] = __builtin_amdgcn_exp2f(w[s] - M);
            l += xch[s * kStateFloats + 4 * 16 * 64 + 64 + lane] * w[s];
        }
        st.m[0] = M;
        st.l[0] = l;
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            if (t % KW != kw) continue;             // (uniform per wavefront)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int s = 0; s < KW; ++s)
                    acc += *reinterpret_cast<const f32x4*>(xch + s * kStateFloats + ((t * 4 + g) * 64 + lane) * 4) * w[s];
                st.o[0][t][4 * g] = acc.x; st.o[0][t][4 * g + 1] = acc.y; st.o[0][t][4 * g + 2] = acc.z; st.o[0][t][4 * g + 3] = acc.w;
            }
        }
    }

    // ---- output: slice kw holds, and stores, the d tiles kw, kw + KW, ... of its head ----------------
    if (n_valid_splits == 1) {
        if (!row_ok) return;
        const float inv = st.l[0] > 0.f ? 1.0f / st.l[0] : 0.f;   // no valid key at all: zeros
        __bf16* orow = P.o + (int64_t)b * P.o_sb + (int64_t)qrow * P.o_ss + (int64_t)head * P.o_sh;
#pragma unroll
        for (int dt = 0; dt < 4; ++dt) {
            if (dt % KW != kw) continue;
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                typename Elem16<E>::vec4 out;
#pragma unroll
                for (int e = 0; e < 4; ++e) out[e] = (E)(st.o[0][dt][4 * g + e] * inv);
                if (d_of_reg(dt, 4 * g, H) < P.head_dim) *reinterpret_cast<typename Elem16<E>::vec4*>(orow + d_of_reg(dt, 4 * g, H)) = out;
            }
        }
        return;
    }
    if (row_ok) {
        const int64_t slot = (((int64_t)b * P.num_q_heads + head) * P.nqt + qt) * P.nsplit + split;
        float* po = P.part_o + (slot * kQTile + r) * kHeadDim;
#pragma unroll
        for (int dt = 0; dt < 4; ++dt) {
            if (dt % KW != kw) continue;
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const f32x4 out = {st.o[0][dt][4 * g], st.o[0][dt][4 * g + 1], st.o[0][dt][4 * g + 2], st.o[0][dt][4 * g + 3]};
                if (P.arrive) store_agent(po + d_of_reg(dt, 4 * g, H), out);
                else *reinterpret_cast<f32x4*>(po + d_of_reg(dt, 4 * g, H)) = out;
            }
        }
        if (kw == 0 && H == 0) {
            float* ml = P.part_ml + (slot * 2 + 0) * kQTile + r;
            if (P.arrive) {
                __hip_atomic_store(ml, st.m[0], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                __hip_atomic_store(ml + kQTile, st.l[0], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            } else {
                ml[0] = st.m[0];
                ml[kQTile] = st.l[0];
            }
        }
    }
    if (!P.arrive) return;                       // two-launch mode: the combine kernel follows

    // ---- single-launch mode: the last split of this (sequence, head group) to arrive merges them ----
    // Every writer waits until its (written-through) partials have reached memory, then the workgroup
    // counts itself in; the workgroup that finds itself last reads all partials of the pair with
    // agent-scope loads.  No cache-wide fence on either side, and nobody waits for anybody: a
    // workgroup that is not last leaves.
    __shared__ int i_am_last;
    wait_vector_memory();
    __syncthreads();
    float* counter = P.arrive + ((int64_t)b * n_groups + hg) * P.nqt + qt;
    if (tid == 0) i_am_last = atomicAdd(counter, 1.0f) == (float)(n_valid_splits - 1) ? 1 : 0;
    __syncthreads();
    if (!i_am_last) return;
    for (int e = tid; e < HPW * 256; e += kThreads) {
        const int s = (e & 255) >> 3;
        if (qt * kQTile + s < P.sq) combine_query<E, true>(P, b, hg * HPW + (e >> 8), qt, s, e & 7, [&]() { return n_valid_splits; });
    }
    if (tid == 0) __hip_atomic_store(counter, 0.f, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // ready for the next launch
}

// One workgroup per (sequence, head): merges the split partials of its 32 queries; thread t takes
// 16 consecutive d values of query t / 8.  A sequence that was not split leaves after one load, and
// there are only bs * Hq workgroups to launch, which is what the common case costs when the
// attention kernel decided that nothing had to be cut.  The kernel is a chain of memory latencies
// (length -> partials -> output), not of bytes: the loads of four splits are issued together.
template <typename E>
__global__ __launch_bounds__(256) void paged_combine_kernel(const PagedParams P)
{
    const int qt = blockIdx.x % P.nqt, hq = (blockIdx.x / P.nqt) % P.num_q_heads, b = blockIdx.x / P.nqt / P.num_q_heads;
    const int s = threadIdx.x >> 3, c = threadIdx.x & 7;
    if (qt * kQTile + s >= P.sq) return;
    combine_query<E, false>(P, b, hq, qt, s, c, [&]() {
        const int ctx = min(P.context_lens[b], P.max_pages * P.page_size);
        const int span = P.span_out ? (int)*P.span_out : P.chunk;     // the attention kernel's choice
        return (ctx + span - 1) / span;
    });
}

// Keys per split.  Measured over batches of 4 to 64 sequences and contexts of 300 to 8000 keys, the
// kernel is fastest with 1.5 to 1.8 workgroups per CU in total (just under the two per CU that are
// resident at once: one round, no tail of late workgroups), with splits of at least 512 keys (a
// workgroup's fixed cost is worth some 300 keys of streaming) and with whole sequences once there
// are about as many (sequence, head group) pairs as CUs (from 192 pairs on) (in the engine's decode pass at batch 32 that beats two
// splits per sequence by 4 %: no partials to write, nothing to combine).  The host knows the
// page-table width, not the lengths: tables are taken to be about 65 % full, and the last split of
// a sequence to be half a split (the attention kernel, which sees the lengths, corrects the split
// both ways: PagedParams::fit_slots).  In the pair-per-CU case up to four splits per sequence are allowed
// and the kernel itself, which sees the lengths, cuts only sequences well above the mean
// (*device_span; the dense workgroup numbering that this needs exists for up to 64 sequences).
//
// The counts behind those rules (1.95 workgroups per CU, pairs per CU) are taken from the current device's
// number of compute units, read once per device; 256 on the MI355X that the rules were measured on, and
// where no device can be asked (a shape query in a process without a GPU).
int cu_count() {
    constexpr int kMaxDevices = 64;
    static std::atomic<int> cached[kMaxDevices];
    int device = -1;
    if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= kMaxDevices) return 256;
    int n = cached[device].load(std::memory_order_relaxed);
    if (n == 0) {
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess || n <= 0) n = 256;
        cached[device].store(n, std::memory_order_relaxed);
    }
    return n;
}

// head_groups counts the workgroups that one (sequence, split) pair launches: head groups x query tiles.
int pick_chunk(int bs, int head_groups, int max_pages, int page_size, bool* device_span) {
    *device_span = false;
    const int cus = cu_count();
    const int64_t max_keys = (int64_t)max_pages * page_size;
    const int64_t whole = (max_keys + kChunkAlign - 1) / kChunkAlign * kChunkAlign;   // one split per sequence
    const double per_pair = 1.953 * cus / ((double)bs * head_groups) - 0.5;           // workgroups per pair
    if ((int64_t)bs * head_groups >= (cus * 3) / 4 || per_pair <= 1.0) {
        if (bs > 64 || whole < 4 * kChunkAlign) return (int)whole;
        *device_span = true;
        return (int)((whole / 4 + kChunkAlign - 1) / kChunkAlign * kChunkAlign);
    }
    int64_t chunk = (int64_t)(0.65 * (double)max_keys / per_pair / kChunkAlign + 0.5) * kChunkAlign;
    if (chunk < 2 * kChunkAlign) chunk = 2 * kChunkAlign;
    if (2 * chunk >= max_keys && (int64_t)bs * head_groups >= (cus * 25) / 32) chunk = whole;   // two short splits only to fill CUs
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
    if (head_dim > kHeadDim || head_dim % 16 != 0) return 0;       // the fp32-arithmetic kernel: no split, no partials
    const int G = num_q_heads / num_kv_heads;
    const int HPW = (G % 2 == 0) ? 2 : 1;
    const int nqt = sq <= kQTile ? 1 : (sq + kQTile - 1) / kQTile;
    bool device_span;
    const int chunk = pick_chunk(bs, num_q_heads / HPW * nqt, max_pages, page_size, &device_span);
    const int nsplit = nsplit_of(max_pages, page_size, chunk);
    if (nsplit <= 1) return 0;
    return (int64_t)bs * num_q_heads * nqt * nsplit * kQTile * (kHeadDim + 2) * (int64_t)sizeof(float) + 16;   // + the split size
}

namespace mdx {

int launch_paged_f32(const void* q, void* o, const void* k_cache, const void* v_cache,
                     int64_t q_stride_b, int64_t q_stride_s, int64_t q_stride_h,
                     int64_t o_stride_b, int64_t o_stride_s, int64_t o_stride_h,
                     int64_t cache_stride_page, int64_t cache_stride_tok, int64_t cache_stride_head,
                     const int32_t* block_table, int64_t bt_stride, const int32_t* context_lens,
                     int32_t bs, int32_t sq, int32_t num_q_heads, int32_t num_kv_heads,
                     int32_t head_dim, int32_t max_pages, int32_t page_size, int64_t num_pages,
                     float scale, int32_t dtype, hipStream_t stream);                         // paged_attn_f32.hip

// The launch behind every paged entry point of the library.
int launch_paged(const void* q, void* o, const void* k_cache, const void* v_cache,
                 int64_t q_stride_b, int64_t q_stride_s, int64_t q_stride_h,
                 int64_t o_stride_b, int64_t o_stride_s, int64_t o_stride_h,
                 int64_t cache_stride_page, int64_t cache_stride_tok, int64_t cache_stride_head,
                 const int32_t* block_table, int64_t bt_stride, const int32_t* context_lens,
                 int32_t bs, int32_t sq, int32_t num_q_heads, int32_t num_kv_heads,
                 int32_t head_dim, int32_t max_pages, int32_t page_size, int64_t num_pages,
                 float scale, int32_t dtype,
                 void* workspace, int64_t workspace_bytes, bool single_launch, void* counters, int64_t counter_bytes,
                 mdx_stream_t stream_)
{
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    MDX_REQUIRE(bs >= 0 && sq >= 0 && max_pages >= 0 && num_pages >= 0, MDX_EINVAL, "paged_block_attn: negative size");
    MDX_REQUIRE(dtype == MDX_BF16 || dtype == MDX_F16 || dtype == MDX_F32, MDX_EUNSUPPORTED, "paged_block_attn: dtype %d (bf16, fp16 or fp32)", dtype);
    // 16-bit elements and heads of 16, 32, ..., 128 columns run on the 16-bit matrix instructions; fp32 tensors and
    // the other head widths up to 256 on the fp32 one (paged_attn_f32.hip: no split, no workspace)
    const bool f32_arithmetic = dtype == MDX_F32 || head_dim > kHeadDim || head_dim % 16 != 0;
    MDX_REQUIRE(head_dim >= 4 && head_dim <= 256 && head_dim % 4 == 0, MDX_EUNSUPPORTED,
                "paged_block_attn: head_dim %d (multiples of 4 up to 256)", head_dim);
    MDX_REQUIRE(num_q_heads > 0 && num_kv_heads > 0 && num_q_heads % num_kv_heads == 0, MDX_EINVAL,
                "paged_block_attn: Hq %d not a multiple of Hkv %d", num_q_heads, num_kv_heads);
    MDX_REQUIRE(sq <= kMaxSq, MDX_EUNSUPPORTED, "paged_block_attn: %d queries per sequence (max %d)", sq, kMaxSq);
    MDX_REQUIRE(page_size > 0 && page_size % 32 == 0, MDX_EUNSUPPORTED,
                "paged_block_attn: page_size %d not a multiple of 32", page_size);
    MDX_REQUIRE(scale > 0.f, MDX_EINVAL, "paged_block_attn: scale must be positive");
    if (bs == 0 || sq == 0) return MDX_OK;
    MDX_REQUIRE(max_pages > 0, MDX_EINVAL, "paged_block_attn: empty block table");
    MDX_REQUIRE(q && o && k_cache && v_cache && block_table && context_lens, MDX_EINVAL, "paged_block_attn: null pointer");
    MDX_REQUIRE(bt_stride >= max_pages, MDX_EINVAL, "paged_block_attn: bt_stride < max_pages");
    if (f32_arithmetic)
        return launch_paged_f32(q, o, k_cache, v_cache, q_stride_b, q_stride_s, q_stride_h, o_stride_b, o_stride_s, o_stride_h,
                                cache_stride_page, cache_stride_tok, cache_stride_head, block_table, bt_stride, context_lens,
                                bs, sq, num_q_heads, num_kv_heads, head_dim, max_pages, page_size, num_pages, scale, dtype, stream);
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
    P.bs = bs; P.sq = sq; P.heads_per_kv = G; P.page_size = page_size; P.max_pages = max_pages;
    P.page_shift = -1;
    for (int i = 0; i < 31; ++i) if (page_size == (1 << i)) P.page_shift = i; P.num_pages = num_pages;
    bool device_span;
    P.nqt = (sq + kQTile - 1) / kQTile;
    const int64_t wg_per_pair = (int64_t)(num_q_heads / HPW) * P.nqt;               // workgroups of one (sequence, split)
    const int cus = cu_count();
    P.chunk = pick_chunk(bs, (int)wg_per_pair, max_pages, page_size, &device_span);
    P.nsplit = nsplit_of(max_pages, page_size, P.chunk);
    P.num_q_heads = num_q_heads;
    P.head_dim = head_dim;
    P.c = scale * kLog2e;
    P.part_o = nullptr; P.part_ml = nullptr; P.span_out = nullptr; P.arrive = nullptr; P.fit_slots = 0;
    if (P.nsplit > 1) {
        const int64_t n_slots = (int64_t)bs * num_q_heads * P.nqt * P.nsplit;
        const int64_t need = n_slots * kQTile * (kHeadDim + 2) * (int64_t)sizeof(float) + 16;
        MDX_REQUIRE(workspace && workspace_bytes >= need, MDX_EWORKSPACE,
                    "paged_block_attn: workspace of %lld bytes needed, %lld given", (long long)need, (long long)workspace_bytes);
        MDX_REQUIRE(mdx::aligned16(workspace), MDX_EWORKSPACE, "paged_block_attn: workspace not 16-byte aligned");
        P.part_o = static_cast<float*>(workspace);
        P.part_ml = P.part_o + n_slots * kQTile * kHeadDim;
        if (!device_span && bs <= 64) P.fit_slots = cus * (HPW == 2 ? 2 : 1);        // workgroups resident at once
        if (device_span || P.fit_slots > 0) P.span_out = P.part_ml + n_slots * kQTile * 2;
        // Single launch: the partials are written through with agent-scope stores and read back with
        // agent-scope loads, so counting in costs a workgroup the wait for its own stores and one atomic,
        // not a device-wide release (a write-back walk of its XCD's L2).  Where only outliers are cut
        // (device_span) that beats the combine launch (ragged batch of 32: 93 -> 80 us, and a launch
        // whose sequences stay whole pays nothing).  Where every sequence is split the merges all fall
        // at the end of the launch, one after the other behind the written-through stores (config 2:
        // 61 us against 49 with the combine launch; with full release fences it was 145), so those
        // launches keep the combine kernel.
        if (single_launch && device_span) {
            const int64_t need_c = (int64_t)bs * wg_per_pair * (int64_t)sizeof(float);
            MDX_REQUIRE(counters && counter_bytes >= need_c, MDX_EWORKSPACE,
                        "paged_block_attn: %lld bytes of arrival counters needed, %lld given", (long long)need_c, (long long)counter_bytes);
            MDX_REQUIRE(((uintptr_t)counters & 3) == 0, MDX_EWORKSPACE, "paged_block_attn: counters not 4-byte aligned");
            P.arrive = static_cast<float*>(counters);
        }
    }
    // head group fastest, then the dense (sequence, split) index
    MDX_REQUIRE((int64_t)bs * P.nsplit <= 65535, MDX_EUNSUPPORTED, "paged_block_attn: bs * splits %lld > 65535", (long long)bs * P.nsplit);
    // With device-chosen splits of at least 1.25 x the mean length, sum_b ceil(len_b / split) <= 1.8 bs:
    // the dense numbering never needs more than 2 bs (sequence, split) pairs, whatever nsplit allows.
    const int pairs_y = device_span ? (bs * P.nsplit < 2 * bs ? bs * P.nsplit : 2 * bs) : bs * P.nsplit;
    const dim3 grid((unsigned)(num_q_heads / HPW * P.nqt), (unsigned)pairs_y);
    // Up to one (sequence, head group) pair per CU: workgroups of 8 wavefronts on 128-key tiles, so that a
    // CU that holds a single workgroup still has two wavefronts per SIMD (batch 32 x 8 KV heads: 79 -> 69 us
    // on equal lengths); with more pairs than CUs the second round costs more than that gains.
    const bool eight = device_span && (int64_t)bs * wg_per_pair <= cus;
    const unsigned n_combine = (unsigned)(bs * num_q_heads * P.nqt);
    const bool two_launches = P.nsplit > 1 && !P.arrive;
    if (dtype == MDX_F16) {
        if (HPW == 2 && eight) paged_block_attn_kernel<_Float16, 2, 2, 8><<<grid, 512, 0, stream>>>(P);
        else if (HPW == 2)     paged_block_attn_kernel<_Float16, 2, 2, 4><<<grid, 256, 0, stream>>>(P);
        else                   paged_block_attn_kernel<_Float16, 1, 1, 4><<<grid, 256, 0, stream>>>(P);
    } else {
        if (HPW == 2 && eight) paged_block_attn_kernel<__bf16, 2, 2, 8><<<grid, 512, 0, stream>>>(P);
        else if (HPW == 2)     paged_block_attn_kernel<__bf16, 2, 2, 4><<<grid, 256, 0, stream>>>(P);
        else                   paged_block_attn_kernel<__bf16, 1, 1, 4><<<grid, 256, 0, stream>>>(P);
    }
    int rc = mdx::check_launch("paged_block_attn");
    if (rc != MDX_OK || !two_launches) return rc;
    if (dtype == MDX_F16) paged_combine_kernel<_Float16><<<n_combine, 256, 0, stream>>>(P);
    else                  paged_combine_kernel<__bf16><<<n_combine, 256, 0, stream>>>(P);
    return mdx::check_launch("paged_combine");
}

}  // namespace mdx

extern "C" int mdx_paged_block_attn(const void* q, void* o, const void* k_cache, const void* v_cache,
                                    int64_t q_stride_b, int64_t q_stride_s, int64_t q_stride_h,
                                    int64_t o_stride_b, int64_t o_stride_s, int64_t o_stride_h,
                                    int64_t cache_stride_page, int64_t cache_stride_tok, int64_t cache_stride_head,
                                    const int32_t* block_table, int64_t bt_stride, const int32_t* context_lens,
                                    int32_t bs, int32_t sq, int32_t num_q_heads, int32_t num_kv_heads,
                                    int32_t head_dim, int32_t max_pages, int32_t page_size, int64_t num_pages,
                                    float scale, int32_t dtype,
                                    void* workspace, int64_t workspace_bytes, mdx_stream_t stream)
{
    return mdx::launch_paged(q, o, k_cache, v_cache, q_stride_b, q_stride_s, q_stride_h, o_stride_b, o_stride_s, o_stride_h,
                        cache_stride_page, cache_stride_tok, cache_stride_head, block_table, bt_stride, context_lens,
                        bs, sq, num_q_heads, num_kv_heads, head_dim, max_pages, page_size, num_pages, scale, dtype,
                        workspace, workspace_bytes, false, nullptr, 0, stream);
}

extern "C" int64_t mdx_paged_block_attn_counter_bytes(int32_t bs, int32_t num_q_heads, int32_t num_kv_heads)
{
    if (bs <= 0 || num_q_heads <= 0 || num_kv_heads <= 0) return 0;
    const int G = num_q_heads / num_kv_heads;
    // one counter per (sequence, head group, query tile), sized for the largest block (four tiles of 32 queries)
    return (int64_t)bs * (num_q_heads / ((G % 2 == 0) ? 2 : 1)) * (kMaxSq / kQTile) * (int64_t)sizeof(float);
}

extern "C" int mdx_paged_block_attn_single_launch(const void* q, void* o, const void* k_cache, const void* v_cache,
                                                  int64_t q_stride_b, int64_t q_stride_s, int64_t q_stride_h,
                                                  int64_t o_stride_b, int64_t o_stride_s, int64_t o_stride_h,
                                                  int64_t cache_stride_page, int64_t cache_stride_tok, int64_t cache_stride_head,
                                                  const int32_t* block_table, int64_t bt_stride, const int32_t* context_lens,
                                                  int32_t bs, int32_t sq, int32_t num_q_heads, int32_t num_kv_heads,
                                                  int32_t head_dim, int32_t max_pages, int32_t page_size, int64_t num_pages,
                                                  float scale, int32_t dtype,
                                                  void* workspace, int64_t workspace_bytes,
                                                  void* counters, int64_t counter_bytes, mdx_stream_t stream)
{
    return mdx::launch_paged(q, o, k_cache, v_cache, q_stride_b, q_stride_s, q_stride_h, o_stride_b, o_stride_s, o_stride_h,
                        cache_stride_page, cache_stride_tok, cache_stride_head, block_table, bt_stride, context_lens,
                        bs, sq, num_q_heads, num_kv_heads, head_dim, max_pages, page_size, num_pages, scale, dtype,
                        workspace, workspace_bytes, true, counters, counter_bytes, stream);
}
