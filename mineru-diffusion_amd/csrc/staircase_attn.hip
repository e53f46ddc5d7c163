// Staircase block-prefill attention over packed variable-length sequences.
//
// Query row i of a sequence of length L sees key j iff
//   j <= ((i + pad) / S + 1) * S - 1 - pad,   pad = ceil(L/S)*S - L
// (blocks of S tokens, right-aligned; semantics of
// engines/nano_dvlm/nanovllm/kernels/triton/attention/block_prefill_attention_v2.py:46-53,82-102,134-156).
//
// Work decomposition (not the reference's one-program-per-(sequence, head)):
// everything is indexed in PADDED coordinates ip = i + pad, jp = j + pad, in
// which block boundaries fall on multiples of S.  A wavefront owns 32
// consecutive padded query rows of one query head; a workgroup of 4 wavefronts
// owns 128 consecutive rows of that head and stages the K/V tiles they share
// in LDS.  Two such workgroups fit a CU (2 wavefronts per SIMD); they share no
// barrier, so they drift out of phase and one's MFMAs overlap the other's
// softmax arithmetic.  For S >= 32 every 32-row tile lies inside one block, so
// all its rows share one key limit and no element of the tile interior is ever
// masked: only the very first keys (jp < pad) and, for S < 32, the tiles
// straddling the limit take the masked path.  K/V tiles of 64 keys are
// double-buffered in LDS (global -> registers one tile ahead -> LDS), one
// barrier per tile.
//
// Launch order: workgroups are numbered heaviest-first (last row group of every
// sequence first); the query head varies fastest, ordered KV head first, so
// that consecutive workgroups, which the dispatcher deals round-robin to the 8
// XCDs, put all query heads of one KV head on the same XCD (one K/V stream per
// XCD L2 when there are 8 KV heads).
#include "mdx_common.h"
#include "attn_tile.h"
#include <atomic>

namespace {

using namespace mdx_attn;

constexpr int kTileKeys = 64;      // keys staged in LDS per iteration
constexpr int kThreads = 256;      // 4 wavefronts, 2 workgroups per CU
constexpr int kRowsPerWg = 128;    // 4 wavefronts x 32 query rows
constexpr int kTileBytes = kTileKeys * kLdsPitch;

struct StaircaseParams {
    const __bf16* q; const __bf16* k; const __bf16* v; __bf16* o;
    int64_t q_st, q_sh, k_st, k_sh, v_st, v_sh, o_st, o_sh;   // element strides: token, head
    const int32_t* cu_seqlens;
    int total_tokens;
    int batch, n_row_groups, num_q_heads, num_kv_heads;
    int log2_s;
    int head_dim;                                              // <= 128, a multiple of 16
    int o_rows16;                                              // rows of o take 16-byte stores (aligned, strides multiples of 8 elements)
    float c;                                                   // scale * log2(e)
};

// Sequence b's first token and length.  Bounds that do not describe a range inside the packed
// tensors (decreasing, negative, past total_tokens) are clipped to one, so that no row outside
// q/k/v/o is ever touched; what such a call computes is unspecified.
__device__ __forceinline__ void seq_bounds(const StaircaseParams& P, int b, int& seq0, int& L)
{
    const int lo = min(max(P.cu_seqlens[b], 0), P.total_tokens);
    const int hi = min(max(P.cu_seqlens[b + 1], lo), P.total_tokens);
    seq0 = lo;
    L = hi - lo;
}

// Workgroup -> (sequence b, row group rg) for the j-th (sequence, row group) pair in launch order.
// Row groups are handed out heaviest-first (the last row group of a sequence attends to the most
// keys).  The dispatcher deals consecutive workgroups round-robin to XCDs and shader engines and
// blocks on a full one, so neighbours in launch order must weigh the same: the head slot varies
// fastest, then the sequences that own a row group at this level, and workgroups that find no
// work may only sit at the very end of the grid.  With up to 64 sequences each wavefront derives
// this dense numbering itself (lane b holds sequence b's row-group count, lane r evaluates
// F(r) = #pairs at level >= r); with more sequences, 64 of them per step, as long as no sequence has more
// than 64 row groups (8 K tokens); beyond both the grid is the full (level x sequence) rectangle and
// absent pairs return at once.  Returns false when there is no such pair.
// Inclusive prefix sum over the 64 lanes of a wavefront (DPP shifts inside rows of 16 lanes, then the
// two row broadcasts): 6 additions, no LDS traffic.
__device__ __forceinline__ int wave_prefix_sum(int x)
{
    int v = x;
    v += __builtin_amdgcn_update_dpp(0, v, 0x111, 0xf, 0xf, false);   // row_shr:1
    v += __builtin_amdgcn_update_dpp(0, v, 0x112, 0xf, 0xf, false);   // row_shr:2
    v += __builtin_amdgcn_update_dpp(0, v, 0x114, 0xf, 0xf, false);   // row_shr:4
    v += __builtin_amdgcn_update_dpp(0, v, 0x118, 0xf, 0xf, false);   // row_shr:8
    v += __builtin_amdgcn_update_dpp(0, v, 0x142, 0xa, 0xf, false);   // row_bcast:15 into rows 1 and 3
    v += __builtin_amdgcn_update_dpp(0, v, 0x143, 0xc, 0xf, false);   // row_bcast:31 into rows 2 and 3
    return v;
}

// `hist`: 65 ints of LDS that belong to the calling wavefront alone (unused when there are more than 64 row groups).
constexpr int kDenseMaxBatch = 1024;   // sequences per launch that the histogram numbering walks (64 per step)
__device__ __forceinline__ bool locate_row_group(const StaircaseParams& P, int j, int lane, int* hist, int& b, int& rg)
{
    // row groups of sequence s (0 for an empty or absent one); never more than the launch has levels for
    auto groups_of = [&](int s) {
        int g = 0;
        if (s < P.batch) {
            int first, len;
            seq_bounds(P, s, first, len);
            if (len > 0) g = min(P.n_row_groups, ((((len + (1 << P.log2_s) - 1) >> P.log2_s) << P.log2_s) + kRowsPerWg - 1) / kRowsPerWg);
        }
        return g;
    };
    if (P.n_row_groups <= 64 && P.batch <= kDenseMaxBatch) {
        // F(r) = sum over sequences of max(0, g - r) for all 64 levels r at once, without a loop over the
        // sequences (which took 0.9 us of every workgroup's start at 32 sequences, 1.8 at 64): count the
        // sequences per value of g (LDS atomics of this wavefront only, which complete in order; 64 sequences
        // per step, so a prefill of the scheduler's 512 sequences, config.py:38, takes 8 steps), then
        // C(r) = #{g > r} and F(r) = C(r) + C(r + 1) + ... are two prefix sums with the levels laid out
        // backwards over the lanes (lane l = level 63 - l).
        hist[lane] = 0;
        if (lane == 0) hist[64] = 0;
        const int g0 = groups_of(lane);
        if (lane < P.batch) atomicAdd(&hist[g0], 1);
        for (int s0 = 64; s0 < P.batch; s0 += 64)
            if (s0 + lane < P.batch) atomicAdd(&hist[groups_of(s0 + lane)], 1);
        __builtin_amdgcn_wave_barrier();
        const int c = wave_prefix_sum(hist[64 - lane]);        // C(63 - lane)
        const int f = wave_prefix_sum(c);                      // F(63 - lane)
        const unsigned long long above = __ballot(f > j);      // the levels 0 .. n - 1: the high lanes
        const int n = __popcll(above);
        if (n == 0) return false;                              // past the last pair
        const int level = n - 1;
        // index among the sequences that have this row group: the levels above account for F(level) - C(level) pairs
        int nth = j - __builtin_amdgcn_readlane(f, 64 - n) + __builtin_amdgcn_readlane(c, 64 - n);
        b = -1;
        for (int s0 = 0; s0 < P.batch; s0 += 64) {
            const int g = s0 == 0 ? g0 : groups_of(s0 + lane);
            const unsigned long long owners = __ballot(g > level);
            const int here = __popcll(owners);
            if (nth < here) {
                const int before = __popcll(owners & ((1ull << lane) - 1ull));
                const unsigned long long hit = __ballot(((owners >> lane) & 1ull) != 0 && before == nth);
                b = s0 + __ffsll((long long)hit) - 1;
                break;
            }
            nth -= here;
        }
        rg = level;
        return b >= 0;
    }
    if (P.batch <= 64) {
        // sequences longer than 64 row groups (8 K tokens): the levels are walked 64 at a time
        const int g = groups_of(lane);
        int level = -1, f_level = 0;
        for (int base = 0; base < P.n_row_groups; base += 64) {
            const int r_lane = base + lane;
            int f = 0;
            for (int s = 0; s < P.batch; ++s) f += max(0, __builtin_amdgcn_readlane(g, s) - r_lane);
            const unsigned long long above = __ballot(f > j);  // F decreases with the level: low lanes
            if (above == 0) break;
            const int n = __popcll(above);
            level = base + n - 1;
            f_level = __builtin_amdgcn_readlane(f, n - 1);
            if (n < 64) break;
        }
        if (level < 0) return false;                           // past the last pair
        const unsigned long long owners = __ballot(g > level); // sequences that have this row group
        const int nth = j - f_level + __popcll(owners);        // index among them
        const int before = __popcll(owners & ((1ull << lane) - 1ull));
        const unsigned long long hit = __ballot(((owners >> lane) & 1ull) != 0 && before == nth);
        b = __ffsll((long long)hit) - 1;
        rg = level;
        return b >= 0;
    }
    // more than 64 sequences with more than 64 row groups each: the full (level x sequence) rectangle
    b = j % P.batch;
    rg = P.n_row_groups - 1 - j / P.batch;
    return true;
}

// NARROW: head_dim below 128 (a multiple of 16).  Rows of q, k, v are then padded with zeros on their way into
// registers and LDS, products over the padding are skipped, and only head_dim columns of o are written.
template <typename E, bool NARROW>
__global__ __launch_bounds__(kThreads, 2) void staircase_attn_kernel(const StaircaseParams P)
{
    const int width = NARROW ? P.head_dim : kHeadDim;
    __shared__ __attribute__((aligned(16))) char lds_kbuf[2][kTileBytes];   // double-buffered K and V tiles
    __shared__ __attribute__((aligned(16))) char lds_vbuf[2][kTileBytes];
    __shared__ int lds_hist[kThreads / 64][80];                // per wavefront: scratch of the workgroup numbering (no barrier separates it from the first tile store)

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int H = lane >> 5, r = lane & 31;

    // ---- workgroup -> (head slot, sequence b, row group rg) ------------------------------------
    const int hslot = blockIdx.x % P.num_q_heads;
    int b, rg;
    if (!locate_row_group(P, blockIdx.x / P.num_q_heads, lane, lds_hist[wave], b, rg)) return;

    int seq0, L;
    seq_bounds(P, b, seq0, L);
    if (L <= 0) return;
    const int S = 1 << P.log2_s;
    const int Lp = ((L + S - 1) >> P.log2_s) << P.log2_s;     // padded length
    const int pad = Lp - L;
    const int row_g0 = rg * kRowsPerWg;                        // first padded row of the workgroup
    if (row_g0 >= Lp) return;

    const int kvh = hslot % P.num_kv_heads;                    // launch order: KV head fastest
    const int head = kvh * (P.num_q_heads / P.num_kv_heads) + hslot / P.num_kv_heads;

    // ---- this wavefront's 32 rows ----
    const int row_w0 = row_g0 + wave * 32;
    const int ip = row_w0 + r;                                 // this lane's padded query row
    const bool row_ok = ip >= pad && ip < Lp;
    const int64_t tok = (int64_t)seq0 + (ip - pad);
    typename Elem16<E>::vec8 q[1][8];
    load_q(q[0], row_ok ? P.q + tok * P.q_st + (int64_t)head * P.q_sh : nullptr, H, width);

    // exclusive key limit (padded coordinates) of this lane's row, and the wavefront's extremes
    auto limit_of = [&](int row) { return min(Lp, ((row >> P.log2_s) + 1) << P.log2_s); };
    const int key_hi = limit_of(ip);
    const int wave_hi = (row_w0 < Lp) ? limit_of(min(row_w0 + 31, Lp - 1)) : 0;   // 0: idle wavefront
    const int wave_hi_min = limit_of(row_w0);
    const int wg_hi = limit_of(min(row_g0 + kRowsPerWg - 1, Lp - 1));
    const int n_tiles = (wg_hi + kTileKeys - 1) / kTileKeys;

    WaveState<1> st;
    st.init();

    // ---- K/V tile pipeline: registers hold tile t+1 while LDS holds tile t (other buffer: t-1) ----
    // Thread-private row pointers walk down the sequence one tile per fetch; rows outside the
    // sequence (only possible in the first and last tiles) are never dereferenced.
    const int chunk = tid & 15, trow = tid >> 4;
    const bool col_ok = !NARROW || chunk * 8 < width;          // this thread's 16-byte chunk exists in a row
    constexpr int kPasses = TileRegs<kTileKeys, kThreads>::kPasses;
    constexpr int kRowsPerPass = kThreads / 16;
    const int64_t row0 = (int64_t)seq0 - pad + trow;          // token of LDS row `trow` of tile 0
    const __bf16* kcur = P.k + (int64_t)kvh * P.k_sh + row0 * P.k_st + chunk * 8;
    const __bf16* vcur = P.v + (int64_t)kvh * P.v_sh + row0 * P.v_st + chunk * 8;
    const int64_t k_pass = (int64_t)kRowsPerPass * P.k_st, v_pass = (int64_t)kRowsPerPass * P.v_st;
    TileRegs<kTileKeys, kThreads> regs;
    auto fetch = [&](int t) {                  // called with t = 0, 1, 2, ... in order
        const bool interior = t * kTileKeys >= pad && (t + 1) * kTileKeys <= Lp;   // uniform
#pragma unroll
        for (int p = 0; p < kPasses; ++p) {
            const int jp = t * kTileKeys + trow + kRowsPerPass * p;
            if (col_ok && (interior || (jp >= pad && jp < Lp))) {
                regs.k[p] = *reinterpret_cast<const u32x4*>(kcur + p * k_pass);
                regs.v[p] = *reinterpret_cast<const u32x4*>(vcur + p * v_pass);
            } else {                           // keys outside the sequence: zero rows, masked below (or padding columns)
                regs.k[p] = u32x4{0, 0, 0, 0};
                regs.v[p] = u32x4{0, 0, 0, 0};
            }
        }
        kcur += kPasses * k_pass;
        vcur += kPasses * v_pass;
    };

    fetch(0);
    store_tile<kTileKeys, kThreads>(lds_kbuf[0], lds_vbuf[0], regs, tid);
    if (n_tiles > 1) fetch(1);
    __syncthreads();
    for (int t = 0; t < n_tiles; ++t) {
        const char* lds_k = lds_kbuf[t & 1];
        const char* lds_v = lds_vbuf[t & 1];
        const int key0 = t * kTileKeys;
        if (key0 < wave_hi) {
            if (key0 >= pad && key0 + kTileKeys <= wave_hi_min) {
                attn_step<E, 1, 2, false>(lds_k, lds_v, 0, q, st, P.c, lane, key0, pad, key_hi, width);
            } else if (key0 + 32 < wave_hi) {
                attn_step<E, 1, 2, true>(lds_k, lds_v, 0, q, st, P.c, lane, key0, pad, key_hi, width);
            } else {
                attn_step<E, 1, 1, true>(lds_k, lds_v, 0, q, st, P.c, lane, key0, pad, key_hi, width);
            }
        }
        if (t + 1 < n_tiles) {
            // the other buffer was last read in iteration t-1, which every wavefront has left
            store_tile<kTileKeys, kThreads>(lds_kbuf[(t + 1) & 1], lds_vbuf[(t + 1) & 1], regs, tid);
            if (t + 2 < n_tiles) fetch(t + 2);
        }
        __syncthreads();
    }

    // ---- epilogue: O = O^T / l as 16-bit rows ----
    // The accumulators hold O transposed: a lane owns 4 consecutive d of its query per (d tile, group), and stores made
    // from there touch 32 rows with 16 bytes each (16 such instructions cost 12-20 % of a launch of sequences of a few
    // hundred tokens).  Each wavefront therefore turns its 32 x 128 tile around through one of the four K / V tile
    // buffers (the loop's last barrier has retired them) and writes whole rows: 16 lanes x 16 bytes per row, four rows
    // per instruction.  LDS operations of a wavefront complete in order, so its reads see all of its writes.
    const float inv = 1.0f / both_halves_sum(st.l[0]);          // rows outside the sequence: never stored
    if (P.o_rows16) {
        char* tile = (wave & 2) ? lds_vbuf[wave & 1] : lds_kbuf[wave & 1];
#pragma unroll
        for (int dt = 0; dt < 4; ++dt)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                typename Elem16<E>::vec4 out;
#pragma unroll
                for (int e = 0; e < 4; ++e) out[e] = (E)(st.o[0][dt][4 * g + e] * inv);
                *reinterpret_cast<typename Elem16<E>::vec4*>(tile + r * kLdsPitch + d_of_reg(dt, 4 * g, H) * 2) = out;
            }
        __builtin_amdgcn_wave_barrier();
        const int chunk16 = lane & 15, sub = lane >> 4;
        if (!NARROW || chunk16 * 8 < width) {
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const int rho = 4 * j + sub;                    // row of the wavefront's tile
                const int jp = row_w0 + rho;
                const u32x4 v = *reinterpret_cast<const u32x4*>(tile + rho * kLdsPitch + chunk16 * 16);
                if (jp >= pad && jp < Lp)
                    __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(P.o + ((int64_t)seq0 + (jp - pad)) * P.o_st + (int64_t)head * P.o_sh + chunk16 * 8));
            }
        }
        return;
    }
    if (!row_ok) return;
    __bf16* orow = P.o + tok * P.o_st + (int64_t)head * P.o_sh;
#pragma unroll
    for (int dt = 0; dt < 4; ++dt)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            typename Elem16<E>::vec4 out;
#pragma unroll
            for (int e = 0; e < 4; ++e) out[e] = (E)(st.o[0][dt][4 * g + e] * inv);
            if (!NARROW || d_of_reg(dt, 4 * g, H) < width) *reinterpret_cast<typename Elem16<E>::vec4*>(orow + d_of_reg(dt, 4 * g, H)) = out;
        }
}


// ---- pair-of-heads kernel -----------------------------------------------------------------------
// Same decomposition in rows, but a wavefront owns its 32 rows for TWO query heads that share a
// KV head, so that every K / V fragment it fetches from LDS feeds two MFMAs (the one-head form
// needs 1 KB of LDS reads per MFMA and is bound by that).  512 registers per wavefront, one
// workgroup per CU; the key loop is the hand-scheduled asm of staircase_pair_core.inc, in which the
// softmax arithmetic of one tile is issued in the shadow of the next tile's QK MFMAs.  All four
// wavefronts of a workgroup walk the same number of key tiles (they share the tiles' loads and a
// barrier per tile); for tiles beyond a wavefront's own last limit it only loads and waits.
#include "staircase_pair_core.inc"
#include "staircase_pair_core_f16.inc"      // the same core on fp16 elements (the generator run with "f16")
__device__ __forceinline__ void pair_core(const PairCoreArgs& A, const bf16x8 (&q)[2][8]) { staircase_pair_core(A, q); }
__device__ __forceinline__ void pair_core(const PairCoreArgs& A, const f16x8 (&q)[2][8]) { staircase_pair_core_f16(A, q); }

constexpr int kPairSlots = 5;                     // LDS slots of one K tile + one V tile, 256-byte rows
constexpr int kPairLdsBytes = kPairSlots * 2 * kTileKeys * kRowBytes;

// Values the asm reads from scalar registers must be wavefront-uniform in the compiler's eyes.
__device__ __forceinline__ int uniform(int x) { return __builtin_amdgcn_readfirstlane(x); }
__device__ __forceinline__ const void* uniform(const void* p) {
    const uint64_t v = (uint64_t)p;
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    return (const void*)(((uint64_t)hi << 32) | lo);
}

template <typename E>
__global__ __launch_bounds__(kThreads, 1) void staircase_pair_kernel(const StaircaseParams P)
{
    extern __shared__ __attribute__((aligned(1024))) char lds_pair[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int H = lane >> 5, r = lane & 31;
    const int n_hslots = P.num_q_heads / 2;

    // One work item per workgroup: the dispatcher hands the next item to whichever CU frees up
    // first, which balances the ragged item lengths (a fixed item -> CU assignment measured 10%
    // slower although it saves the launch gap between two workgroups of a CU).
    const int item = blockIdx.x;
    const int hslot = item % n_hslots;
    int b, rg;
    // (scratch for the numbering: in slot 4, which no K/V load targets before every wavefront has passed the core's first barrier)
    if (!locate_row_group(P, item / n_hslots, lane, reinterpret_cast<int*>(lds_pair + 4 * (2 * kTileKeys * kRowBytes)) + wave * 80, b, rg)) return;

    int seq0, L;
    seq_bounds(P, b, seq0, L);
    if (L <= 0) return;
    const int S = 1 << P.log2_s;
    const int Lp = ((L + S - 1) >> P.log2_s) << P.log2_s;
    const int pad = Lp - L;
    const int row_g0 = rg * kRowsPerWg;
    if (row_g0 >= Lp) return;

    const int heads_per_kv = P.num_q_heads / P.num_kv_heads;
    const int kvh = hslot % P.num_kv_heads;                    // launch order: KV head fastest
    const int head0 = kvh * heads_per_kv + 2 * (hslot / P.num_kv_heads);

    const int row_w0 = row_g0 + wave * 32;
    const int ip = row_w0 + r;
    const bool row_ok = ip >= pad && ip < Lp;
    const int64_t tok = (int64_t)seq0 + (ip - pad);
    // Q^T fragments, pre-multiplied by scale * log2(e) (the MFMA then yields scores in log2 units)
    typename Elem16<E>::vec8 q[2][8];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        load_q(q[h], row_ok ? P.q + tok * P.q_st + (int64_t)(head0 + h) * P.q_sh : nullptr, H);
#pragma unroll
        for (int ks = 0; ks < 8; ++ks)
#pragma unroll
            for (int j = 0; j < 8; ++j) q[h][ks][j] = (E)((float)q[h][ks][j] * P.c);
    }

    auto limit_of = [&](int row) { return min(Lp, ((row >> P.log2_s) + 1) << P.log2_s); };
    const int wg_hi = limit_of(min(row_g0 + kRowsPerWg - 1, Lp - 1));

    const unsigned lds0 = lds_address(lds_pair);
    const int l16 = lane & 15, gi = (lane >> 4) & 1;
    PairCoreArgs A;
    {   // K fragment of k-step 0: row key_of_mfma_row(r), chunk H, swizzled by row % 16
        const int row = key_of_mfma_row(r), f = row & 15;
        A.ka = lds0 + (unsigned)(row * kRowBytes + ((f & 14) << 4) + (((H ^ f) & 1) << 4));
    }
    {   // V^T fragment of d tile 0: rows rho, rho + 1; chunk c0, 8-byte half sub
        const int rho = 4 * (l16 >> 2) + 2 * H, c0 = gi * 2 + ((l16 & 3) >> 1), sub = (l16 & 1) * 8;
        const unsigned vbase = lds0 + (unsigned)(kTileKeys * kRowBytes);
        A.val = vbase + (unsigned)(rho * kRowBytes + (((rho & 12) | (c0 ^ (rho & 3))) << 4) + sub);
        A.vah = vbase + (unsigned)((rho + 1) * kRowBytes + (((rho & 12) | (c0 ^ ((rho & 3) | 1))) << 4) + sub);
    }
    A.jpl = 4 * wave + (lane >> 4);
    A.ch = (unsigned)(((lane & 15) ^ (A.jpl & 15)) * 16);
    A.wrow = (unsigned)uniform((int)(lds0 + (unsigned)(4 * wave * kRowBytes)));
    A.mrel = 2 * H - pad;
    A.mlim = limit_of(min(ip, Lp - 1)) - pad;
    A.ob0 = uniform((const void*)(P.o + ((int64_t)seq0 + (row_w0 - pad)) * P.o_st + (int64_t)head0 * P.o_sh));
    A.ob1 = uniform((const void*)(P.o + ((int64_t)seq0 + (row_w0 - pad)) * P.o_st + (int64_t)(head0 + 1) * P.o_sh));
    A.ostb = (unsigned)uniform((int)(P.o_st * 2));
    A.owave = (unsigned)uniform((int)(lds0 + (unsigned)(wave * 32 * kRowBytes)));
    A.orow0 = uniform(row_w0 - pad);
    A.olen = uniform(L);
    A.kb = uniform((const void*)(P.k + (int64_t)kvh * P.k_sh + ((int64_t)seq0 - pad) * P.k_st));
    A.vb = uniform((const void*)(P.v + (int64_t)kvh * P.v_sh + ((int64_t)seq0 - pad) * P.v_st));
    A.krb = (unsigned)uniform((int)(P.k_st * 2));
    A.vrb = (unsigned)uniform((int)(P.v_st * 2));
    A.pad = uniform(pad);
    A.lpm1 = uniform(Lp - 1);
    A.nt = uniform((wg_hi + kTileKeys - 1) / kTileKeys);
    A.whm = uniform(limit_of(min(row_w0, Lp - 1)));
    A.whx = uniform(row_w0 < Lp ? limit_of(min(row_w0 + 31, Lp - 1)) : 0);   // tiles from here on hold nothing this wavefront may see
    pair_core(A, q);
}

}  // namespace

namespace mdx {
int launch_staircase_f32(const void* q, const void* k, const void* v, void* o,
                         int64_t q_stride_t, int64_t q_stride_h, int64_t k_stride_t, int64_t k_stride_h,
                         int64_t v_stride_t, int64_t v_stride_h, int64_t o_stride_t, int64_t o_stride_h,
                         const int32_t* cu_seqlens, int32_t batch, int64_t max_l, int64_t total_tokens,
                         int32_t num_q_heads, int32_t num_kv_heads, int32_t head_dim,
                         int32_t log2_s, float scale, int32_t dtype, hipStream_t stream);      // staircase_attn_f32.hip
}

extern "C" int mdx_staircase_attn_varlen(const void* q, const void* k, const void* v, void* o,
                                         int64_t q_stride_t, int64_t q_stride_h,
                                         int64_t k_stride_t, int64_t k_stride_h,
                                         int64_t v_stride_t, int64_t v_stride_h,
                                         int64_t o_stride_t, int64_t o_stride_h,
                                         const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k,
                                         int32_t batch, int32_t max_seqlen, int64_t total_tokens,
                                         int32_t num_q_heads, int32_t num_kv_heads, int32_t head_dim,
                                         int32_t staircase_size, float scale, int32_t dtype,
                                         mdx_stream_t stream_)
{
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    MDX_REQUIRE(batch >= 0 && total_tokens >= 0 && max_seqlen >= 0, MDX_EINVAL, "staircase_attn: negative size");
    MDX_REQUIRE(dtype == MDX_BF16 || dtype == MDX_F16 || dtype == MDX_F32, MDX_EUNSUPPORTED, "staircase_attn: dtype %d (bf16, fp16 or fp32)", dtype);
    // 16-bit elements and heads of 16, 32, ..., 128 columns run on the 16-bit matrix instructions; everything else that
    // the reference's kernel takes (fp32 tensors, heads of up to 256 columns) on the fp32 one (staircase_attn_f32.hip)
    const bool f32_arithmetic = dtype == MDX_F32 || head_dim > kHeadDim || head_dim % 16 != 0;
    MDX_REQUIRE(head_dim >= 4 && head_dim <= 256 && head_dim % 4 == 0, MDX_EUNSUPPORTED,
                "staircase_attn: head_dim %d (multiples of 4 up to 256)", head_dim);
    MDX_REQUIRE(num_q_heads > 0 && num_kv_heads > 0 && num_q_heads % num_kv_heads == 0, MDX_EINVAL,
                "staircase_attn: Hq %d not a multiple of Hkv %d", num_q_heads, num_kv_heads);
    int log2_s = -1;
    for (int i = 0; i <= 7; ++i) if (staircase_size == (1 << i)) log2_s = i;
    MDX_REQUIRE(log2_s >= 0, MDX_EINVAL, "staircase_attn: staircase_size %d not in {1,2,...,128}", staircase_size);
    MDX_REQUIRE(scale > 0.f, MDX_EINVAL, "staircase_attn: scale must be positive");
    if (batch == 0 || total_tokens == 0 || max_seqlen == 0) return MDX_OK;
    MDX_REQUIRE(q && k && v && o && cu_seqlens_q && cu_seqlens_k, MDX_EINVAL, "staircase_attn: null pointer");
    MDX_REQUIRE(total_tokens < ((int64_t)1 << 31) - 256, MDX_EUNSUPPORTED, "staircase_attn: too many tokens");
    if (f32_arithmetic) {
        const int64_t longest = max_seqlen < total_tokens ? max_seqlen : total_tokens;
        return mdx::launch_staircase_f32(q, k, v, o, q_stride_t, q_stride_h, k_stride_t, k_stride_h, v_stride_t, v_stride_h,
                                         o_stride_t, o_stride_h, cu_seqlens_k, batch, longest, total_tokens, num_q_heads, num_kv_heads, head_dim,
                                         log2_s, scale, dtype, stream);
    }
    // 16-byte vector access to every row of q/k/v, 8-byte to o
    MDX_REQUIRE(mdx::aligned16(q) && mdx::aligned16(k) && mdx::aligned16(v) && mdx::aligned16(o) &&
                q_stride_t % 8 == 0 && q_stride_h % 8 == 0 && k_stride_t % 8 == 0 && k_stride_h % 8 == 0 &&
                v_stride_t % 8 == 0 && v_stride_h % 8 == 0 && o_stride_t % 4 == 0 && o_stride_h % 4 == 0,
                MDX_EUNSUPPORTED, "staircase_attn: q/k/v/o must be 16-byte aligned with strides that are multiples of 8 elements");

    const int rows_per_wg = kRowsPerWg;
    StaircaseParams P;
    P.q = (const __bf16*)q; P.k = (const __bf16*)k; P.v = (const __bf16*)v; P.o = (__bf16*)o;
    P.q_st = q_stride_t; P.q_sh = q_stride_h; P.k_st = k_stride_t; P.k_sh = k_stride_h;
    P.v_st = v_stride_t; P.v_sh = v_stride_h; P.o_st = o_stride_t; P.o_sh = o_stride_h;
    P.cu_seqlens = cu_seqlens_k;
    P.total_tokens = (int)total_tokens;
    P.batch = batch;
    const int64_t max_l = max_seqlen < total_tokens ? max_seqlen : total_tokens;
    P.n_row_groups = (int)((max_l + staircase_size - 1 + rows_per_wg - 1) / rows_per_wg);
    P.num_q_heads = num_q_heads;
    P.num_kv_heads = num_kv_heads;
    P.head_dim = head_dim;
    P.o_rows16 = (o_stride_t % 8 == 0 && o_stride_h % 8 == 0) ? 1 : 0;
    P.log2_s = log2_s;
    P.c = scale * kLog2e;
    // dense numbering: at most ceil((L_b + S - 1) / rows) row groups per sequence
    const bool dense = batch <= 64 || (P.n_row_groups <= 64 && batch <= kDenseMaxBatch);
    const int64_t n_pairs = dense ? (total_tokens + (int64_t)batch * (staircase_size + rows_per_wg - 2)) / rows_per_wg
                                  : (int64_t)P.n_row_groups * batch;
    // Two query heads per wavefront when the heads of a KV head pair up and 32-bit row offsets suffice.
    const int64_t row_elems = k_stride_t > v_stride_t ? k_stride_t : v_stride_t;
    // Sequences of a few hundred tokens are left to the one-head kernel: a pair workgroup owns a whole CU and its fixed cost (set-up,
    // prologue, epilogue: 10 us) is then most of its time, while two one-head workgroups share a CU and hide each
    // other's (one-head against pair, ms: 64 x 300 tokens 0.088 / 0.103, 32 x 500 0.074 / 0.081, 64 x 600 0.222 / 0.216,
    // 32 x 700 0.130 / 0.128, 32 x 800 0.162 / 0.155, 32 x 1000 0.230 / 0.204, 16 x 2048 0.383 / 0.304).
    const bool narrow = head_dim < kHeadDim;                   // one-head kernel, rows padded with zeros
    // (its epilogue writes rows of o in 16-byte pieces, through 32-bit byte offsets from the wavefront's first row)
    const bool pairs = !narrow && max_l > 560 && o_stride_t % 8 == 0 && o_stride_h % 8 == 0 && o_stride_t > 0 &&
                       o_stride_t * 2 * 128 < ((int64_t)1 << 31) && (num_q_heads / num_kv_heads) % 2 == 0 && k_stride_t > 0 && v_stride_t > 0 &&
                       (max_l + 2 * rows_per_wg) * row_elems * 2 < ((int64_t)1 << 31) && row_elems * 2 < (1 << 24) && max_l + 2 * rows_per_wg < (1 << 24);
    const int64_t grid = n_pairs * (pairs ? num_q_heads / 2 : num_q_heads);
    MDX_REQUIRE(grid < ((int64_t)1 << 31), MDX_EUNSUPPORTED, "staircase_attn: grid too large");
    if (pairs) {
        // the kernel's LDS limit is raised once per device (the attribute belongs to the device's copy of the kernel)
        static std::atomic<bool> lds_limit_raised[2][64];
        int device = 0;
        hipError_t e = hipGetDevice(&device);
        MDX_REQUIRE(e == hipSuccess && device >= 0 && device < 64, MDX_ELAUNCH, "staircase_attn: no current device (%s)", hipGetErrorString(e));
        const bool half = dtype == MDX_F16;
        if (!lds_limit_raised[half][device].load(std::memory_order_acquire)) {
            e = hipFuncSetAttribute(half ? reinterpret_cast<const void*>(staircase_pair_kernel<_Float16>)
                                         : reinterpret_cast<const void*>(staircase_pair_kernel<__bf16>),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, kPairLdsBytes);
            MDX_REQUIRE(e == hipSuccess, MDX_ELAUNCH, "staircase_attn: cannot reserve %d bytes of LDS (%s)", kPairLdsBytes, hipGetErrorString(e));
            lds_limit_raised[half][device].store(true, std::memory_order_release);
        }
        if (half) staircase_pair_kernel<_Float16><<<(unsigned)grid, kThreads, kPairLdsBytes, stream>>>(P);
        else      staircase_pair_kernel<__bf16><<<(unsigned)grid, kThreads, kPairLdsBytes, stream>>>(P);
    } else if (dtype == MDX_F16) {
        if (narrow) staircase_attn_kernel<_Float16, true><<<(unsigned)grid, kThreads, 0, stream>>>(P);
        else        staircase_attn_kernel<_Float16, false><<<(unsigned)grid, kThreads, 0, stream>>>(P);
    } else {
        if (narrow) staircase_attn_kernel<__bf16, true><<<(unsigned)grid, kThreads, 0, stream>>>(P);
        else        staircase_attn_kernel<__bf16, false><<<(unsigned)grid, kThreads, 0, stream>>>(P);
    }
    return mdx::check_launch("staircase_attn");
}
