// Wavefront-level building block shared by the two attention kernels
// (staircase block-prefill and paged single-block decode), head_dim 128, bf16 or fp16 (pointers are
// typed __bf16 throughout as "16-bit element"; the element type E of a kernel says what the bits mean).
//
// One wavefront owns 32 query rows (one MFMA column tile) of NH query heads that share a KV
// head and walks over keys 32 at a time:
//
//   S^T[key, query]  = K[key, :] . Q[query, :]      v_mfma_f32_32x32x16_bf16, A = K (LDS), B = Q^T (registers)
//   online softmax   per query = per LANE            row max / sum live in the lane, one permlane32_swap per step
//   O^T[d, query]   += V^T[d, key] . P^T[key, query] A = V^T (LDS, ds_read_b64_tr_b16), B = P^T (registers)
//
// Computing the transposed products keeps each query in one lane (l % 32), so
// the softmax needs no cross-lane reduction beyond the two half-waves, and the
// S^T accumulator registers are already in B-operand order for the second
// product: no shuffles between the two MFMAs.
//
// Register/lane maps used throughout (l = lane, H = l / 32):
//   MFMA A operand: lane holds row l%32, k = 8H..8H+7;  B operand: column l%32, k = 8H..8H+7
//   MFMA C/D:       register i holds row 8*(i/4) + 4H + i%4, column l%32
// The contraction index of the second product may be permuted freely as long
// as both operands agree, and so may the assignment of keys to MFMA rows of the
// first product.  Keys are assigned so that accumulator register i of half H
// holds key  key_of_reg(i, H) = 16*(i/8) + 4*(i%4) + 2H + (i/4)%2  of the
// 32-key sub-tile; registers 8t..8t+7 are then exactly the B operand of PV
// k-step t, whose A operand is fetched by two transposing LDS reads of rows
// 16t + 4j + 2H + q (j = 0..3, q = 0,1): rows 4 apart, which with the 272-byte
// row pitch land in disjoint bank groups.
#pragma once
#include <hip/hip_runtime.h>
#include <cstdint>
#include "mdx_common.h"

namespace mdx_attn {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((ext_vector_type(8))) short s16x8;

constexpr int kHeadDim = 128;
constexpr int kRowBytes = kHeadDim * 2;      // one K or V row of one head
constexpr int kLdsPitch = kRowBytes + 16;    // 272: consecutive rows shift by 4 banks
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kMinusBig = -1.0e30f;        // finite initial running max (avoids inf - inf)
constexpr float kMaxSlack = 8.0f;            // running max may lag by up to 2^8 before O is rescaled

// The two 16-bit element types the tile code runs in.  Everything that moves K/V/Q bytes is type-blind
// (16-byte copies); the type decides the MFMA instruction and the two float -> element conversions
// (probabilities, output).
template <typename E> struct Elem16;
template <> struct Elem16<__bf16> {
    typedef bf16x8 vec8;
    typedef __attribute__((ext_vector_type(4))) __bf16 vec4;
    static __device__ __forceinline__ f32x16 mfma(vec8 a, vec8 b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0); }
};
template <> struct Elem16<_Float16> {
    typedef f16x8 vec8;
    typedef __attribute__((ext_vector_type(4))) _Float16 vec4;
    static __device__ __forceinline__ f32x16 mfma(vec8 a, vec8 b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0); }
};

__device__ __forceinline__ int key_of_reg(int i, int H) {
    return 16 * (i >> 3) + 4 * (i & 3) + 2 * H + ((i >> 2) & 1);
}
// LDS row read by the lane that feeds MFMA row r of the first product.
__device__ __forceinline__ int key_of_mfma_row(int r) {
    return (r & 16) | ((r & 3) << 2) | (((r >> 2) & 1) << 1) | ((r >> 3) & 1);
}

__device__ __forceinline__ float other_half_max(float x) {
    // permlane32_swap(x, x): element 0 = x of lane l%32, element 1 = x of lane l%32 + 32
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float both_halves_sum(float x) {
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

typedef __attribute__((address_space(3))) char lds_char;
typedef __attribute__((address_space(3))) s16x4 lds_s16x4;

// 32-bit LDS byte address of a pointer into shared memory (what ds_* instructions take).
__device__ __forceinline__ unsigned lds_address(const void* p) {
    return (unsigned)(uintptr_t)(const lds_char*)p;
}

// Running state of one wavefront: NH heads x 32 queries.  With NH = 2 the two query heads of a
// grouped-query pair share every K and V fragment fetched from LDS (half the LDS bytes per MFMA).
template <int NH>
struct WaveState {
    float m[NH];            // running max, in log2 units (score * scale * log2 e); same in both half-waves
    float l[NH];            // running sum of this half-wave's keys only
    f32x16 o[NH][4];        // O^T: 4 tiles of 32 d-rows x 32 queries
    __device__ __forceinline__ void init() {
#pragma unroll
        for (int h = 0; h < NH; ++h) {
            m[h] = kMinusBig;
            l[h] = 0.f;
#pragma unroll
            for (int t = 0; t < 4; ++t)
#pragma unroll
                for (int i = 0; i < 16; ++i) o[h][t][i] = 0.f;
        }
    }
};

// The three phases of one online-softmax step over NSUB*32 keys held in LDS rows
// n0 .. n0+NSUB*32-1 of tiles with row pitch kLdsPitch.

// S^T = K Q^T.  q[h][ks] are the B-operand fragments of Q^T for d = 16ks .. 16ks+15.
// Columns from `width` on (a multiple of 16) are zeros on both sides and skipped.
template <typename E, int NH, int NSUB>
__device__ __forceinline__ void qk_phase(const char* lds_k, int n0, const typename Elem16<E>::vec8 (&q)[NH][8], f32x16 (&s)[NH][NSUB], int lane,
                                         int width = kHeadDim)
{
    typedef typename Elem16<E>::vec8 vec8;
    const int H = lane >> 5, r = lane & 31;
#pragma unroll
    for (int h = 0; h < NH; ++h)
#pragma unroll
        for (int u = 0; u < NSUB; ++u)
#pragma unroll
            for (int i = 0; i < 16; ++i) s[h][u][i] = 0.f;
    const char* kbase = lds_k + (n0 + key_of_mfma_row(r)) * kLdsPitch + H * 16;
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) {
        if (ks * 16 >= width) break;
#pragma unroll
        for (int u = 0; u < NSUB; ++u) {
            const vec8 kf = *reinterpret_cast<const vec8*>(kbase + u * 32 * kLdsPitch + ks * 32);
#pragma unroll
            for (int h = 0; h < NH; ++h)
                s[h][u] = Elem16<E>::mfma(kf, q[h][ks], s[h][u]);
        }
    }
}

// Online softmax, per lane = per query.  c = softmax scale * log2(e) (> 0).
// MASK: keys with absolute index outside [key_lo, key_hi) are excluded; key_abs0 is the
// absolute index of LDS row n0; key_hi may differ per lane (per query), key_lo is uniform.
// Produces the bf16 B-operand fragments p[h][u][t] of P^T and updates m, l and (when the
// running max moves) rescales O.
template <typename E, int NH, int NSUB, bool MASK>
__device__ __forceinline__ void softmax_phase(f32x16 (&s)[NH][NSUB], typename Elem16<E>::vec8 (&p)[NH][NSUB][2], WaveState<NH>& st, float c,
                                              int lane, int key_abs0, int key_lo, int key_hi)
{
    const int H = lane >> 5;
#pragma unroll
    for (int h = 0; h < NH; ++h) {
        if (MASK) {
#pragma unroll
            for (int u = 0; u < NSUB; ++u)
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const int key = key_abs0 + 32 * u + key_of_reg(i, H);
                    s[h][u][i] = (key >= key_lo && key < key_hi) ? s[h][u][i] : -INFINITY;
                }
        }
        float mx = s[h][0][0];
#pragma unroll
        for (int u = 0; u < NSUB; ++u)
#pragma unroll
            for (int i = 0; i < 16; ++i) mx = fmaxf(mx, s[h][u][i]);
        mx = other_half_max(mx);
        // Lazy rescale: the running max only moves when some query's new max exceeds it by more
        // than kMaxSlack (log2 units).  Until then probabilities are taken relative to the stale
        // max (at most 2^kMaxSlack, harmless in fp32/bf16) and O, l need no rescaling; the final
        // O / l is unchanged because numerator and denominator share the same reference.
        const float m_cand = fmaxf(st.m[h], mx * c);
        const bool moved = __any(m_cand > st.m[h] + kMaxSlack);         // wave-uniform
        const float m_new = moved ? m_cand : st.m[h];
        float sum = 0.f;
#pragma unroll
        for (int u = 0; u < NSUB; ++u)
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const float e = __builtin_amdgcn_exp2f(fmaf(s[h][u][8 * t + j], c, -m_new));
                    sum += e;
                    p[h][u][t][j] = (E)e;
                }
        if (moved) {
            const float alpha = __builtin_amdgcn_exp2f(st.m[h] - m_new);
            st.l[h] *= alpha;
#pragma unroll
            for (int t = 0; t < 4; ++t)
#pragma unroll
                for (int i = 0; i < 16; ++i) st.o[h][t][i] *= alpha;
            st.m[h] = m_new;
        }
        st.l[h] += sum;
    }
}

// O^T += V^T P^T.  The lane supplies the row address for the transposing read:
// row 4*(i'/4) + 2H (+q), d chunk i'%4, with i' = lane % 16.
// O^T tiles whose 32 rows all lie beyond `width` stay zero and are skipped.
template <typename E, int NH, int NSUB>
__device__ __forceinline__ void pv_phase(const char* lds_v, int n0, const typename Elem16<E>::vec8 (&p)[NH][NSUB][2], WaveState<NH>& st, int lane,
                                         int width = kHeadDim)
{
    typedef typename Elem16<E>::vec8 vec8;
    const int H = lane >> 5, ip = lane & 15, gi = (lane >> 4) & 1;
    const lds_char* vbase = (const lds_char*)lds_v + (n0 + 4 * (ip >> 2) + 2 * H) * kLdsPitch + (gi * 16 + (ip & 3) * 4) * 2;
#pragma unroll
    for (int u = 0; u < NSUB; ++u)
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int dt = 0; dt < 4; ++dt) {
                if (dt * 32 >= width) break;
                const lds_char* a = vbase + (u * 32 + t * 16) * kLdsPitch + dt * 64;
                const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)a);
                const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(a + kLdsPitch));
                const s16x8 both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
                const vec8 vf = __builtin_bit_cast(vec8, both);
#pragma unroll
                for (int h = 0; h < NH; ++h)
                    st.o[h][dt] = Elem16<E>::mfma(vf, p[h][u][t], st.o[h][dt]);
            }
}

// All three phases back to back.
template <typename E, int NH, int NSUB, bool MASK>
__device__ __forceinline__ void attn_step(const char* lds_k, const char* lds_v, int n0, const typename Elem16<E>::vec8 (&q)[NH][8],
                                          WaveState<NH>& st, float c, int lane, int key_abs0, int key_lo, int key_hi, int width = kHeadDim)
{
    f32x16 s[NH][NSUB];
    typename Elem16<E>::vec8 p[NH][NSUB][2];
    qk_phase<E, NH, NSUB>(lds_k, n0, q, s, lane, width);
    softmax_phase<E, NH, NSUB, MASK>(s, p, st, c, lane, key_abs0, key_lo, key_hi);
    pv_phase<E, NH, NSUB>(lds_v, n0, p, st, lane, width);
}

// d index held by accumulator register i of O^T tile dt in half-wave H.
__device__ __forceinline__ int d_of_reg(int dt, int i, int H) { return dt * 32 + 8 * (i >> 2) + 4 * H + (i & 3); }

// Loads the Q^T B-operand fragments of one head for this lane's query row
// (row pointer may be null: zeros).  q_row points at Q[query, head, 0]; a head narrower than 128
// (width: a multiple of 16) is padded with zeros.
template <typename V8>
__device__ __forceinline__ void load_q(V8 (&q)[8], const __bf16* q_row, int H, int width = kHeadDim) {
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) {
        if (q_row && ks * 16 < width) {
            q[ks] = *reinterpret_cast<const V8*>(q_row + ks * 16 + H * 8);
        } else {
#pragma unroll
            for (int j = 0; j < 8; ++j) q[ks][j] = 0;
        }
    }
}

// Global -> register staging of one K/V tile of TK rows x 256 B by T threads:
// thread t moves chunk t%16 (16 B) of rows t/16, t/16 + T/16, ...
template <int TK, int T>
struct TileRegs {
    static constexpr int kPasses = TK * 16 / T;
    static_assert(kPasses >= 1 && (TK * 16) % T == 0, "tile does not divide over the workgroup");
    u32x4 k[kPasses];
    u32x4 v[kPasses];
};

template <int TK, int T>
__device__ __forceinline__ void store_tile(char* lds_k, char* lds_v, const TileRegs<TK, T>& regs, int tid) {
    const int chunk = tid & 15, row0 = tid >> 4;
#pragma unroll
    for (int p = 0; p < TileRegs<TK, T>::kPasses; ++p) {
        const int off = (row0 + (T / 16) * p) * kLdsPitch + chunk * 16;
        *reinterpret_cast<u32x4*>(lds_k + off) = regs.k[p];
        *reinterpret_cast<u32x4*>(lds_v + off) = regs.v[p];
    }
}

}  // namespace mdx_attn
