// Tile arithmetic shared by the two fp32-arithmetic attention kernels (staircase_attn_f32.hip, paged_attn_f32.hip):
// the forms of the attention calls for fp32 tensors and for heads that the 16-bit kernels do not take (wider than
// 128 columns, or not a multiple of 16).  Built for exactness, not for speed: both products run on the fp32 matrix
// instruction (v_mfma_f32_32x32x2_f32), the probabilities are never rounded, 16-bit inputs are widened on their way
// into LDS.
//
// Products are transposed (S^T = K Q^T, O^T = V^T P^T), as in the 16-bit kernels, so that a query is a column of the
// matrix instruction and lives in the lane pair (r, r + 32): the softmax over keys is arithmetic inside a lane plus
// one exchange with the other half-wavefront.  A wavefront owns 32 queries of one head; K and V tiles of 32 keys sit
// in LDS as fp32.
#pragma once
#include "mdx_common.h"

namespace mdx_attn_f32 {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int kTileKeys = 32;
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kMinusBig = -1.0e30f;

// Four consecutive elements as floats (the pointer is 16-byte aligned for fp32, 8-byte for 16-bit elements).
__device__ __forceinline__ f32x4 load4(const float* p) { return *reinterpret_cast<const f32x4*>(p); }
__device__ __forceinline__ f32x4 load4(const __bf16* p) {
    const uint2 raw = *reinterpret_cast<const uint2*>(p);
    return f32x4{__uint_as_float(raw.x << 16), __uint_as_float(raw.x & 0xffff0000u),
                 __uint_as_float(raw.y << 16), __uint_as_float(raw.y & 0xffff0000u)};
}
__device__ __forceinline__ f32x4 load4(const _Float16* p) {
    typedef _Float16 h4 __attribute__((ext_vector_type(4)));
    const h4 raw = *reinterpret_cast<const h4*>(p);
    return f32x4{(float)raw[0], (float)raw[1], (float)raw[2], (float)raw[3]};
}
__device__ __forceinline__ void store4(float* p, f32x4 v) { *reinterpret_cast<f32x4*>(p) = v; }
__device__ __forceinline__ void store4(__bf16* p, f32x4 v) {
    typedef __bf16 b4 __attribute__((ext_vector_type(4)));
    *reinterpret_cast<b4*>(p) = b4{(__bf16)v[0], (__bf16)v[1], (__bf16)v[2], (__bf16)v[3]};
}
__device__ __forceinline__ void store4(_Float16* p, f32x4 v) {
    typedef _Float16 h4 __attribute__((ext_vector_type(4)));
    *reinterpret_cast<h4*>(p) = h4{(_Float16)v[0], (_Float16)v[1], (_Float16)v[2], (_Float16)v[3]};
}

// Row of the 32 x 32 result that accumulator register i of a lane in half-wavefront H holds.
__device__ __forceinline__ int row_of_reg(int i, int H) { return 8 * (i >> 2) + 4 * H + (i & 3); }

// D: 128 or 256, the head width that registers and LDS are laid out for (narrower heads are padded with zeros;
// products over the padding are skipped).
template <int D> struct Lds {
    // floats; rows stay 16-byte aligned and consecutive rows shift by 4 banks: the 16-byte reads of 8 consecutive keys
    // (K fragments: four columns of a key per read) cover all banks once, and so do the two keys of a V k-step
    static constexpr int kPitchK = D + 4;
    static constexpr int kPitchV = D + 4;
    static constexpr int kFloats = kTileKeys * (kPitchK + kPitchV);
    static constexpr int kBytes = kFloats * (int)sizeof(float);
    static __device__ __forceinline__ float* k_tile(float* lds) { return lds; }
    static __device__ __forceinline__ float* v_tile(float* lds) { return lds + kTileKeys * kPitchK; }
};

// One query's row of Q^T for lane (H, r): the elements d = 2 j + H (row may be null: zeros).
template <typename T, int D>
__device__ __forceinline__ void load_q(float (&q)[D / 2], const T* row, int H, int width) {
#pragma unroll
    for (int m = 0; m < D / 4; ++m) {
        f32x4 x = f32x4{0.f, 0.f, 0.f, 0.f};
        if (row && 4 * m < width) x = load4(row + 4 * m);
        q[2 * m] = H ? x[1] : x[0];
        q[2 * m + 1] = H ? x[3] : x[2];
    }
}

// Row `row` of the K and V tiles, columns 4 c4 .. 4 c4 + 3 (null pointers: zeros).
template <typename T, int D>
__device__ __forceinline__ void stage4(float* lds, int row, int c4, const T* k4, const T* v4) {
    f32x4 kx = f32x4{0.f, 0.f, 0.f, 0.f}, vx = kx;
    if (k4) { kx = load4(k4); vx = load4(v4); }
    *reinterpret_cast<f32x4*>(Lds<D>::k_tile(lds) + row * Lds<D>::kPitchK + 4 * c4) = kx;
    *reinterpret_cast<f32x4*>(Lds<D>::v_tile(lds) + row * Lds<D>::kPitchV + 4 * c4) = vx;
}

// Running softmax state of a wavefront's 32 queries: l is this half-wavefront's share of the row sum.
template <int D> struct State {
    float m, l;
    f32x16 o[D / 32];
    __device__ __forceinline__ void init() {
        m = kMinusBig; l = 0.f;
#pragma unroll
        for (int dt = 0; dt < D / 32; ++dt)
#pragma unroll
            for (int i = 0; i < 16; ++i) o[dt][i] = 0.f;
    }
};

// One tile of 32 keys against the wavefront's 32 queries.  visible(key in tile) says whether this lane's query sees it.
template <int D, typename Visible>
__device__ __forceinline__ void tile_step(const float* lds, const float (&q)[D / 2], State<D>& st, float c, int width, int lane, Visible visible)
{
    const int H = lane >> 5, r = lane & 31;
    // ---- S^T = K Q^T: rows = keys, columns = queries; k-step j covers d = 2 j, 2 j + 1 (half-wavefront H holds d = 2 j + H);
    //      a 16-byte read of key r's columns 4 m .. 4 m + 3 feeds the k-steps 2 m and 2 m + 1 ----
    f32x16 s;
#pragma unroll
    for (int i = 0; i < 16; ++i) s[i] = 0.f;
    const float* krow = Lds<D>::k_tile(const_cast<float*>(lds)) + r * Lds<D>::kPitchK;
#pragma unroll
    for (int m = 0; m < D / 4; ++m) {
        if (4 * m >= width) continue;
        const f32x4 kx = *reinterpret_cast<const f32x4*>(krow + 4 * m);
        s = __builtin_amdgcn_mfma_f32_32x32x2f32(H ? kx[1] : kx[0], q[2 * m], s, 0, 0, 0);
        s = __builtin_amdgcn_mfma_f32_32x32x2f32(H ? kx[3] : kx[2], q[2 * m + 1], s, 0, 0, 0);
    }

    // ---- online softmax over the keys, base 2 ----
    float mx = kMinusBig;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        s[i] = visible(row_of_reg(i, H)) ? s[i] * c : -INFINITY;
        mx = fmaxf(mx, s[i]);
    }
    mx = fmaxf(mx, __shfl_xor(mx, 32));
    const float m_new = fmaxf(st.m, mx);
    const float alpha = __builtin_amdgcn_exp2f(st.m - m_new);
    float sum = 0.f;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        s[i] = __builtin_amdgcn_exp2f(s[i] - m_new);
        sum += s[i];
    }
    st.l = st.l * alpha + sum;
    st.m = m_new;
#pragma unroll
    for (int dt = 0; dt < D / 32; ++dt)
#pragma unroll
        for (int i = 0; i < 16; ++i) st.o[dt][i] *= alpha;

    // ---- O^T += V^T P^T: rows = d, columns = queries; k-step (g, e) covers the keys 8 g + e and 8 g + 4 + e,
    //      which are the keys of this lane's register 4 g + e in the two half-wavefronts ----
#pragma unroll
    for (int dt = 0; dt < D / 32; ++dt) {
        if (dt * 32 >= width) continue;
        const float* vcol = Lds<D>::v_tile(const_cast<float*>(lds)) + dt * 32 + r;
#pragma unroll
        for (int i = 0; i < 16; ++i)
            st.o[dt] = __builtin_amdgcn_mfma_f32_32x32x2f32(vcol[row_of_reg(i, H) * Lds<D>::kPitchV], s[i], st.o[dt], 0, 0, 0);
    }
}

// O = O^T / l into this lane's query row (4 consecutive d per (d tile, register group)); a row that saw no key: zeros.
template <typename T, int D>
__device__ __forceinline__ void store_o(T* orow, const State<D>& st, int H, int width) {
    const float l_all = st.l + __shfl_xor(st.l, 32);
    const float inv = l_all > 0.f ? 1.0f / l_all : 0.f;
    if (!orow) return;
#pragma unroll
    for (int dt = 0; dt < D / 32; ++dt)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const int d = dt * 32 + 8 * g + 4 * H;
            if (d < width) store4(orow + d, f32x4{st.o[dt][4 * g] * inv, st.o[dt][4 * g + 1] * inv, st.o[dt][4 * g + 2] * inv, st.o[dt][4 * g + 3] * inv});
        }
}

}  // namespace mdx_attn_f32
