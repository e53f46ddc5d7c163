// The per-block confidence unmask step: softmax confidence + first-index argmax
// over the vocabulary, then threshold / top-k selection of masked positions.
//
// The vocabulary pass is a single HBM stream over the logits (311 MB at
// [32 x 32 x 151936] bf16), so it is built for bandwidth, not MFMA: 16-byte
// coalesced loads, several in flight per lane, an online (max, sum-of-exp)
// pair per lane that is only rescaled when a 16-byte chunk raises the running
// maximum, wavefront shuffles and one LDS hop for the row reduction.  The
// argmax is found without per-element index bookkeeping: a lane notes the
// position of a new maximum only when a 16-byte chunk raises its running maximum,
// while that chunk is still in registers.
//
// Semantics follow engines/nano_dvlm/nanovllm/layers/sampler.py:11-61 and
// mineru_diffusion/modeling_mineru_diffusion.py:518-532.
#include "mdx_common.h"
#include <hip/hip_fp16.h>

namespace {

constexpr int kThreads = 256;
constexpr int kUnroll = 2;               // 16-byte loads in flight per lane
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kNegBig = -3.0e38f;      // finite stand-in for -inf: keeps (m - m) away from inf - inf
constexpr int kNoIndex = 0x7fffffff;

struct Partial {                         // one row's (or row split's) running state
    float m;                             // max of the raw logits seen
    float s;                             // sum of exp((x - m)/T)
    int idx;                             // first index holding m
    float pick;                          // with noise: best (x/T + g); else unused
    float pick_x;                        // with noise: raw logit at that index
    int pick_idx;                        // with noise: first index of the best
};

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// max of three in one instruction.  fmaxf(fmaxf(a, b), c) costs the compiler two more instructions per
// freshly unpacked pair, to quiet signalling NaNs that logits do not hold.
__device__ __forceinline__ float max3(float a, float b, float c) {
    float r;
    asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}

// Combine b into a.  c = log2(e)/T.
__device__ __forceinline__ void combine(Partial& a, const Partial& b, float c, bool noise) {
    const float M = fmaxf(a.m, b.m);
    a.s = a.s * fast_exp2((a.m - M) * c) + b.s * fast_exp2((b.m - M) * c);
    a.idx = (b.m > a.m) ? b.idx : ((b.m == a.m) ? min(a.idx, b.idx) : a.idx);
    a.m = M;
    if (noise) {
        const bool take = (b.pick > a.pick) || (b.pick == a.pick && b.pick_idx < a.pick_idx);
        if (take) { a.pick = b.pick; a.pick_x = b.pick_x; a.pick_idx = b.pick_idx; }
    }
}

__device__ __forceinline__ Partial shfl_xor(const Partial& p, int mask, bool noise) {
    Partial r;
    r.m = __shfl_xor(p.m, mask);
    r.s = __shfl_xor(p.s, mask);
    r.idx = __shfl_xor(p.idx, mask);
    if (noise) {
        r.pick = __shfl_xor(p.pick, mask);
        r.pick_x = __shfl_xor(p.pick_x, mask);
        r.pick_idx = __shfl_xor(p.pick_idx, mask);
    } else {
        r.pick = kNegBig; r.pick_x = 0.f; r.pick_idx = kNoIndex;
    }
    return r;
}

// A row's final answer.  A row without any finite logit (all -inf) has no softmax: it reports
// token 0 (where an argmax over equal values lands) with confidence 0, so no rule ever commits it.
template <bool NOISE>
__device__ __forceinline__ void finish_row(const Partial& r, float c, int64_t& x0, float& x0_p) {
    if (r.idx == kNoIndex) { x0 = 0; x0_p = 0.f; return; }
    if (NOISE) {
        x0 = r.pick_idx;
        x0_p = fast_exp2((r.pick_x - r.m) * c) / r.s;
    } else {
        x0 = r.idx;
        x0_p = fminf(1.0f / r.s, 1.0f);          // the sum holds exp2(0) up to rounding
    }
}

// --- element access by logits type: EPC = elements per 16-byte chunk ---------
template <typename T> struct Elem;
template <> struct Elem<__bf16> {
    static constexpr int EPC = 8;
    static __device__ __forceinline__ void unpack(const u32x4& u, float* x) {
        const uint32_t w[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            x[2 * i] = __uint_as_float(w[i] << 16);
            x[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
        }
    }
    static __device__ __forceinline__ float one(const __bf16* p) {
        return __uint_as_float((uint32_t)(*reinterpret_cast<const uint16_t*>(p)) << 16);
    }
};
template <> struct Elem<__half> {
    static constexpr int EPC = 8;
    static __device__ __forceinline__ void unpack(const u32x4& u, float* x) {
        const __half2* h = reinterpret_cast<const __half2*>(&u);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float2 f = __half22float2(h[i]);
            x[2 * i] = f.x;
            x[2 * i + 1] = f.y;
        }
    }
    static __device__ __forceinline__ float one(const __half* p) { return __half2float(*p); }
};
template <> struct Elem<float> {
    static constexpr int EPC = 4;
    static __device__ __forceinline__ void unpack(const u32x4& u, float* x) {
        x[0] = __uint_as_float(u.x); x[1] = __uint_as_float(u.y);
        x[2] = __uint_as_float(u.z); x[3] = __uint_as_float(u.w);
    }
    static __device__ __forceinline__ float one(const float* p) { return *p; }
};

// One element through the slow path (row head/tail).  With noise, l = x / T is a
// true fp32 division so the noisy argmax matches an fp32 host computation bit for bit.
template <bool NOISE>
__device__ __forceinline__ void visit(Partial& p, float x, int index, float c, float T, float g) {
    if (x > p.m) {
        p.s *= fast_exp2((p.m - x) * c);
        p.m = x;
        p.idx = index;
    } else if (x == p.m && index < p.idx) {
        p.idx = index;
    }
    p.s += fast_exp2((x - p.m) * c);
    if (NOISE) {
        const float l = x / T;
        const float v = l + g;
        if (v > p.pick || (v == p.pick && index < p.pick_idx)) { p.pick = v; p.pick_x = x; p.pick_idx = index; }
    }
}

// --- Gumbel noise drawn in the kernel ------------------------------------------------------------
// Sampler.prepare draws gumbel = -log(Exponential(1)) per logit (sampler.py:15-16).  Here the draw is
// a pure function of (seed, offset, row, column): Philox-4x32-10 (Salmon et al., "Parallel random
// numbers: as easy as 1, 2, 3", 2011) with key = seed and counter = (column / 4, row, offset), whose
// four 32-bit outputs serve columns 4*(column/4) .. +3.  So the noise does not depend on the launch
// geometry, a caller reproduces a step from three integers, and nothing is read from memory.
struct NoiseSpec {
    const float* noise; int64_t noise_row_stride;      // explicit noise tensor, or
    bool philox; uint32_t key0, key1;                   // noise from the generator: seed,
    uint64_t offset; const int64_t* offset_dev;         // offset (+ *offset_dev when given: a counter a graph replay can advance),
    const int64_t* row_ids;                             // and the row coordinate of each logits row (NULL: the row's own index)
};

struct U4 { uint32_t x, y, z, w; };

__device__ __forceinline__ U4 philox4x32_10(U4 c, uint32_t k0, uint32_t k1) {
#pragma unroll
    for (int r = 0; r < 10; ++r) {
        // one 32 x 32 -> 64 multiply per product (v_mad_u64_u32) instead of a high and a low one: 32-bit integer
        // multiplies are what this generator costs, and the full-width form is 6.5 % faster over a logits pass
        const uint64_t p0 = (uint64_t)0xD2511F53u * (uint64_t)c.x, p1 = (uint64_t)0xCD9E8D57u * (uint64_t)c.z;
        const uint32_t hi0 = (uint32_t)(p0 >> 32), lo0 = (uint32_t)p0, hi1 = (uint32_t)(p1 >> 32), lo1 = (uint32_t)p1;
        c = U4{hi1 ^ c.y ^ k0, lo1, hi0 ^ c.w ^ k1, lo0};
        k0 += 0x9E3779B9u;
        k1 += 0xBB67AE85u;
    }
    return c;
}

// 32 random bits -> u = (top 23 bits + 1/2) / 2^23 in (0, 1) -> -ln(-ln u), the negated logarithm of a unit
// exponential.  With t = log2 u: -ln(-ln u) = -ln 2 * log2(-t) - ln(ln 2).  The largest noise values, the ones
// that decide an argmax, come from u next to 1, where t is tiny: the hardware logarithm keeps its relative
// accuracy there (over all 2^23 values of u the result is within 2e-6 of the fp64 one).
constexpr float kGumbelMax = 17.0f;      // above every value of gumbel_of (16.64 at u = 1 - 2^-24)
__device__ __forceinline__ float gumbel_of(uint32_t bits) {
    const float u = __builtin_fmaf((float)(bits >> 9), 1.1920928955078125e-07f, 5.9604644775390625e-08f);   // (k + 1/2) * 2^-23
    const float t = __builtin_amdgcn_logf(u);
    return __builtin_fmaf(-0.69314718055994531f, __builtin_amdgcn_logf(-t), 0.36651292058166435f);
}

struct RowNoise {                       // the generator's coordinates of one logits row
    uint32_t key0, key1, row, off_lo, off_hi;
    __device__ __forceinline__ U4 group(uint32_t column_group) const {
        return philox4x32_10(U4{column_group, row, off_lo, off_hi}, key0, key1);
    }
    __device__ __forceinline__ float at(int column) const {
        const U4 r = group((uint32_t)column >> 2);
        const uint32_t b[4] = {r.x, r.y, r.z, r.w};
        return gumbel_of(b[column & 3]);
    }
};

__device__ __forceinline__ RowNoise row_noise(const NoiseSpec& N, int64_t row) {
    const uint64_t off = N.offset + (N.offset_dev ? (uint64_t)*N.offset_dev : 0ull);
    const int64_t rid = N.row_ids ? N.row_ids[row] : row;
    return RowNoise{N.key0, N.key1, (uint32_t)rid, (uint32_t)off, (uint32_t)(off >> 32)};
}

// grid = (rows, nsplit).  Each workgroup reduces chunks [split*cps, (split+1)*cps)
// of one row; split 0 also takes the unaligned head and tail elements.
// NOISE: 0 = plain argmax, 1 = noise read from a tensor, 2 = noise drawn in the kernel.
template <typename T, int NOISE>
__global__ __launch_bounds__(kThreads) void confidence_argmax_kernel(
    const T* __restrict__ logits, int64_t row_stride,
    const float* __restrict__ temperatures, int rows_per_temp,
    const NoiseSpec N,
    int64_t vocab, int nsplit,
    Partial* __restrict__ partials,          // [rows, nsplit] when nsplit > 1
    int64_t* __restrict__ x0, float* __restrict__ x0_p)
{
    constexpr int EPC = Elem<T>::EPC;
    const int64_t row = blockIdx.x;
    const int split = blockIdx.y;
    const int tid = threadIdx.x;
    const T* rp = logits + row * row_stride;
    const float* np = NOISE == 1 ? N.noise + row * N.noise_row_stride : nullptr;
    const float T_ = temperatures ? temperatures[row / rows_per_temp] : 1.0f;
    const float c = kLog2e / T_;

    // Row geometry: `lead` scalar elements up to the first 16-byte boundary,
    // `nchunk` aligned chunks, then a scalar tail.
    const uintptr_t addr = reinterpret_cast<uintptr_t>(rp);
    int64_t lead = ((16 - (addr & 15)) & 15) / sizeof(T);
    if (lead > vocab) lead = vocab;
    const int64_t nchunk = (vocab - lead) / EPC;
    const int64_t tail0 = lead + nchunk * EPC;
    const u32x4* cp = reinterpret_cast<const u32x4*>(rp + lead);

    const int64_t cps = (nchunk + nsplit - 1) / nsplit;      // chunks per split
    const int64_t cbeg = split * cps;
    const int64_t cend = min(nchunk, cbeg + cps);

    Partial p;
    p.m = kNegBig; p.s = 0.f; p.idx = kNoIndex; p.pick = kNegBig; p.pick_x = 0.f; p.pick_idx = kNoIndex;
    __shared__ float lead_seen;              // mode 2: the best noisy logit any wavefront of the workgroup has published
    if (NOISE == 2) {
        if (tid == 0) lead_seen = kNegBig;
        __syncthreads();
    }

    // Softmax over 16-byte chunks (modes 0 and 2).  Per lane: running max m, h = -(m * c) rounded to fp32,
    // and s = sum of exp2(x * c + h), each exponent one FMA (x * c + h is rounded once, so the term of x == m is exp2(lo) with
    // lo = m * c + h, the rounding error of the product, known exactly).  The sum that the row
    // reduction wants, sum of exp2((x - m) * c), is s * exp2(-lo): applied once per lane after
    // the loop.  Folding m * c into the FMA without that correction would carry its rounding,
    // 2^-24 |m c|, into every term (1e-3 at logits of thousands).
    float m = kNegBig, s = 0.f, h = 0.f;
    int first_at = -1;           // element (counted from the first aligned chunk) that first held m
    auto take_values = [&](const float (&x)[EPC], int64_t chunk) -> float {     // returns the chunk's largest element
        float cm = x[EPC - 1];
#pragma unroll
        for (int i = 0; i + 2 < EPC; i += 2) cm = max3(cm, x[i], x[i + 1]);
        if (EPC % 2 == 0) cm = max3(cm, x[EPC - 2], x[EPC - 2]);
        if (cm > m) {
            // found here, while the chunk is in registers: reading it again at the end
            // would fetch a whole cache line per lane from HBM (10 % more traffic)
            int j = EPC - 1;
#pragma unroll
            for (int i = EPC - 2; i >= 0; --i) if (x[i] == cm) j = i;
            first_at = (int)chunk * EPC + j;
            const float h_new = -(cm * c);
            s = s > 0.f ? s * fast_exp2(h_new - h) : 0.f;   // h_new <= h once a finite maximum exists
            m = cm;
            h = h_new;
        }
        float acc = fast_exp2(__builtin_fmaf(x[0], c, h));
#pragma unroll
        for (int i = 1; i < EPC; ++i) acc += fast_exp2(__builtin_fmaf(x[i], c, h));
        s += acc;
        return cm;
    };
    auto lane_softmax_done = [&]() {
        if (m > kNegBig) s *= fast_exp2(-__builtin_fmaf(m, c, h));   // to the base of m itself (a lane that saw no finite element keeps s == 0)
        p.m = m;
        p.s = s;
        if (first_at >= 0) p.idx = (int)lead + first_at;
    };

    if (NOISE == 0) {
        auto take = [&](const u32x4 u, int64_t chunk) {
            float x[EPC];
            Elem<T>::unpack(u, x);
            take_values(x, chunk);
        };
        int64_t ch = cbeg + tid;
        // Main loop: the next group's kUnroll loads are issued before this group is reduced, so a lane
        // always has loads outstanding while it computes (measured on [1024 x 151936] bf16: 53.7 -> 50.9 us
        // for the step with two loads per group; four per group, or alternating between two register
        // sets instead of handing the prefetched group over, are 3 to 5 % slower).
        constexpr int64_t kStep = (int64_t)kUnroll * kThreads;
        auto have = [&](int64_t at) { return at + kStep - kThreads < cend; };
        auto fetch = [&](u32x4 (&r)[kUnroll], int64_t at) {
#pragma unroll
            for (int k = 0; k < kUnroll; ++k) r[k] = __builtin_nontemporal_load(cp + at + (int64_t)k * kThreads);
        };
        auto reduce = [&](const u32x4 (&r)[kUnroll], int64_t at) {
#pragma unroll
            for (int k = 0; k < kUnroll; ++k) take(r[k], at + (int64_t)k * kThreads);
        };
        u32x4 u[kUnroll];
        if (have(ch)) fetch(u, ch);
        for (; have(ch); ch += kStep) {
            const bool more = have(ch + kStep);
            u32x4 w[kUnroll];
            if (more) fetch(w, ch + kStep);
            reduce(u, ch);
            if (more) {
#pragma unroll
                for (int k = 0; k < kUnroll; ++k) u[k] = w[k];
            }
        }
        for (; ch < cend; ch += kThreads) take(__builtin_nontemporal_load(cp + ch), ch);
        lane_softmax_done();
        if (split == 0) {            // unaligned head and tail, a handful of elements
            for (int64_t e = tid; e < lead; e += kThreads) visit<false>(p, Elem<T>::one(rp + e), (int)e, c, T_, 0.f);
            for (int64_t e = tail0 + tid; e < vocab; e += kThreads) visit<false>(p, Elem<T>::one(rp + e), (int)e, c, T_, 0.f);
        }
    } else {
        // With noise.  The softmax runs over 16-byte chunks as without noise; the noisy argmax is element by
        // element: l = x / T by a true division (skipped, not approximated, when T = 1: x / 1 == x), v = l + g, the
        // larger v or at equal v the lower index wins -- the arithmetic of an fp32 host computation, bit for bit.
        // The noise g of an element is read from the tensor (mode 1; 16-byte loads when the row's noise lines up
        // with its chunks) or drawn from the generator (mode 2: a chunk whose first column is a multiple of 4 --
        // every row that starts on a 16-byte boundary -- takes whole generator outputs, EPC / 4 of them; otherwise
        // every element asks for its own), so both modes draw the same tokens from the same noise.
        const RowNoise rn = NOISE == 2 ? row_noise(N, row) : RowNoise{0, 0, 0, 0, 0};
        const bool whole_groups = (lead & 3) == 0;
        const bool noise_lines_up = NOISE == 1 && (reinterpret_cast<uintptr_t>(np + lead) & 15) == 0;
        const bool unit_T = T_ == 1.0f;
        float best = kNegBig, best_x = 0.f;
        float seen = kNegBig;            // mode 2: what this wavefront knows of the workgroup's best noisy logit (same in all lanes)
        int best_idx = kNoIndex, since_look = 0;
        auto offer = [&](float x, int index, float g) {
            const float v = (unit_T ? x : x / T_) + g;
            if (v > best || (v == best && index < best_idx)) { best = v; best_x = x; best_idx = index; }
        };
        auto noise_at = [&](int64_t e) { return NOISE == 1 ? np[e] : rn.at((int)e); };
        for (int64_t ch = cbeg + tid; ch < cend; ch += kThreads) {
            float x[EPC];
            Elem<T>::unpack(__builtin_nontemporal_load(cp + ch), x);
            const float cmx = take_values(x, ch);
            const int c0 = (int)(lead + ch * EPC);
            // No draw of the generator exceeds kGumbelMax, and rounding is monotonic: an element of this chunk can
            // take (or tie) the row's lead only if (largest element) / T + kGumbelMax reaches the best noisy logit
            // that anybody in the workgroup has found so far (lead_seen: published by the wavefronts as they go; an
            // old value only makes the test more cautious).  Where that holds in no lane of the wavefront the
            // chunk's noise is not drawn -- every chunk of -inf that a top-k / top-p filter left behind, and the
            // bulk of a peaked row; what is skipped could not have been picked.  (A noise tensor may hold
            // anything: mode 1 reads all of it.)
            if (NOISE == 2) {
                if ((++since_look & 7) == 0)           // the others' news every eighth chunk: an LDS read per chunk would cost what it saves
                    seen = fmaxf(seen, __hip_atomic_load(&lead_seen, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP));
                const bool may_lead = (unit_T ? cmx : cmx / T_) + kGumbelMax >= fmaxf(best, seen);
                if (__builtin_amdgcn_ballot_w64(may_lead) == 0) continue;
            }
            if (NOISE == 1) {
                float g[EPC];
                if (noise_lines_up) {
#pragma unroll
                    for (int q = 0; q < EPC / 4; ++q) {
                        const u32x4 w = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(np + c0) + q);
                        g[4 * q + 0] = __uint_as_float(w.x); g[4 * q + 1] = __uint_as_float(w.y);
                        g[4 * q + 2] = __uint_as_float(w.z); g[4 * q + 3] = __uint_as_float(w.w);
                    }
                } else {
#pragma unroll
                    for (int i = 0; i < EPC; ++i) g[i] = np[c0 + i];
                }
#pragma unroll
                for (int i = 0; i < EPC; ++i) offer(x[i], c0 + i, g[i]);
            } else if (whole_groups) {
                U4 r[EPC / 4];
#pragma unroll
                for (int q = 0; q < EPC / 4; ++q) r[q] = rn.group((uint32_t)(c0 >> 2) + q);
                // The generator's bits decide before any logarithm is taken.  An element reaches the lead only with
                // noise -ln(-ln u) >= need = lead - (largest element) / T, i.e. -ln u <= e^-need; and -ln u >= 1 - u
                // = (j + 1/2) 2^-23, where j = ~bits >> 9 counts u down from its largest value.  So only draws with
                // j <= e^-need 2^23 matter: at need = 10, one in 22 000.  need is taken 0.02 + 2^-22 |lead| lower than
                // computed, which covers the error of the hardware logarithms (2e-6) and every rounding on the way.
                const float lim = fmaxf(best, seen);
                const float need = lim - (unit_T ? cmx : cmx / T_) - __builtin_fmaf(fabsf(lim), 2.384185791015625e-07f, 0.02f);
                const float reach = fminf(fast_exp2(__builtin_fmaf(-kLog2e, need, 23.f)), 8388608.f);    // NaN (lead and element both infinite) -> the other operand
                uint32_t top = 0;
#pragma unroll
                for (int q = 0; q < EPC / 4; ++q) top = max(max(top, max(r[q].x, r[q].y)), max(r[q].z, r[q].w));
                if (__builtin_amdgcn_ballot_w64((~top >> 9) <= (uint32_t)reach + 1u) == 0) continue;
#pragma unroll
                for (int q = 0; q < EPC / 4; ++q) {
                    offer(x[4 * q + 0], c0 + 4 * q + 0, gumbel_of(r[q].x));
                    offer(x[4 * q + 1], c0 + 4 * q + 1, gumbel_of(r[q].y));
                    offer(x[4 * q + 2], c0 + 4 * q + 2, gumbel_of(r[q].z));
                    offer(x[4 * q + 3], c0 + 4 * q + 3, gumbel_of(r[q].w));
                }
            } else {
#pragma unroll
                for (int i = 0; i < EPC; ++i) offer(x[i], c0 + i, rn.at(c0 + i));
            }
            if (NOISE == 2) {
                // the wavefront's best so far, to everybody (only when it has grown: few chunks of a row raise it).
                // Only with all 64 lanes still in the loop: on the row's last, partly filled trip the lanes that
                // have left are switched off, a shuffle reads 0 from them, and a 0 published above a row whose
                // noisy logits are all negative would let the others skip the real winner.  Not publishing on
                // that one trip costs nothing (an old lead_seen only makes the skip test more cautious).
                if (__builtin_amdgcn_ballot_w64(best > seen) != 0 && __builtin_amdgcn_ballot_w64(true) == ~0ull) {
                    float wb = best;
#pragma unroll
                    for (int off = 32; off >= 1; off >>= 1) wb = fmaxf(wb, __shfl_xor(wb, off));
                    seen = fmaxf(seen, wb);
                    if ((tid & (mdx::kWave - 1)) == 0) __hip_atomic_fetch_max(&lead_seen, wb, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                }
            }
        }
        lane_softmax_done();
        p.pick = best; p.pick_x = best_x; p.pick_idx = best_idx;
        if (split == 0) {
            for (int64_t e = tid; e < lead; e += kThreads) visit<true>(p, Elem<T>::one(rp + e), (int)e, c, T_, noise_at(e));
            for (int64_t e = tail0 + tid; e < vocab; e += kThreads) visit<true>(p, Elem<T>::one(rp + e), (int)e, c, T_, noise_at(e));
        }
    }

    // Wavefront reduction, then across the workgroup's wavefronts through LDS.
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
        const Partial o = shfl_xor(p, off, NOISE != 0);
        combine(p, o, c, NOISE != 0);
    }
    __shared__ Partial wave_part[kThreads / mdx::kWave];
    if ((tid & (mdx::kWave - 1)) == 0) wave_part[tid / mdx::kWave] = p;
    __syncthreads();
    if (tid == 0) {
        Partial r = wave_part[0];
#pragma unroll
        for (int w = 1; w < kThreads / mdx::kWave; ++w) combine(r, wave_part[w], c, NOISE != 0);
        if (nsplit > 1) {
            partials[row * nsplit + split] = r;
        } else {
            int64_t tok; float conf;
            finish_row<(NOISE != 0)>(r, c, tok, conf);
            x0[row] = tok;
            x0_p[row] = conf;
        }
    }
}

// Merges the row splits: one lane per row.
template <bool NOISE>
__global__ __launch_bounds__(kThreads) void confidence_finalize_kernel(
    const Partial* __restrict__ partials, int nsplit,
    const float* __restrict__ temperatures, int rows_per_temp,
    int64_t rows, int64_t* __restrict__ x0, float* __restrict__ x0_p)
{
    const int64_t row = (int64_t)blockIdx.x * kThreads + threadIdx.x;
    if (row >= rows) return;
    const float T_ = temperatures ? temperatures[row / rows_per_temp] : 1.0f;
    const float c = kLog2e / T_;
    Partial r = partials[row * nsplit];
    for (int s = 1; s < nsplit; ++s) combine(r, partials[row * nsplit + s], c, NOISE);
    int64_t tok; float conf;
    finish_row<NOISE>(r, c, tok, conf);
    x0[row] = tok;
    x0_p[row] = conf;
}

// One workgroup per sequence; lane p owns block position p.  With FROM_PARTIALS the row splits
// of the vocabulary pass are merged here (and x0 / x0_p written), saving a launch.
constexpr int kMaxBlockLen = 1024;
template <bool FROM_PARTIALS>
__global__ __launch_bounds__(kMaxBlockLen) void select_transfer_kernel(
    int64_t* __restrict__ x0, float* __restrict__ x0_p, int64_t* __restrict__ tokens,
    const Partial* __restrict__ partials, int nsplit, const float* __restrict__ temperatures,
    int64_t mask_token_id, float threshold, int k,
    uint8_t* __restrict__ transfer, int32_t* __restrict__ count, int block_len)
{
    __shared__ float conf_s[kMaxBlockLen];
    __shared__ int n_hi, n_masked, n_commit;
    const int b = blockIdx.x;
    const int p = threadIdx.x;
    const bool on = p < block_len;
    const int64_t at = (int64_t)b * block_len + p;
    if (p == 0) { n_hi = 0; n_masked = 0; n_commit = 0; }
    __syncthreads();
    int64_t pick = 0;
    float pick_p = 0.f;
    if (on) {
        if (FROM_PARTIALS) {
            const float c = kLog2e / (temperatures ? temperatures[b] : 1.0f);
            Partial r = partials[at * nsplit];
            for (int s = 1; s < nsplit; ++s) combine(r, partials[at * nsplit + s], c, false);
            finish_row<false>(r, c, pick, pick_p);
            x0[at] = pick;
            x0_p[at] = pick_p;
        } else {
            pick = x0[at];
            pick_p = x0_p[at];
        }
    }
    const bool masked = on && tokens[at] == mask_token_id;
    const float conf = masked ? pick_p : -INFINITY;
    const bool hi = conf > threshold;
    if (on) conf_s[p] = conf;
    if (hi) atomicAdd(&n_hi, 1);
    if (masked) atomicAdd(&n_masked, 1);
    __syncthreads();
    bool commit;
    if (n_hi >= k) {
        commit = hi;
    } else {
        // rank among masked positions: higher confidence first, lower position first on ties
        int rank = 0;
        if (masked) {
            for (int j = 0; j < block_len; ++j) {
                const float cj = conf_s[j];
                rank += (cj > conf || (cj == conf && j < p)) ? 1 : 0;
            }
        }
        commit = masked && rank < k && conf > -INFINITY;     // at most min(k, n_masked) positions; a confidence of -inf is never committed
    }
    if (on) {
        transfer[at] = commit ? 1 : 0;
        if (commit) {
            tokens[at] = pick;
            atomicAdd(&n_commit, 1);
        }
    }
    __syncthreads();
    if (p == 0) count[b] = n_commit;
}

// The same rule for blocks of up to 64 positions (the engine's blocks hold 32) with ONE wavefront per
// sequence: lane p owns position p, counts are ballots, and the rank among the masked positions comes
// from reading every lane's confidence in turn -- no LDS, no atomics, no barrier, so the launch costs
// little more than its one round trip to memory.
template <bool FROM_PARTIALS>
__global__ __launch_bounds__(mdx::kWave) void select_transfer_wave_kernel(
    int64_t* __restrict__ x0, float* __restrict__ x0_p, int64_t* __restrict__ tokens,
    const Partial* __restrict__ partials, int nsplit, const float* __restrict__ temperatures,
    int64_t mask_token_id, float threshold, int k,
    uint8_t* __restrict__ transfer, int32_t* __restrict__ count, int block_len)
{
    const int b = blockIdx.x;
    const int p = threadIdx.x;
    const bool on = p < block_len;
    const int64_t at = (int64_t)b * block_len + p;
    int64_t pick = 0;
    float pick_p = 0.f;
    int64_t tok = 0;
    if (on) {
        tok = tokens[at];
        if (FROM_PARTIALS) {
            const float c = kLog2e / (temperatures ? temperatures[b] : 1.0f);
            Partial r = partials[at * nsplit];
            for (int s = 1; s < nsplit; ++s) combine(r, partials[at * nsplit + s], c, false);
            finish_row<false>(r, c, pick, pick_p);
            x0[at] = pick;
            x0_p[at] = pick_p;
        } else {
            pick = x0[at];
            pick_p = x0_p[at];
        }
    }
    const bool masked = on && tok == mask_token_id;
    const float conf = masked ? pick_p : -INFINITY;
    const bool hi = conf > threshold;
    bool commit;
    if (__popcll(__ballot(hi)) >= k) {
        commit = hi;
    } else {
        // rank among masked positions: higher confidence first, lower position first on ties
        int rank = 0;
        for (int j = 0; j < block_len; ++j) {
            const float cj = __shfl(conf, j);
            rank += (cj > conf || (cj == conf && j < p)) ? 1 : 0;
        }
        commit = masked && rank < k && conf > -INFINITY;     // at most min(k, #masked) positions; a confidence of -inf is never committed
    }
    const int n_commit = __popcll(__ballot(commit));
    if (on) {
        transfer[at] = commit ? 1 : 0;
        if (commit) tokens[at] = pick;
    }
    if (p == 0) count[b] = n_commit;
}

int launch_select(int64_t* x0, float* x0_p, int64_t* tokens, const Partial* partials, int nsplit, const float* temperatures,
                  int64_t mask_token_id, float threshold, int k, uint8_t* transfer, int32_t* count, int bs, int block_len,
                  hipStream_t stream)
{
    const bool from_partials = partials != nullptr && nsplit > 1;
    if (block_len <= mdx::kWave) {
        if (from_partials)
            select_transfer_wave_kernel<true><<<(unsigned)bs, mdx::kWave, 0, stream>>>(
                x0, x0_p, tokens, partials, nsplit, temperatures, mask_token_id, threshold, k, transfer, count, block_len);
        else
            select_transfer_wave_kernel<false><<<(unsigned)bs, mdx::kWave, 0, stream>>>(
                x0, x0_p, tokens, nullptr, 1, nullptr, mask_token_id, threshold, k, transfer, count, block_len);
    } else {
        const int threads = ((block_len + mdx::kWave - 1) / mdx::kWave) * mdx::kWave;
        if (from_partials)
            select_transfer_kernel<true><<<(unsigned)bs, threads, 0, stream>>>(
                x0, x0_p, tokens, partials, nsplit, temperatures, mask_token_id, threshold, k, transfer, count, block_len);
        else
            select_transfer_kernel<false><<<(unsigned)bs, threads, 0, stream>>>(
                x0, x0_p, tokens, nullptr, 1, nullptr, mask_token_id, threshold, k, transfer, count, block_len);
    }
    return mdx::check_launch("select_transfer");
}

// Splits per row so that small batches still fill the chip: target >= 4 workgroups per CU
// while keeping at least 32 KiB of logits per workgroup.
int pick_nsplit(int64_t rows, int64_t vocab) {
    const int64_t target = 1024;
    int64_t n = (target + rows - 1) / rows;
    const int64_t max_by_size = vocab / 16384 > 0 ? vocab / 16384 : 1;
    if (n > max_by_size) n = max_by_size;
    if (n < 1) n = 1;
    if (n > 64) n = 64;
    return (int)n;
}

template <typename T>
int launch_confidence(const void* logits, int64_t row_stride, const float* temperatures, int rows_per_temp,
                      const NoiseSpec& N, int64_t* x0, float* x0_p,
                      int64_t rows, int64_t vocab, int nsplit, Partial* partials, bool finalize, hipStream_t stream)
{
    const dim3 grid((unsigned)rows, (unsigned)nsplit);
    const bool noisy = N.noise != nullptr || N.philox;
    if (N.philox)
        confidence_argmax_kernel<T, 2><<<grid, kThreads, 0, stream>>>(
            (const T*)logits, row_stride, temperatures, rows_per_temp, N, vocab, nsplit, partials, x0, x0_p);
    else if (N.noise)
        confidence_argmax_kernel<T, 1><<<grid, kThreads, 0, stream>>>(
            (const T*)logits, row_stride, temperatures, rows_per_temp, N, vocab, nsplit, partials, x0, x0_p);
    else
        confidence_argmax_kernel<T, 0><<<grid, kThreads, 0, stream>>>(
            (const T*)logits, row_stride, temperatures, rows_per_temp, N, vocab, nsplit, partials, x0, x0_p);
    int rc = mdx::check_launch("confidence_argmax");
    if (rc != MDX_OK || nsplit == 1 || !finalize) return rc;
    const unsigned fgrid = (unsigned)((rows + kThreads - 1) / kThreads);
    if (noisy)
        confidence_finalize_kernel<true><<<fgrid, kThreads, 0, stream>>>(partials, nsplit, temperatures, rows_per_temp, rows, x0, x0_p);
    else
        confidence_finalize_kernel<false><<<fgrid, kThreads, 0, stream>>>(partials, nsplit, temperatures, rows_per_temp, rows, x0, x0_p);
    return mdx::check_launch("confidence_finalize");
}

// The noise tensor that the generator stands for, written out: [rows, vocab] fp32.
__global__ __launch_bounds__(kThreads) void gumbel_noise_kernel(float* __restrict__ out, int64_t out_row_stride, int64_t vocab, const NoiseSpec N)
{
    const int64_t row = blockIdx.y;
    const RowNoise rn = row_noise(N, row);
    const int64_t group = (int64_t)blockIdx.x * kThreads + threadIdx.x;
    if (group * 4 >= vocab) return;
    const U4 r = rn.group((uint32_t)group);
    const uint32_t b[4] = {r.x, r.y, r.z, r.w};
    float* dst = out + row * out_row_stride + group * 4;
#pragma unroll
    for (int i = 0; i < 4; ++i)
        if (group * 4 + i < vocab) dst[i] = gumbel_of(b[i]);
}

NoiseSpec no_noise() { return NoiseSpec{nullptr, 0, false, 0, 0, 0, nullptr, nullptr}; }
NoiseSpec tensor_noise(const float* noise, int64_t stride) { NoiseSpec n = no_noise(); n.noise = noise; n.noise_row_stride = stride; return n; }
NoiseSpec generator_noise(uint64_t seed, uint64_t offset, const int64_t* offset_dev, const int64_t* row_ids) {
    NoiseSpec n = no_noise();
    n.philox = true; n.key0 = (uint32_t)seed; n.key1 = (uint32_t)(seed >> 32);
    n.offset = offset; n.offset_dev = offset_dev; n.row_ids = row_ids;
    return n;
}

}  // namespace

extern "C" int64_t mdx_confidence_argmax_workspace_bytes(int64_t rows, int64_t vocab) {
    if (rows <= 0 || vocab <= 0) return 0;
    const int nsplit = pick_nsplit(rows, vocab);
    return nsplit > 1 ? rows * nsplit * (int64_t)sizeof(Partial) : 0;
}

namespace {

int confidence_pass(const void* logits, int64_t row_stride, int32_t dtype,
                    const float* temperatures, int32_t rows_per_temp,
                    const NoiseSpec& N,
                    int64_t* x0, float* x0_p, int64_t rows, int64_t vocab,
                    void* workspace, int64_t workspace_bytes, bool finalize, int* nsplit_out, hipStream_t stream)
{
    MDX_REQUIRE(rows >= 0 && vocab >= 0, MDX_EINVAL, "confidence_argmax: negative size");
    if (nsplit_out) *nsplit_out = 1;
    if (rows == 0) return MDX_OK;
    MDX_REQUIRE(vocab > 0, MDX_EINVAL, "confidence_argmax: empty vocabulary");
    MDX_REQUIRE(logits && x0 && x0_p, MDX_EINVAL, "confidence_argmax: null pointer");
    MDX_REQUIRE(vocab < (int64_t)0x7fffffff && rows < (int64_t)0x7fffffff, MDX_EUNSUPPORTED,
                "confidence_argmax: rows %lld or vocab %lld out of range", (long long)rows, (long long)vocab);
    MDX_REQUIRE(row_stride >= vocab, MDX_EUNSUPPORTED, "confidence_argmax: row_stride %lld < vocab %lld", (long long)row_stride, (long long)vocab);
    MDX_REQUIRE(!temperatures || rows_per_temp > 0, MDX_EINVAL, "confidence_argmax: rows_per_temp must be positive");
    MDX_REQUIRE(!N.noise || N.noise_row_stride >= vocab, MDX_EINVAL, "confidence_argmax: noise_row_stride < vocab");
    const int esz = dtype == MDX_F32 ? 4 : 2;
    MDX_REQUIRE((reinterpret_cast<uintptr_t>(logits) % esz) == 0, MDX_EUNSUPPORTED, "confidence_argmax: logits not element-aligned");
    const int nsplit = pick_nsplit(rows, vocab);
    if (nsplit_out) *nsplit_out = nsplit;
    const int64_t need = nsplit > 1 ? rows * nsplit * (int64_t)sizeof(Partial) : 0;
    MDX_REQUIRE(need == 0 || (workspace && workspace_bytes >= need), MDX_EWORKSPACE,
                "confidence_argmax: workspace of %lld bytes needed, %lld given", (long long)need, (long long)workspace_bytes);
    Partial* partials = static_cast<Partial*>(workspace);
    switch (dtype) {
        case MDX_BF16: return launch_confidence<__bf16>(logits, row_stride, temperatures, rows_per_temp, N, x0, x0_p, rows, vocab, nsplit, partials, finalize, stream);
        case MDX_F16:  return launch_confidence<__half>(logits, row_stride, temperatures, rows_per_temp, N, x0, x0_p, rows, vocab, nsplit, partials, finalize, stream);
        case MDX_F32:  return launch_confidence<float>(logits, row_stride, temperatures, rows_per_temp, N, x0, x0_p, rows, vocab, nsplit, partials, finalize, stream);
        default: return mdx::fail(MDX_EUNSUPPORTED, "confidence_argmax: dtype %d", dtype);
    }
}

}  // namespace

extern "C" int mdx_confidence_argmax(const void* logits, int64_t row_stride, int32_t dtype,
                                     const float* temperatures, int32_t rows_per_temp,
                                     const float* noise, int64_t noise_row_stride,
                                     int64_t* x0, float* x0_p, int64_t rows, int64_t vocab,
                                     void* workspace, int64_t workspace_bytes, mdx_stream_t stream)
{
    return confidence_pass(logits, row_stride, dtype, temperatures, rows_per_temp, tensor_noise(noise, noise_row_stride), x0, x0_p,
                           rows, vocab, workspace, workspace_bytes, true, nullptr, static_cast<hipStream_t>(stream));
}

extern "C" int mdx_confidence_argmax_gumbel(const void* logits, int64_t row_stride, int32_t dtype,
                                            const float* temperatures, int32_t rows_per_temp,
                                            uint64_t seed, uint64_t offset, const int64_t* offset_dev, const int64_t* row_ids,
                                            int64_t* x0, float* x0_p, int64_t rows, int64_t vocab,
                                            void* workspace, int64_t workspace_bytes, mdx_stream_t stream)
{
    return confidence_pass(logits, row_stride, dtype, temperatures, rows_per_temp, generator_noise(seed, offset, offset_dev, row_ids),
                           x0, x0_p, rows, vocab, workspace, workspace_bytes, true, nullptr, static_cast<hipStream_t>(stream));
}

extern "C" int mdx_gumbel_noise(float* noise, int64_t noise_row_stride, int64_t rows, int64_t vocab,
                                uint64_t seed, uint64_t offset, const int64_t* offset_dev, const int64_t* row_ids,
                                mdx_stream_t stream)
{
    MDX_REQUIRE(rows >= 0 && vocab >= 0, MDX_EINVAL, "gumbel_noise: negative size");
    if (rows == 0 || vocab == 0) return MDX_OK;
    MDX_REQUIRE(noise, MDX_EINVAL, "gumbel_noise: null pointer");
    MDX_REQUIRE(noise_row_stride >= vocab, MDX_EINVAL, "gumbel_noise: noise_row_stride < vocab");
    MDX_REQUIRE(vocab < (int64_t)0x7fffffff && rows <= 65535, MDX_EUNSUPPORTED,
                "gumbel_noise: rows %lld (max 65535) or vocab %lld out of range", (long long)rows, (long long)vocab);
    const dim3 grid((unsigned)(((vocab + 3) / 4 + kThreads - 1) / kThreads), (unsigned)rows);
    gumbel_noise_kernel<<<grid, kThreads, 0, static_cast<hipStream_t>(stream)>>>(noise, noise_row_stride, vocab,
                                                                                 generator_noise(seed, offset, offset_dev, row_ids));
    return mdx::check_launch("gumbel_noise");
}

extern "C" int mdx_select_transfer(const int64_t* x0, const float* x0_p, int64_t* tokens,
                                   int64_t mask_token_id, float threshold, int32_t k,
                                   uint8_t* transfer, int32_t* count,
                                   int32_t bs, int32_t block_len, mdx_stream_t stream_)
{
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    MDX_REQUIRE(bs >= 0 && block_len >= 0, MDX_EINVAL, "select_transfer: negative size");
    if (bs == 0 || block_len == 0) return MDX_OK;
    MDX_REQUIRE(x0 && x0_p && tokens && transfer && count, MDX_EINVAL, "select_transfer: null pointer");
    MDX_REQUIRE(block_len <= kMaxBlockLen, MDX_EUNSUPPORTED, "select_transfer: block_len %d > %d", block_len, kMaxBlockLen);
    MDX_REQUIRE(k >= 0, MDX_EINVAL, "select_transfer: k %d < 0", k);
    return launch_select(const_cast<int64_t*>(x0), const_cast<float*>(x0_p), tokens, nullptr, 1, nullptr, mask_token_id, threshold, k,
                         transfer, count, bs, block_len, stream);
}

namespace {

int unmask_step_impl(const void* logits, int64_t row_stride, int32_t dtype,
                     const float* temperatures, const NoiseSpec& N,
                     int64_t* tokens, int64_t mask_token_id, float threshold, int32_t k,
                     int64_t* x0, float* x0_p, uint8_t* transfer, int32_t* count,
                     int32_t bs, int32_t block_len, int64_t vocab,
                     void* workspace, int64_t workspace_bytes, hipStream_t stream)
{
    MDX_REQUIRE(bs >= 0 && block_len >= 0, MDX_EINVAL, "unmask_step: negative size");
    MDX_REQUIRE(k >= 0, MDX_EINVAL, "unmask_step: k %d < 0", k);
    MDX_REQUIRE(block_len <= kMaxBlockLen, MDX_EUNSUPPORTED, "unmask_step: block_len %d > %d", block_len, kMaxBlockLen);
    if (bs == 0 || block_len == 0) return MDX_OK;
    MDX_REQUIRE(tokens && transfer && count, MDX_EINVAL, "unmask_step: null pointer");
    // Without noise the selection kernel merges the row splits itself (one launch fewer).
    const bool noisy = N.noise != nullptr || N.philox;
    int nsplit = 1;
    int rc = confidence_pass(logits, row_stride, dtype, temperatures, block_len, N,
                             x0, x0_p, (int64_t)bs * block_len, vocab, workspace, workspace_bytes, noisy, &nsplit, stream);
    if (rc != MDX_OK) return rc;
    return launch_select(x0, x0_p, tokens, (nsplit > 1 && !noisy) ? static_cast<const Partial*>(workspace) : nullptr, nsplit, temperatures,
                         mask_token_id, threshold, k, transfer, count, bs, block_len, stream);
}

}  // namespace

extern "C" int mdx_unmask_step(const void* logits, int64_t row_stride, int32_t dtype,
                               const float* temperatures, const float* noise, int64_t noise_row_stride,
                               int64_t* tokens, int64_t mask_token_id, float threshold, int32_t k,
                               int64_t* x0, float* x0_p, uint8_t* transfer, int32_t* count,
                               int32_t bs, int32_t block_len, int64_t vocab,
                               void* workspace, int64_t workspace_bytes, mdx_stream_t stream)
{
    return unmask_step_impl(logits, row_stride, dtype, temperatures, tensor_noise(noise, noise_row_stride), tokens, mask_token_id,
                            threshold, k, x0, x0_p, transfer, count, bs, block_len, vocab, workspace, workspace_bytes,
                            static_cast<hipStream_t>(stream));
}

extern "C" int mdx_unmask_step_gumbel(const void* logits, int64_t row_stride, int32_t dtype,
                                      const float* temperatures,
                                      uint64_t seed, uint64_t offset, const int64_t* offset_dev, const int64_t* row_ids,
                                      int64_t* tokens, int64_t mask_token_id, float threshold, int32_t k,
                                      int64_t* x0, float* x0_p, uint8_t* transfer, int32_t* count,
                                      int32_t bs, int32_t block_len, int64_t vocab,
                                      void* workspace, int64_t workspace_bytes, mdx_stream_t stream)
{
    return unmask_step_impl(logits, row_stride, dtype, temperatures, generator_noise(seed, offset, offset_dev, row_ids), tokens,
                            mask_token_id, threshold, k, x0, x0_p, transfer, count, bs, block_len, vocab, workspace, workspace_bytes,
                            static_cast<hipStream_t>(stream));
}
