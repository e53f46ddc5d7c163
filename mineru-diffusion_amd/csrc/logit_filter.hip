// Top-k / top-p filtering of a row of logits before sampling: the HF variant's top_k_logits and
// top_p_logits (mineru_diffusion/modeling_mineru_diffusion.py:585-600, applied in that order by
// sample_with_temperature_topk_topp, :608-611).  The reference sorts every row; here a row is never
// sorted.  Both filters keep exactly the elements at or above one VALUE of the row:
//
//   top-k   the k-th largest value (elements equal to it are all kept, as `logits < min_values` keeps them)
//   top-p   the value of the element at which the cumulative probability, taken from the largest
//           element down, first exceeds p (softmax over what top-k kept, at temperature T)
//
// and a 16-bit logit has only 65 536 possible values, so that value is found by counting: one pass
// histograms the high byte of an order-preserving key (element count and probability mass per bin),
// the bin where the running count / mass crosses the target is found, and a second pass histograms the
// low byte inside that bin.  Two passes per filter (top-p needs the row maximum that its softmax terms are
// relative to: the first top-k pass finds it on the way, a top-p without top-k takes a pass for it) and one
// pass that writes the filtered copy; one workgroup per row.  Every pass reads the row from memory again (the
// rows in flight exceed the L2), and with two workgroups per CU that traffic and the LDS atomics of the
// counting cost about the same: holding the row in registers (one workgroup per CU) measured slower.
//
// Where the reference's sort leaves the order of equal values open, all elements equal to the crossing
// value are kept.  The probability masses are fp32 terms summed in fixed point, so the result does not
// depend on the order of the additions; against a computation in higher precision, a target that falls
// within fp32 rounding of a cumulative probability can resolve either way.
#include "mdx_common.h"
#include <hip/hip_fp16.h>

namespace {

constexpr int kFilterThreads = 1024;
constexpr float kLog2e = 1.4426950408889634f;

template <typename T> struct Bits16;
template <> struct Bits16<__bf16> {
    static constexpr uint32_t kNegInf = 0xff80u;
    static __device__ __forceinline__ float value(uint32_t b) { return __uint_as_float(b << 16); }
};
template <> struct Bits16<__half> {
    static constexpr uint32_t kNegInf = 0xfc00u;
    static __device__ __forceinline__ float value(uint32_t b) { return __half2float(__ushort_as_half((unsigned short)b)); }
};

// Bit pattern -> key that grows with the value (-0 counts as +0); and back.
__device__ __forceinline__ uint32_t key_of(uint32_t b) {
    if (b == 0x8000u) b = 0;
    return (b & 0x8000u) ? (~b & 0xffffu) : (b | 0x8000u);
}
__device__ __forceinline__ uint32_t bits_of(uint32_t k) { return (k & 0x8000u) ? (k & 0x7fffu) : (~k & 0xffffu); }

struct RowView {                        // a row as scalar head, aligned 16-byte chunks, scalar tail
    const uint16_t* p;
    const u32x4* chunks;
    int lead, nchunk, tail0, vocab;
};

template <typename F>
__device__ __forceinline__ void scan_row(const RowView& r, int tid, F f) {
    for (int e = tid; e < r.lead; e += kFilterThreads) f((uint32_t)r.p[e]);
    for (int ch = tid; ch < r.nchunk; ch += kFilterThreads) {
        const u32x4 u = r.chunks[ch];
        const uint32_t w[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) { f(w[i] & 0xffffu); f(w[i] >> 16); }
    }
    for (int e = r.tail0 + tid; e < r.vocab; e += kFilterThreads) f((uint32_t)r.p[e]);
}

// Neighbouring logits mostly share a bin (a bin spans two octaves of bf16 values), and LDS atomics of
// one wavefront to one address are served one lane at a time: every bin therefore has kSlots counters,
// lane l adds to counter l % kSlots, and the counters are summed once per pass.
constexpr int kSlots = 16;
// Softmax terms (at most 1 each, relative to the row maximum) are summed as 64-bit integers in units
// of 2^-40: integer LDS atomics are several times faster than floating-point ones, the sum does not
// depend on the order of the additions, and what truncation drops over a row of 2^18 elements is
// below 2^-22 of the largest term.
constexpr float kMassScale = 1099511627776.f;        // 2^40

struct Shared {
    int cnt_slots[256 * kSlots];
    unsigned long long mass_slots[256 * kSlots];     // fixed point, kMassScale per unit
    int cnt[256];
    float mass[256];
    uint32_t max_key;        // key of the row's largest element
    int bin;                 // the bin that holds the crossing
    int cnt_before;          // elements in the bins above it
    float mass_before;       // their mass: sum of exp2((x - row max) * c)
    float target;            // mass to exceed
    uint32_t key;            // result of a selection
};

// Among the elements with key >= floor_key: MASS ? the key at which the cumulative mass from the top
// first exceeds top_p of the total : the key of the k-th largest.  Returns floor_key when the
// target is never reached (k at or beyond the number of such elements).  Masses are softmax terms
// relative to the row maximum m, exp2((x - m) * c) <= 1.
// TRACK_MAX: the first pass also leaves the key of the row's largest element in sh.max_key (which the caller has
// cleared), so that a top-p selection that follows needs no pass of its own for it.
template <typename T, bool MASS, bool TRACK_MAX = false>
__device__ uint32_t select_key(const RowView& row, Shared& sh, uint32_t floor_key, int k, float top_p, float c, float m) {
    const int tid = threadIdx.x, slot = tid % kSlots;
    uint32_t mk = 0;
    auto clear_slots = [&]() {
        for (int i = tid; i < 256 * kSlots; i += kFilterThreads) { sh.cnt_slots[i] = 0; if (MASS) sh.mass_slots[i] = 0ull; }
        __syncthreads();
    };
    auto sum_slots = [&]() {
        __syncthreads();
        if (tid < 256) {
            int n = 0;
            unsigned long long a = 0ull;
            for (int j = 0; j < kSlots; ++j) {
                const int at = tid * kSlots + (j + tid) % kSlots;       // staggered: lane t starts at bank t
                n += sh.cnt_slots[at];
                if (MASS) a += sh.mass_slots[at];
            }
            sh.cnt[tid] = n;
            sh.mass[tid] = (float)a * (1.0f / kMassScale);
        }
        __syncthreads();
    };
    clear_slots();
    scan_row(row, tid, [&](uint32_t b) {
        const uint32_t key = key_of(b);
        if (TRACK_MAX) mk = key > mk ? key : mk;
        if (key < floor_key) return;
        const int at = (int)(key >> 8) * kSlots + slot;
        atomicAdd(&sh.cnt_slots[at], 1);
        if (MASS) atomicAdd(&sh.mass_slots[at], (unsigned long long)(__builtin_amdgcn_exp2f((Bits16<T>::value(b) - m) * c) * kMassScale));
    });
    if (TRACK_MAX) {
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) { const uint32_t o = __shfl_xor(mk, off); mk = o > mk ? o : mk; }
        if ((tid & 63) == 0) atomicMax(&sh.max_key, mk);
    }
    sum_slots();
    if (tid == 0) {
        float target = 0.f;
        if (MASS) {
            float Z = 0.f;
            for (int b = 255; b >= 0; --b) Z += sh.mass[b];
            target = top_p * Z;
        }
        int found = -1, lowest = -1, cnt = 0;
        float mass = 0.f;
        for (int b = 255; b >= 0; --b) {
            if (!sh.cnt[b]) continue;
            lowest = b;
            const bool crosses = MASS ? (mass + sh.mass[b] > target) : (cnt + sh.cnt[b] >= k);
            if (crosses) { found = b; break; }
            cnt += sh.cnt[b];
            mass += sh.mass[b];
        }
        if (MASS && found < 0 && lowest >= 0) {   // the running sum rounded onto the target: the lowest bin in use,
            found = lowest;                       // whose share comes out of the running sums again
            cnt -= sh.cnt[found];
            mass -= sh.mass[found];
        }
        sh.bin = found; sh.cnt_before = cnt; sh.mass_before = mass; sh.target = target;
    }
    __syncthreads();
    const int bin = sh.bin;
    if (bin < 0) return floor_key;
    clear_slots();
    scan_row(row, tid, [&](uint32_t b) {
        const uint32_t key = key_of(b);
        if (key >= floor_key && (int)(key >> 8) == bin) atomicAdd(&sh.cnt_slots[(int)(key & 0xffu) * kSlots + slot], 1);
    });
    sum_slots();
    if (tid == 0) {
        int cnt = sh.cnt_before, lowest = 0, found = -1;
        float mass = sh.mass_before;
        for (int lo = 255; lo >= 0; --lo) {
            if (!sh.cnt[lo]) continue;
            lowest = lo;
            cnt += sh.cnt[lo];
            if (MASS) {
                const float v = Bits16<T>::value(bits_of(((uint32_t)bin << 8) | (uint32_t)lo));
                mass += (float)sh.cnt[lo] * __builtin_amdgcn_exp2f((v - m) * c);
            }
            if (MASS ? (mass > sh.target) : (cnt >= k)) { found = lo; break; }
        }
        if (found < 0) found = lowest;     // the per-value sums round otherwise than the bin's running sum did
        sh.key = ((uint32_t)bin << 8) | (uint32_t)found;
    }
    __syncthreads();
    const uint32_t key = sh.key;
    __syncthreads();
    return key > floor_key ? key : floor_key;
}

template <typename T>
__global__ __launch_bounds__(kFilterThreads) void logit_filter_kernel(
    const uint16_t* logits, int64_t row_stride,          // may be `out` itself
    const float* __restrict__ temperatures, int rows_per_temp,
    int top_k, float top_p, uint16_t* out, int64_t out_row_stride, int vocab)
{
    __shared__ Shared sh;
    const int64_t r = blockIdx.x;
    const int tid = threadIdx.x;
    RowView row;
    row.p = logits + r * row_stride;
    row.vocab = vocab;
    const uintptr_t addr = reinterpret_cast<uintptr_t>(row.p);
    row.lead = (int)(((16 - (addr & 15)) & 15) / 2);
    if (row.lead > vocab) row.lead = vocab;
    row.nchunk = (vocab - row.lead) / 8;
    row.tail0 = row.lead + row.nchunk * 8;
    row.chunks = reinterpret_cast<const u32x4*>(row.p + row.lead);
    const float T_ = temperatures ? temperatures[r / rows_per_temp] : 1.0f;
    const float c = kLog2e / T_;

    uint32_t floor_key = 0;
    if (tid == 0) sh.max_key = 0;
    __syncthreads();
    const bool with_k = top_k > 0 && top_k < vocab;
    if (with_k) floor_key = select_key<T, false, true>(row, sh, floor_key, top_k, 1.f, c, 0.f);   // also finds the row maximum
    if (top_p < 1.0f) {
        if (!with_k) {
            uint32_t mk = 0;
            scan_row(row, tid, [&](uint32_t b) { const uint32_t key = key_of(b); mk = key > mk ? key : mk; });
#pragma unroll
            for (int off = 32; off >= 1; off >>= 1) { const uint32_t o = __shfl_xor(mk, off); mk = o > mk ? o : mk; }
            if ((tid & 63) == 0) atomicMax(&sh.max_key, mk);
            __syncthreads();
        }
        // a row whose largest element is not finite has no softmax to take a share of: left as it is
        const float m = Bits16<T>::value(bits_of(sh.max_key));
        if (m > -INFINITY && m < INFINITY)
            floor_key = select_key<T, true>(row, sh, floor_key, 0, top_p, c, m);
    }

    uint16_t* op = out + r * out_row_stride;
    auto keep = [&](uint32_t b) { return key_of(b) >= floor_key ? b : Bits16<T>::kNegInf; };
    if (((reinterpret_cast<uintptr_t>(op) ^ addr) & 15) == 0) {
        u32x4* oc = reinterpret_cast<u32x4*>(op + row.lead);
        for (int e = tid; e < row.lead; e += kFilterThreads) op[e] = (uint16_t)keep(row.p[e]);
        for (int ch = tid; ch < row.nchunk; ch += kFilterThreads) {
            const u32x4 u = row.chunks[ch];
            uint32_t w[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
            for (int i = 0; i < 4; ++i) w[i] = keep(w[i] & 0xffffu) | (keep(w[i] >> 16) << 16);
            u32x4 o; o.x = w[0]; o.y = w[1]; o.z = w[2]; o.w = w[3];
            oc[ch] = o;
        }
        for (int e = row.tail0 + tid; e < vocab; e += kFilterThreads) op[e] = (uint16_t)keep(row.p[e]);
    } else {
        for (int e = tid; e < vocab; e += kFilterThreads) op[e] = (uint16_t)keep(row.p[e]);
    }
}

}  // namespace

extern "C" int mdx_filter_logits(const void* logits, int64_t row_stride, int32_t dtype,
                                 const float* temperatures, int32_t rows_per_temp,
                                 int32_t top_k, float top_p,
                                 void* out, int64_t out_row_stride,
                                 int64_t rows, int64_t vocab, mdx_stream_t stream_)
{
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    MDX_REQUIRE(rows >= 0 && vocab >= 0, MDX_EINVAL, "filter_logits: negative size");
    MDX_REQUIRE(top_k >= 0, MDX_EINVAL, "filter_logits: top_k %d < 0", top_k);
    MDX_REQUIRE(top_p >= 0.f, MDX_EINVAL, "filter_logits: top_p %g < 0 (or not a number)", (double)top_p);
    if (rows == 0) return MDX_OK;
    MDX_REQUIRE(vocab > 0, MDX_EINVAL, "filter_logits: empty vocabulary");
    MDX_REQUIRE(logits && out, MDX_EINVAL, "filter_logits: null pointer");
    MDX_REQUIRE(dtype == MDX_BF16 || dtype == MDX_F16, MDX_EUNSUPPORTED, "filter_logits: dtype %d (16-bit logits only)", dtype);
    // a bin's mass is a 64-bit sum of terms of up to 2^40 each: exact for rows of up to 2^23 elements
    MDX_REQUIRE(vocab <= (int64_t)1 << 23 && rows < (int64_t)0x7fffffff, MDX_EUNSUPPORTED,
                "filter_logits: rows %lld or vocab %lld out of range (vocab at most 8388608)", (long long)rows, (long long)vocab);
    MDX_REQUIRE(row_stride >= vocab && out_row_stride >= vocab, MDX_EUNSUPPORTED, "filter_logits: row stride smaller than the vocabulary");
    MDX_REQUIRE(!temperatures || rows_per_temp > 0, MDX_EINVAL, "filter_logits: rows_per_temp must be positive");
    MDX_REQUIRE((reinterpret_cast<uintptr_t>(logits) % 2) == 0 && (reinterpret_cast<uintptr_t>(out) % 2) == 0,
                MDX_EUNSUPPORTED, "filter_logits: logits not element-aligned");
    if (dtype == MDX_BF16)
        logit_filter_kernel<__bf16><<<(unsigned)rows, kFilterThreads, 0, stream>>>(
            static_cast<const uint16_t*>(logits), row_stride, temperatures, rows_per_temp, top_k, top_p,
            static_cast<uint16_t*>(out), out_row_stride, (int)vocab);
    else
        logit_filter_kernel<__half><<<(unsigned)rows, kFilterThreads, 0, stream>>>(
            static_cast<const uint16_t*>(logits), row_stride, temperatures, rows_per_temp, top_k, top_p,
            static_cast<uint16_t*>(out), out_row_stride, (int)vocab);
    return mdx::check_launch("filter_logits");
}
