// Vocabulary projection fused with the confidence reduction of the unmask step: the logits
// x . W^T are produced on the matrix pipe, rounded to bf16 like the projection's output in the reference,
// and reduced to (max, sum of exp, first argmax) while still in registers, so the [rows, vocab] logits
// (311 MB at 1024 rows x 151 936) never travel to HBM and back.
//
// Replaces, for the rows of still-masked positions, ParallelLMHead.forward's F.linear
// (engines/nano_dvlm/nanovllm/layers/embed_head.py:61-67) followed by Sampler.prepare's softmax
// confidence and argmax without noise (layers/sampler.py:11-22).
//
// A workgroup computes a 256-vocab x 256-row tile over the whole hidden dimension (the hand-scheduled core
// of lm_head_core.inc) and leaves two 16-byte records per x row, one per 128-vocab slice; a second, small
// kernel folds a row's records (vocab / 128 of them) into x0 / x0_p.  Launch order: the row tiles of one
// vocab tile sit 8 workgroups apart, so that the dispatcher, which deals consecutive workgroups round-robin
// to the 8 XCDs, puts them on the same XCD next to each other in time and its L2 fetches that tile of W from
// HBM once.
#include "mdx_common.h"
#include <atomic>

namespace {

#include "lm_head_core.inc"

constexpr int kThreads = 256;
constexpr int kTile = 256;                     // vocab rows and x rows per workgroup
constexpr int kSlice = 128;                    // vocab rows per record (one wavefront's share)
constexpr int kLdsBytes = 2 * 2 * kTile * 128; // two stages of (W tile + x tile), 128-byte rows
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kClamp = -1.0e30f;

struct Record { float m, s; int idx, pad; };   // max logit, sum of exp2((x - m) c), first index of the max

struct LmHeadParams {
    const __bf16* x; const __bf16* w;
    int64_t x_stride, w_stride;                // elements between rows
    const float* temperatures; int rows_per_temp; const int64_t* row_ids;
    int rows, vocab, hidden;
    int n_row_tiles, n_vocab_tiles, n_slices;
    Record* records;                           // [rows, n_slices]
    int64_t* x0; float* x0_p;
};

// 32-bit LDS byte address of a pointer into shared memory (what ds_* instructions and M0 take).
typedef __attribute__((address_space(3))) char lds_char;
__device__ __forceinline__ unsigned lds_address(const void* p) { return (unsigned)(uintptr_t)(const lds_char*)p; }

__device__ __forceinline__ int uniform(int x) { return __builtin_amdgcn_readfirstlane(x); }
__device__ __forceinline__ const void* uniform(const void* p) {
    const uint64_t v = (uint64_t)p;
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    return (const void*)(((uint64_t)hi << 32) | lo);
}

__device__ __forceinline__ float row_scale(const LmHeadParams& P, int row) {
    if (!P.temperatures || row >= P.rows) return kLog2e;
    const int64_t id = P.row_ids ? P.row_ids[row] : row;
    return kLog2e / P.temperatures[id / P.rows_per_temp];
}

__global__ __launch_bounds__(kThreads, 1) void lm_head_confidence_kernel(const LmHeadParams P)
{
    extern __shared__ __attribute__((aligned(1024))) char lds[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int H = lane >> 5, r = lane & 31;
    const int wv = wave >> 1, wx = wave & 1;              // this wavefront's half of the vocab rows / of the x rows

    // workgroup -> (vocab tile, row tile): groups of 8 vocab tiles, the row tiles of one vocab tile 8 apart
    const int per_group = 8 * P.n_row_tiles;
    const int group = blockIdx.x / per_group, rem = blockIdx.x % per_group;
    const int vtile = group * 8 + (rem & 7), rtile = rem >> 3;
    if (vtile >= P.n_vocab_tiles) return;
    const int v0 = vtile * kTile, xr0 = rtile * kTile;

    const unsigned lds0 = lds_address(lds);
    LmHeadCoreArgs A;
    {
        const int f = (r >> 1) & 7;
        const unsigned pos0 = (unsigned)((f & 6) | ((H ^ f) & 1));
        A.aw = lds0 + (unsigned)((kSlice * wv + r) * 128) + (pos0 << 4);
        A.ax = lds0 + (unsigned)(kTile * 128) + (unsigned)((kSlice * wx + r) * 128) + (pos0 << 4);
    }
    A.row0 = (unsigned)(8 * wave + (lane >> 3));
    A.trow = (unsigned)tid;
    A.ch = (unsigned)((((lane & 7) ^ (((wave & 1) << 2) | (lane >> 4))) & 7) << 4);
    A.wlast = (unsigned)uniform(min(kTile - 1, P.vocab - 1 - v0));
    A.xlast = (unsigned)uniform(min(kTile - 1, P.rows - 1 - xr0));
    A.wsb = (unsigned)uniform((int)(P.w_stride * 2));
    A.xsb = (unsigned)uniform((int)(P.x_stride * 2));
    A.wb = uniform((const void*)(P.w + (int64_t)v0 * P.w_stride));
    A.xb = uniform((const void*)(P.x + (int64_t)xr0 * P.x_stride));
    A.ldsw = (unsigned)uniform((int)(lds0 + (unsigned)(wave * 1024)));
    A.nkb = (unsigned)uniform(P.hidden / 64);
    const int xrow = xr0 + kSlice * wx + r;               // this lane's x row in x tile 0
    A.c0 = row_scale(P, xrow);
    A.c1 = row_scale(P, xrow + 32);
    A.c2 = row_scale(P, xrow + 64);
    A.c3 = row_scale(P, xrow + 96);
    A.vlane = (unsigned)(v0 + kSlice * wv + 4 * H);
    A.vocab = (unsigned)uniform(P.vocab);
    A.edge = (unsigned)uniform(v0 + kTile > P.vocab ? 1 : 0);
    A.xrow = H == 0 ? (unsigned)xrow : 0x7fffffffu;
    A.rows = (unsigned)uniform(P.rows);
    A.pb = uniform((const void*)P.records);
    A.po = (unsigned)(((int64_t)xrow * P.n_slices + (2 * vtile + wv)) * (int64_t)sizeof(Record));
    A.postep = (unsigned)uniform((int)(32 * P.n_slices * (int)sizeof(Record)));
    lm_head_core(A);
}

// One wavefront per x row: folds the row's records (ascending vocabulary slices) into token and confidence.
__global__ __launch_bounds__(kThreads) void lm_head_finalize_kernel(const LmHeadParams P)
{
    const int row = blockIdx.x * (kThreads / 64) + (threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    if (row >= P.rows) return;
    const float c = row_scale(P, row);
    float m = -INFINITY, s = 0.f;
    int idx = 0x7fffffff;
    auto fold = [&](float m2, float s2, int i2) {
        if (!(m2 > -INFINITY)) return;                    // an empty slice (all of it beyond the vocabulary, or -inf logits)
        const float M = fmaxf(m, m2);
        const float a = fmaxf(m, kClamp) - fmaxf(M, kClamp), b = fmaxf(m2, kClamp) - fmaxf(M, kClamp);
        s = s * __builtin_amdgcn_exp2f(a * c) + s2 * __builtin_amdgcn_exp2f(b * c);
        idx = (m2 > m) ? i2 : ((m2 == m) ? min(idx, i2) : idx);
        m = M;
    };
    // the row's records, eight per lane in flight at a time (a fold per load would make this a chain of memory latencies)
    const u32x4* rec = reinterpret_cast<const u32x4*>(P.records + (int64_t)row * P.n_slices);
    for (int i0 = lane; i0 < P.n_slices; i0 += 64 * 8) {
        u32x4 q[8];
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            const int i = i0 + 64 * k;
            q[k] = __builtin_nontemporal_load(rec + (i < P.n_slices ? i : lane));   // (lane < n_slices here: i0 = lane is)
        }
#pragma unroll
        for (int k = 0; k < 8; ++k)
            if (i0 + 64 * k < P.n_slices) fold(__uint_as_float(q[k].x), __uint_as_float(q[k].y), (int)q[k].z);
    }
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
        const float m2 = __shfl_xor(m, off), s2 = __shfl_xor(s, off);
        const int i2 = __shfl_xor(idx, off);
        fold(m2, s2, i2);
    }
    if (lane == 0) {
        // a row without any finite logit reports token 0 with confidence 0, like the two-step path
        P.x0[row] = idx == 0x7fffffff ? 0 : idx;
        P.x0_p[row] = idx == 0x7fffffff ? 0.f : fminf(1.0f / s, 1.0f);
    }
}

int slices_of(int64_t vocab) { return (int)((vocab + kTile - 1) / kTile) * (kTile / kSlice); }

}  // namespace

extern "C" int64_t mdx_lm_head_confidence_workspace_bytes(int64_t rows, int64_t vocab)
{
    if (rows <= 0 || vocab <= 0) return 0;
    return rows * slices_of(vocab) * (int64_t)sizeof(Record);
}

extern "C" int mdx_lm_head_confidence(const void* x, int64_t x_row_stride, const void* w, int64_t w_row_stride,
                                      const float* temperatures, int32_t rows_per_temp, const int64_t* row_ids,
                                      int64_t* x0, float* x0_p,
                                      int64_t rows, int64_t vocab, int64_t hidden,
                                      void* workspace, int64_t workspace_bytes, mdx_stream_t stream_)
{
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    MDX_REQUIRE(rows >= 0 && vocab >= 0 && hidden >= 0, MDX_EINVAL, "lm_head_confidence: negative size");
    if (rows == 0) return MDX_OK;
    MDX_REQUIRE(vocab > 0, MDX_EINVAL, "lm_head_confidence: empty vocabulary");
    MDX_REQUIRE(x && w && x0 && x0_p, MDX_EINVAL, "lm_head_confidence: null pointer");
    MDX_REQUIRE(hidden >= 128 && hidden % 128 == 0, MDX_EUNSUPPORTED, "lm_head_confidence: hidden %lld (multiples of 128)", (long long)hidden);
    MDX_REQUIRE(rows <= 65536 && vocab < ((int64_t)1 << 24), MDX_EUNSUPPORTED,
                "lm_head_confidence: rows %lld (max 65536) or vocab %lld (below 2^24) out of range", (long long)rows, (long long)vocab);
    MDX_REQUIRE(mdx::aligned16(x) && mdx::aligned16(w) && x_row_stride % 8 == 0 && w_row_stride % 8 == 0 &&
                x_row_stride >= hidden && w_row_stride >= hidden, MDX_EUNSUPPORTED,
                "lm_head_confidence: x and W must be 16-byte aligned with row strides that are multiples of 8 elements and at least hidden");
    MDX_REQUIRE(x_row_stride * 2 * kTile < ((int64_t)1 << 31) && w_row_stride * 2 * kTile < ((int64_t)1 << 31) &&
                x_row_stride * 2 < (1 << 24) && w_row_stride * 2 < (1 << 24), MDX_EUNSUPPORTED, "lm_head_confidence: row stride too large");
    MDX_REQUIRE(!temperatures || rows_per_temp > 0, MDX_EINVAL, "lm_head_confidence: rows_per_temp must be positive");
    const int64_t need = mdx_lm_head_confidence_workspace_bytes(rows, vocab);
    MDX_REQUIRE(workspace && workspace_bytes >= need, MDX_EWORKSPACE,
                "lm_head_confidence: workspace of %lld bytes needed, %lld given", (long long)need, (long long)workspace_bytes);
    MDX_REQUIRE(mdx::aligned16(workspace), MDX_EWORKSPACE, "lm_head_confidence: workspace not 16-byte aligned");
    MDX_REQUIRE(need < ((int64_t)1 << 32), MDX_EUNSUPPORTED, "lm_head_confidence: too many records");

    LmHeadParams P;
    P.x = (const __bf16*)x; P.w = (const __bf16*)w; P.x_stride = x_row_stride; P.w_stride = w_row_stride;
    P.temperatures = temperatures; P.rows_per_temp = rows_per_temp; P.row_ids = row_ids;
    P.rows = (int)rows; P.vocab = (int)vocab; P.hidden = (int)hidden;
    P.n_row_tiles = (int)((rows + kTile - 1) / kTile);
    P.n_vocab_tiles = (int)((vocab + kTile - 1) / kTile);
    P.n_slices = slices_of(vocab);
    P.records = static_cast<Record*>(workspace);
    P.x0 = x0; P.x0_p = x0_p;

    // the kernel's LDS limit is raised once per device
    static std::atomic<bool> lds_limit_raised[64];
    int device = 0;
    hipError_t e = hipGetDevice(&device);
    MDX_REQUIRE(e == hipSuccess && device >= 0 && device < 64, MDX_ELAUNCH, "lm_head_confidence: no current device (%s)", hipGetErrorString(e));
    if (!lds_limit_raised[device].load(std::memory_order_acquire)) {
        e = hipFuncSetAttribute(reinterpret_cast<const void*>(lm_head_confidence_kernel), hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes);
        MDX_REQUIRE(e == hipSuccess, MDX_ELAUNCH, "lm_head_confidence: cannot reserve %d bytes of LDS (%s)", kLdsBytes, hipGetErrorString(e));
        lds_limit_raised[device].store(true, std::memory_order_release);
    }
    const int64_t grid = (int64_t)((P.n_vocab_tiles + 7) / 8) * 8 * P.n_row_tiles;
    lm_head_confidence_kernel<<<(unsigned)grid, kThreads, kLdsBytes, stream>>>(P);
    int rc = mdx::check_launch("lm_head_confidence");
    if (rc != MDX_OK) return rc;
    lm_head_finalize_kernel<<<(unsigned)((rows + kThreads / 64 - 1) / (kThreads / 64)), kThreads, 0, stream>>>(P);
    return mdx::check_launch("lm_head_finalize");
}
