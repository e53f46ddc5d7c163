// Paged single-block attention for callers that cannot allocate: the split-KV partials live in a
// file-scope device array of this file instead of a caller workspace.  The array's name is only a
// host-side handle; its device address is looked up once per device with hipGetSymbolAddress, and
// that pointer is what the kernels (those of paged_attn.hip, unchanged) receive.
#include "mdx_common.h"
#include <atomic>

namespace mdx {
int launch_paged(const void* q, void* o, const void* k_cache, const void* v_cache,
                 int64_t q_stride_b, int64_t q_stride_s, int64_t q_stride_h,
                 int64_t o_stride_b, int64_t o_stride_s, int64_t o_stride_h,
                 int64_t cache_stride_page, int64_t cache_stride_tok, int64_t cache_stride_head,
                 const int32_t* block_table, int64_t bt_stride, const int32_t* context_lens,
                 int32_t bs, int32_t sq, int32_t num_q_heads, int32_t num_kv_heads,
                 int32_t head_dim, int32_t max_pages, int32_t page_size, int64_t num_pages,
                 float scale, int32_t dtype,
                 void* workspace, int64_t workspace_bytes, bool single_launch, void* counters, int64_t counter_bytes,
                 mdx_stream_t stream_);
}

namespace {

constexpr int64_t kStaticScratchBytes = 40ll << 20;       // covers 32 sequences x 16 heads x 4 splits (32.5 MiB) and 16 x 16 x 6 (24.4 MiB)
constexpr int kMaxDevices = 64;
__attribute__((used)) static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];
std::atomic<void*> scratch_ptr[kMaxDevices];              // per device: each GPU holds its own copy of the array

int static_scratch(void** out)
{
    int device = -1;
    hipError_t e = hipGetDevice(&device);
    MDX_REQUIRE(e == hipSuccess && device >= 0 && device < kMaxDevices, MDX_ELAUNCH,
                "paged_block_attn_static: no current device (%s)", hipGetErrorString(e));
    void* ptr = scratch_ptr[device].load(std::memory_order_acquire);
    if (!ptr) {
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        MDX_REQUIRE(e == hipSuccess && ptr, MDX_ELAUNCH, "paged_block_attn_static: hipGetSymbolAddress failed (%s)", hipGetErrorString(e));
        scratch_ptr[device].store(ptr, std::memory_order_release);   // two racing first calls store the same address
    }
    *out = ptr;
    return MDX_OK;
}

}  // namespace

extern "C" int mdx_paged_block_attn_static(const void* q, void* o, const void* k_cache, const void* v_cache,
                                           int64_t q_stride_b, int64_t q_stride_s, int64_t q_stride_h,
                                           int64_t o_stride_b, int64_t o_stride_s, int64_t o_stride_h,
                                           int64_t cache_stride_page, int64_t cache_stride_tok, int64_t cache_stride_head,
                                           const int32_t* block_table, int64_t bt_stride, const int32_t* context_lens,
                                           int32_t bs, int32_t sq, int32_t num_q_heads, int32_t num_kv_heads,
                                           int32_t head_dim, int32_t max_pages, int32_t page_size, int64_t num_pages,
                                           float scale, int32_t dtype, mdx_stream_t stream)
{
    const int64_t need = mdx_paged_block_attn_workspace_bytes(bs, sq, num_q_heads, num_kv_heads, head_dim, max_pages, page_size);
    MDX_REQUIRE(need <= kStaticScratchBytes, MDX_EWORKSPACE,
                "paged_block_attn_static: this shape needs %lld bytes of split partials, the static array holds %lld; "
                "use mdx_paged_block_attn with a workspace", (long long)need, (long long)kStaticScratchBytes);
    void* ws = nullptr;
    if (need > 0) {
        const int rc = static_scratch(&ws);
        if (rc != MDX_OK) return rc;
    }
    // Nothing in the array has to start at zero: every partial slot that the combine kernel reads was
    // written by the attention kernel of the same call.
    return mdx::launch_paged(q, o, k_cache, v_cache, q_stride_b, q_stride_s, q_stride_h, o_stride_b, o_stride_s, o_stride_h,
                        cache_stride_page, cache_stride_tok, cache_stride_head, block_table, bt_stride, context_lens,
                        bs, sq, num_q_heads, num_kv_heads, head_dim, max_pages, page_size, num_pages, scale, dtype,
                        ws, need > 0 ? kStaticScratchBytes : 0, false, nullptr, 0, stream);
}
