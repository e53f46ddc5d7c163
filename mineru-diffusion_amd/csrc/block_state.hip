// Per-sequence denoising-block state kept on the device between passes, so that a decode pass needs
// neither an upload of its inputs nor a blocking download of its results:
//
//   block_prepare   positions, slot_mapping and context_lens of the pass from each sequence's length and
//                   page table -- ModelRunner.prepare_decode, engine/model_runner.py:169-185, with
//                   Sequence.get_slots (engine/sequence.py:117-141) evaluated per position
//   masked_rows     the rows (sequence, position) of the batch that are still masked, compacted in order,
//                   for a vocabulary projection restricted to them (the sampler reads no other row:
//                   layers/sampler.py:39,54)
//   block_advance   what Sampler.forward does to the Sequence after the selection (layers/sampler.py:56-59)
//                   and Scheduler.postprocess after that (engine/scheduler.py:65-82): step map, step
//                   counter, denoising -> caching once no mask is left, and after the caching pass the
//                   append of the finished block, the stop-token / budget check and a fresh all-mask block
//
// All three are tiny (one wavefront per sequence); they exist so that the whole pass is a fixed
// sequence of launches that a HIP graph can hold.
#include "mdx_common.h"

namespace {

constexpr int kIdle = 0, kDenoising = 1, kCaching = 2;     // MDX_PHASE_*

__global__ __launch_bounds__(64) void block_prepare_kernel(
    const int32_t* __restrict__ lens, const int32_t* __restrict__ phase,
    const int32_t* __restrict__ block_table, int64_t bt_stride, int max_pages, int page_size, int block_len,
    int64_t* __restrict__ positions, int32_t* __restrict__ slot_mapping, int32_t* __restrict__ context_lens)
{
    const int b = blockIdx.x;
    const bool live = phase[b] != kIdle;
    const int len = lens[b];
    for (int p = threadIdx.x; p < block_len; p += 64) {
        const int t = len + p;
        int slot = -1;
        if (live && t >= 0) {
            const int pg = t / page_size;
            if (pg < max_pages) {
                const int id = block_table[(int64_t)b * bt_stride + pg];
                if (id >= 0) slot = id * page_size + t % page_size;
            }
        }
        positions[(int64_t)b * block_len + p] = live ? t : 0;
        slot_mapping[(int64_t)b * block_len + p] = slot;
    }
    if (threadIdx.x == 0) context_lens[b] = live ? len + block_len : 0;
}

// One workgroup scans the whole batch in order; 1024 elements per round, ballots give the offsets.
__global__ __launch_bounds__(1024) void masked_rows_kernel(
    const int64_t* __restrict__ tokens, const int32_t* __restrict__ phase, int64_t mask_token_id,
    int n, int block_len, int64_t* __restrict__ rows_out, int rows_cap, int32_t* __restrict__ n_rows_out)
{
    __shared__ int wave_count[16];
    __shared__ int base_s;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    if (tid == 0) base_s = 0;
    __syncthreads();
    for (int at = 0; at < n; at += 1024) {
        const int e = at + tid;
        const bool m = e < n && phase[e / block_len] == kDenoising && tokens[e] == mask_token_id;
        const unsigned long long bal = __ballot(m);
        if (lane == 0) wave_count[wave] = __popcll(bal);
        __syncthreads();
        int before = base_s;
        for (int w = 0; w < wave; ++w) before += wave_count[w];
        const int mine = before + __popcll(bal & ((1ull << lane) - 1ull));
        if (m && mine < rows_cap) rows_out[mine] = e;
        __syncthreads();
        if (tid == 0) {
            int total = 0;
            for (int w = 0; w < 16; ++w) total += wave_count[w];
            base_s += total;
        }
        __syncthreads();
    }
    const int found = base_s;
    // the rest of the fixed-size list repeats its first entry (row 0 when nothing is masked): rows
    // computed twice give the same values, so scattering their results back is harmless
    __syncthreads();
    const int64_t fill = (found > 0 && rows_cap > 0) ? rows_out[0] : 0;     // rows_cap == 0: rows_out may be null, only the count is wanted
    for (int i = (found < rows_cap ? found : rows_cap) + tid; i < rows_cap; i += 1024) rows_out[i] = fill;
    if (tid == 0) *n_rows_out = found;
}

struct AdvanceParams {
    int64_t* tokens; const uint8_t* transfer;
    int32_t* step_map; int32_t* step; int32_t* phase; int32_t* lens;
    const int32_t* first_len; const int32_t* max_new;
    const int64_t* stop_ids; int n_stop;
    int64_t* out_tokens; int32_t* out_steps; int64_t out_stride;
    int32_t* status;
    int64_t mask_token_id; int block_len;
};

__global__ __launch_bounds__(64) void block_advance_kernel(const AdvanceParams P)
{
    const int b = blockIdx.x, lane = threadIdx.x;
    const int ph = P.phase[b];
    const int S = P.block_len;
    if (ph == kIdle) {
        if (lane == 0) { P.status[4 * b + 0] = kIdle; P.status[4 * b + 2] = 0; P.status[4 * b + 3] = 0; }
        return;
    }
    const int step = P.step[b];
    int n_masked = 0, n_moved = 0;
    bool stop_hit = false;
    for (int p0 = 0; p0 < S; p0 += 64) {
        const int p = p0 + lane;
        const bool on = p < S;
        const int64_t at = (int64_t)b * S + p;
        const int64_t tok = on ? P.tokens[at] : 0;
        const bool moved = on && P.transfer[at] != 0;
        if (moved) P.step_map[at] = step;                                   // sampler.py:58
        n_moved += __popcll(__ballot(moved));
        n_masked += __popcll(__ballot(on && tok == P.mask_token_id));
        if (ph == kCaching) {
            bool hit = false;
            for (int s = 0; s < P.n_stop; ++s) hit |= on && tok == P.stop_ids[(int64_t)b * P.n_stop + s] && P.stop_ids[(int64_t)b * P.n_stop + s] >= 0;
            stop_hit |= __ballot(hit) != 0;
        }
    }
    int new_phase = ph, len = P.lens[b];
    if (ph == kDenoising) {
        if (n_masked == 0) new_phase = kCaching;                             // scheduler.py:67-69
    } else {
        // this pass stored the finished block's K/V: append it (sequence.py:97-101), then finish or go on
        const int done = len - P.first_len[b];
        for (int p = lane; p < S; p += 64) {
            const int64_t at = (int64_t)b * S + p;
            if (done >= 0 && done + p < P.out_stride) {                           // a full output row drops the rest
                P.out_tokens[(int64_t)b * P.out_stride + done + p] = P.tokens[at];
                P.out_steps[(int64_t)b * P.out_stride + done + p] = P.step_map[at];   // written by this same lane above, if at all
            }
            P.tokens[at] = P.mask_token_id;
        }
        len += S;
        n_masked = S;
        new_phase = (stop_hit || len - P.first_len[b] >= P.max_new[b]) ? kIdle : kDenoising;   // scheduler.py:76-82
    }
    if (lane == 0) {
        P.step[b] = step + 1;                                                // sampler.py:59
        P.phase[b] = new_phase;
        P.lens[b] = len;
        P.status[4 * b + 0] = new_phase;
        P.status[4 * b + 1] = len;
        P.status[4 * b + 2] = new_phase == kIdle ? 0 : n_masked;
        P.status[4 * b + 3] = n_moved;
    }
}

}  // namespace

extern "C" int mdx_block_prepare(const int32_t* lens, const int32_t* phase,
                                 const int32_t* block_table, int64_t bt_stride, int32_t max_pages,
                                 int32_t page_size, int32_t block_len,
                                 int64_t* positions, int32_t* slot_mapping, int32_t* context_lens,
                                 int32_t bs, mdx_stream_t stream)
{
    MDX_REQUIRE(bs >= 0 && block_len >= 0 && max_pages >= 0, MDX_EINVAL, "block_prepare: negative size");
    MDX_REQUIRE(page_size > 0, MDX_EINVAL, "block_prepare: page_size %d", page_size);
    if (bs == 0) return MDX_OK;
    MDX_REQUIRE(lens && phase && block_table && positions && slot_mapping && context_lens, MDX_EINVAL, "block_prepare: null pointer");
    MDX_REQUIRE(bt_stride >= max_pages, MDX_EINVAL, "block_prepare: bt_stride < max_pages");
    block_prepare_kernel<<<(unsigned)bs, 64, 0, static_cast<hipStream_t>(stream)>>>(
        lens, phase, block_table, bt_stride, max_pages, page_size, block_len, positions, slot_mapping, context_lens);
    return mdx::check_launch("block_prepare");
}

extern "C" int mdx_masked_rows(const int64_t* tokens, const int32_t* phase, int64_t mask_token_id,
                               int32_t bs, int32_t block_len,
                               int64_t* rows_out, int32_t rows_cap, int32_t* n_rows_out, mdx_stream_t stream)
{
    MDX_REQUIRE(bs >= 0 && block_len > 0 && rows_cap >= 0, MDX_EINVAL, "masked_rows: bad size");
    MDX_REQUIRE((int64_t)bs * block_len < (1ll << 30), MDX_EUNSUPPORTED, "masked_rows: batch too large");
    MDX_REQUIRE(n_rows_out && (rows_cap == 0 || rows_out), MDX_EINVAL, "masked_rows: null pointer");
    MDX_REQUIRE(bs == 0 || (tokens && phase), MDX_EINVAL, "masked_rows: null pointer");
    masked_rows_kernel<<<1, 1024, 0, static_cast<hipStream_t>(stream)>>>(
        tokens, phase, mask_token_id, bs * block_len, block_len, rows_out, rows_cap, n_rows_out);
    return mdx::check_launch("masked_rows");
}

extern "C" int mdx_block_advance(int64_t* tokens, const uint8_t* transfer,
                                 int32_t* step_map, int32_t* step, int32_t* phase, int32_t* lens,
                                 const int32_t* first_len, const int32_t* max_new,
                                 const int64_t* stop_ids, int32_t n_stop,
                                 int64_t* out_tokens, int32_t* out_steps, int64_t out_stride,
                                 int32_t* status, int64_t mask_token_id,
                                 int32_t bs, int32_t block_len, mdx_stream_t stream)
{
    MDX_REQUIRE(bs >= 0 && block_len > 0 && n_stop >= 0, MDX_EINVAL, "block_advance: bad size");
    if (bs == 0) return MDX_OK;
    MDX_REQUIRE(tokens && transfer && step_map && step && phase && lens && first_len && max_new && out_tokens && out_steps && status,
                MDX_EINVAL, "block_advance: null pointer");
    MDX_REQUIRE(n_stop == 0 || stop_ids, MDX_EINVAL, "block_advance: stop_ids missing");
    MDX_REQUIRE(out_stride >= block_len, MDX_EINVAL, "block_advance: out_stride smaller than a block");
    AdvanceParams P;
    P.tokens = tokens; P.transfer = transfer; P.step_map = step_map; P.step = step; P.phase = phase; P.lens = lens;
    P.first_len = first_len; P.max_new = max_new; P.stop_ids = stop_ids; P.n_stop = n_stop;
    P.out_tokens = out_tokens; P.out_steps = out_steps; P.out_stride = out_stride; P.status = status;
    P.mask_token_id = mask_token_id; P.block_len = block_len;
    block_advance_kernel<<<(unsigned)bs, 64, 0, static_cast<hipStream_t>(stream)>>>(P);
    return mdx::check_launch("block_advance");
}
