// Device-side commit plan of the request-row KDA replay (vLLM-style runner).  From the sampled-token counts,
// the source checkpoints and, in align mode, the block table, every request gets four integers
//     commit length, final slot, boundary slot, boundary length
// without any value leaving the device, so a commit can be captured in a graph.  The plan must equal the one
// the reference computes (src/decode/kda_replayssm_vllm/commit_plan.cu:19-117; expected values
// tests/test_kda_replayssm_vllm.py:148-178); the rules, as a specification:
//
//   live       a request whose source slot is valid (> null_block_id, >= 0, < slots) and whose query interval
//              [offsets[b], offsets[b + 1]) is well formed (0 <= begin < end <= token_capacity, length <= Q).
//   commits    a live request with offsets[0] == 0 and a sampler row (mapping[b], or b) inside the table commits
//              n = min(max(sampled[row], 0), length) tokens into its source slot.
//   align      with a block table (block_size > 0) and p = computed[row] tokens already in the cache, the state
//              after n tokens belongs to the block holding token p + n - 1 (the last column when beyond the
//              table), and when the window reaches the next block boundary (n >= block_size - p % block_size)
//              the state after that many tokens also belongs to the block of position p.  A row outside the
//              block table, a negative p, an invalid destination, a boundary column beyond the table, or a
//              boundary block equal to the final block with a different length cancels the request.
//   exclusive  every slot a request writes (final, boundary) must be touched by no other request, where a
//              live request touches its source and a committing one also its destinations; and the source of a
//              committing request must be no other request's destination.  Both sides of a clash are cancelled.
//
// One kernel, one workgroup.  Pass 1 (a thread per request) turns each request into three claims - the slot it
// reads and the up to two slots it writes, -1 for none - and a provisional plan row.  Pass 2 (a wavefront per
// committing request, lanes striding over the other requests) looks its slots up among everybody else's claims;
// the claims are never modified, so a clash cancels both sides whichever is examined first.  The claims live in
// LDS, or in the caller's scratch rows when the capacity exceeds what LDS holds.

#include "common.h"

namespace pla {

struct PlanInputs {
  const void* sampled; const void* source; const void* offsets; const void* mapping; const void* computed;
  const void* blocks;
  int sampled_wide, source_wide, offsets_wide, mapping_wide, computed_wide, blocks_wide;
  int batch, capacity, sampler_rows, block_rows, block_cols, slots, Q, null_id, token_capacity;
  int64_t block_row_stride, block_col_stride, block_size;

  __device__ int64_t at(const void* base, int wide, int64_t i) const {
    return wide ? static_cast<const int64_t*>(base)[i] : (int64_t) static_cast<const int32_t*>(base)[i];
  }
  __device__ bool slot_ok(int64_t slot) const { return slot > null_id && slot >= 0 && slot < slots; }
  __device__ int64_t block_of(int64_t row, int64_t col) const {
    return at(blocks, blocks_wide, row * block_row_stride + col * block_col_stride);
  }
};

constexpr int32_t NO_CLAIM = -1;        // an absent claim of another request: equals no valid slot
constexpr int32_t NO_SLOT = -2;         // an absent slot of the examined request: equals no claim at all
constexpr int PLAN_THREADS = 1024;
constexpr int PLAN_LDS_CAPACITY = 4096; // requests whose claims fit into 48 KB of LDS (3 x 4 bytes each)

struct Request {
  int32_t reads;                        // source slot of a live request, else NO_CLAIM
  int32_t tokens, final_slot, boundary_slot, boundary_tokens;     // zeroes unless it commits
};

__device__ Request classify(const PlanInputs& in, int b) {
  Request r{NO_CLAIM, 0, 0, 0, 0};
  if (b >= in.batch) return r;
  const int64_t source = in.at(in.source, in.source_wide, b);
  const int64_t begin = in.at(in.offsets, in.offsets_wide, b), end = in.at(in.offsets, in.offsets_wide, b + 1);
  const int64_t length = end - begin;
  const bool live = in.slot_ok(source) && begin >= 0 && length > 0 && end <= in.token_capacity && length <= in.Q;
  if (!live) return r;
  r.reads = (int32_t)source;
  const int64_t row = in.mapping ? in.at(in.mapping, in.mapping_wide, b) : (int64_t)b;
  if (in.at(in.offsets, in.offsets_wide, 0) != 0 || row < 0 || row >= in.sampler_rows) return r;
  const int64_t sampled = in.at(in.sampled, in.sampled_wide, row);
  const int64_t n = sampled <= 0 ? 0 : (sampled < length ? sampled : length);
  if (n == 0) return r;
  int64_t final_slot = source, boundary_slot = 0, boundary_tokens = 0;
  bool ok = true;
  if (in.block_size != 0) {             // align mode: destinations come from the block table
    ok = row < in.block_rows;
    const int64_t cached = ok ? in.at(in.computed, in.computed_wide, row) : -1;
    ok = ok && cached >= 0 && cached <= INT64_MAX - in.Q;
    if (ok) {
      int64_t last_col = (cached + n - 1) / in.block_size;
      if (last_col > in.block_cols - 1) last_col = in.block_cols - 1;
      final_slot = in.block_of(row, last_col);
      ok = in.slot_ok(final_slot);
      const int64_t to_boundary = in.block_size - cached % in.block_size;
      if (ok && n >= to_boundary) {     // the window reaches the end of the block that holds position `cached`
        const int64_t col = cached / in.block_size;
        ok = col < in.block_cols;
        if (ok) {
          boundary_slot = in.block_of(row, col);
          // one block cannot hold two different states
          ok = in.slot_ok(boundary_slot) && !(boundary_slot == final_slot && to_boundary != n);
          boundary_tokens = to_boundary;
        }
      }
    }
  }
  if (!ok) return r;
  r.tokens = (int32_t)n;
  r.final_slot = (int32_t)final_slot;
  r.boundary_slot = (int32_t)boundary_slot;
  r.boundary_tokens = (int32_t)boundary_tokens;
  return r;
}

__global__ __launch_bounds__(PLAN_THREADS) void commit_plan_kernel(const PlanInputs in, int32_t* spill, int32_t* plan) {
  extern __shared__ int32_t claims_lds[];
  int32_t* const reads = in.capacity <= PLAN_LDS_CAPACITY ? claims_lds : spill;
  int32_t* const writes_final = reads + in.capacity;
  int32_t* const writes_boundary = writes_final + in.capacity;
  const int cap = in.capacity;

  for (int b = threadIdx.x; b < cap; b += PLAN_THREADS) {
    const Request r = classify(in, b);
    reads[b] = r.reads;
    writes_final[b] = r.tokens > 0 ? r.final_slot : NO_CLAIM;
    writes_boundary[b] = r.boundary_tokens > 0 ? r.boundary_slot : NO_CLAIM;
    plan[b] = r.tokens;
    plan[cap + b] = r.final_slot;
    plan[2 * cap + b] = r.boundary_slot;
    plan[3 * cap + b] = r.boundary_tokens;
  }
  __syncthreads();

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (int b = wave; b < in.batch; b += PLAN_THREADS / 64) {
    const int32_t mine_final = writes_final[b];
    if (mine_final == NO_CLAIM) continue;                      // wave-uniform: b commits nothing
    const int32_t mine_boundary = writes_boundary[b] == NO_CLAIM ? NO_SLOT : writes_boundary[b];
    const int32_t mine_source = reads[b];                      // a committing request is live
    bool clash = false;
    for (int other = lane; other < in.batch; other += 64) {
      if (other == b) continue;
      const int32_t r = reads[other], f = writes_final[other], d = writes_boundary[other];
      const bool written_slot_taken = mine_final == r || mine_final == f || mine_final == d ||
                                      mine_boundary == r || mine_boundary == f || mine_boundary == d;
      const bool source_overwritten = mine_source == f || mine_source == d;
      clash = clash || written_slot_taken || source_overwritten;
    }
    if (__ballot(clash) != 0 && lane < 4) plan[lane * cap + b] = 0;
  }
}

}  // namespace pla

extern "C" int pla_kda_commit_plan_launch(
    const void* sampled, int sampled_wide, const void* source, int source_wide, const void* offsets, int offsets_wide,
    const void* mapping, int mapping_wide, const void* computed, int computed_wide, const void* blocks, int blocks_wide,
    int batch, int capacity, int sampler_rows, int block_rows, int block_cols, int slots, int Q, int null_block_id,
    int token_capacity, int64_t block_row_stride, int64_t block_col_stride, int64_t block_size,
    int32_t* candidate, int32_t* plan, void* stream) {
  using namespace pla;
  if (capacity == 0) return 0;
  PLA_REQUIRE(sampled && source && offsets && candidate && plan, "null tensor pointer");
  PLA_REQUIRE(batch >= 0 && batch <= capacity && capacity > 0, "commit query count exceeds capacity");
  PLA_REQUIRE(Q >= 1 && Q <= 32 && slots > 0, "invalid commit plan dimensions");
  PLA_REQUIRE(null_block_id == -1 || null_block_id == 0, "null_block_id must be -1 or 0");
  PLA_REQUIRE(token_capacity >= 0, "token_capacity must be between 0 and INT32_MAX");
  PLA_REQUIRE((blocks != nullptr) == (computed != nullptr) && (blocks != nullptr) == (block_size != 0),
              "align arguments must be supplied together");
  PLA_REQUIRE(blocks == nullptr || (block_size >= Q && block_cols > 0 && block_rows >= 0), "invalid align table/count/block size");
  const PlanInputs in{sampled, source, offsets, mapping, computed, blocks,
                      sampled_wide, source_wide, offsets_wide, mapping_wide, computed_wide, blocks_wide,
                      batch, capacity, sampler_rows, block_rows, block_cols, slots, Q, null_block_id, token_capacity,
                      block_row_stride, block_col_stride, block_size};
  const size_t lds = capacity <= PLAN_LDS_CAPACITY ? (size_t)capacity * 3 * sizeof(int32_t) : 0;
  commit_plan_kernel<<<dim3(1), dim3(PLAN_THREADS), lds, static_cast<hipStream_t>(stream)>>>(in, candidate, plan);
  return check_launch("commit_plan_kernel");
}
