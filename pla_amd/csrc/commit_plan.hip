// Device-side commit plan of the request-row KDA replay (vLLM-style runner): from the sampled-token
// counts, the source checkpoints and, in align mode, the block table, every request gets
//     commit_len, final slot, boundary slot, boundary length
// without any value leaving the device, so a commit can be captured in a graph.  Restates
// build_plan / protect_plan of the reference (src/decode/kda_replayssm_vllm/commit_plan.cu:19-117):
//   * a request commits min(max(sampled[row], 0), query length) tokens, row = mapping[b] or b, provided
//     offsets[0] == 0, the row is inside the sampler table, the source slot is valid (> null_block_id,
//     < slots) and the query interval is well formed (0 <= begin < end <= token_capacity, length <= Q);
//   * align mode (block_size > 0): with p tokens already computed, the final state goes to the block that
//     holds token p + n - 1 (last column when beyond the table); when the window reaches the next block
//     boundary (n >= block_size - p % block_size) the state after that many tokens also goes to the block
//     of position p.  An invalid destination, or a boundary equal to the final block with a different
//     length, cancels the request;
//   * a request is cancelled when one of its destinations is another live query's source or one of another
//     committing request's destinations, or when its source is another request's destination (both sides
//     of a conflict are cancelled: the check reads the immutable candidate table and writes a separate plan).
// Cancelled and inactive rows hold zeroes in all four columns.

#include "common.h"

namespace pla {

struct PlanParams {
  const void* sampled; const void* source; const void* offsets; const void* mapping; const void* computed;
  const void* blocks;
  int sampled_wide, source_wide, offsets_wide, mapping_wide, computed_wide, blocks_wide;
  int batch, capacity, sampler_rows, block_rows, block_cols, slots, Q, null_id, token_capacity;
  int64_t block_row_stride, block_col_stride, block_size;
};

__device__ __forceinline__ int64_t plan_value(const void* p, int wide, int64_t i) {
  return wide ? reinterpret_cast<const int64_t*>(p)[i] : (int64_t) reinterpret_cast<const int32_t*>(p)[i];
}
__device__ __forceinline__ bool plan_valid_slot(int64_t slot, const PlanParams& p) {
  return slot > p.null_id && slot >= 0 && slot < p.slots;
}
__device__ __forceinline__ bool plan_valid_interval(int64_t begin, int64_t end, const PlanParams& p) {
  return begin >= 0 && end > begin && end <= p.token_capacity && end - begin <= p.Q;
}

// candidate[c * capacity + b], c = 0..3: commit length, final slot, boundary slot, boundary length
__global__ void commit_plan_candidates_kernel(const PlanParams p, int32_t* candidate) {
  const int b = blockIdx.x * blockDim.x + threadIdx.x;
  if (b >= p.capacity) return;
  int64_t count = 0, final_slot = 0, boundary = 0, bc = 0;
  if (b < p.batch) {
    const int64_t row = p.mapping != nullptr ? plan_value(p.mapping, p.mapping_wide, b) : b;
    const int64_t source = plan_value(p.source, p.source_wide, b);
    const int64_t begin = plan_value(p.offsets, p.offsets_wide, b), end = plan_value(p.offsets, p.offsets_wide, b + 1);
    if (plan_value(p.offsets, p.offsets_wide, 0) == 0 && row >= 0 && row < p.sampler_rows && plan_valid_slot(source, p) &&
        plan_valid_interval(begin, end, p)) {
      const int64_t sampled = plan_value(p.sampled, p.sampled_wide, row);
      count = sampled <= 0 ? 0 : (sampled > end - begin ? end - begin : sampled);
      final_slot = source;
      if (count > 0 && p.block_size > 0) {
        const int64_t pos = row < p.block_rows ? plan_value(p.computed, p.computed_wide, row) : -1;
        if (row >= p.block_rows || pos < 0 || pos > INT64_MAX - p.Q) {
          count = 0;
        } else {
          int64_t col = (pos + count - 1) / p.block_size;
          if (col >= p.block_cols) col = p.block_cols - 1;
          const int64_t f = plan_value(p.blocks, p.blocks_wide, row * p.block_row_stride + col * p.block_col_stride);
          if (!plan_valid_slot(f, p)) count = 0;
          else final_slot = f;
          const int64_t distance = p.block_size - pos % p.block_size;       // tokens up to the next block boundary
          if (count > 0 && count >= distance) {
            const int64_t boundary_col = pos / p.block_size;
            if (boundary_col >= p.block_cols) {
              count = 0;
            } else {
              const int64_t dest = plan_value(p.blocks, p.blocks_wide,
                                              row * p.block_row_stride + boundary_col * p.block_col_stride);
              if (!plan_valid_slot(dest, p) || (dest == final_slot && distance != count)) count = 0;
              else { boundary = dest; bc = distance; }
            }
          }
        }
      }
    }
  }
  candidate[b] = (int32_t)count;
  candidate[p.capacity + b] = count ? (int32_t)final_slot : 0;
  candidate[2 * p.capacity + b] = count ? (int32_t)boundary : 0;
  candidate[3 * p.capacity + b] = count ? (int32_t)bc : 0;
}

// One wavefront per row: its lanes stride over the other requests.
__global__ __launch_bounds__(256) void commit_plan_protect_kernel(const PlanParams p, const int32_t* candidate, int32_t* plan) {
  const int lane = threadIdx.x & 63;
  const int b = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (b >= p.capacity) return;
  bool conflict = false;
  if (candidate[b] != 0) {
    const int64_t source = plan_value(p.source, p.source_wide, b);
    const int f = candidate[p.capacity + b], d = candidate[2 * p.capacity + b];
    const bool has_d = candidate[3 * p.capacity + b] > 0;
    for (int other = lane; other < p.batch; other += 64) {
      if (other == b) continue;
      const int64_t os = plan_value(p.source, p.source_wide, other);
      const int64_t begin = plan_value(p.offsets, p.offsets_wide, other), end = plan_value(p.offsets, p.offsets_wide, other + 1);
      // a live query that commits nothing still owns its source checkpoint
      if (plan_valid_slot(os, p) && plan_valid_interval(begin, end, p)) conflict |= f == os || (has_d && d == os);
      if (candidate[other] == 0) continue;
      const int of = candidate[p.capacity + other], od = candidate[2 * p.capacity + other];
      const bool has_od = candidate[3 * p.capacity + other] > 0;
      conflict |= f == os || f == of || (has_od && f == od) || (has_d && (d == os || d == of || (has_od && d == od))) ||
                  source == of || (has_od && source == od);
    }
  }
  conflict = __ballot(conflict) != 0;
  if (lane < 4) plan[lane * p.capacity + b] = conflict ? 0 : candidate[lane * p.capacity + b];
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
  PlanParams p{sampled, source, offsets, mapping, computed, blocks,
               sampled_wide, source_wide, offsets_wide, mapping_wide, computed_wide, blocks_wide,
               batch, capacity, sampler_rows, block_rows, block_cols, slots, Q, null_block_id, token_capacity,
               block_row_stride, block_col_stride, block_size};
  hipStream_t s = static_cast<hipStream_t>(stream);
  commit_plan_candidates_kernel<<<dim3((capacity + 127) / 128), dim3(128), 0, s>>>(p, candidate);
  if (check_launch("commit_plan_candidates_kernel")) return 1;
  commit_plan_protect_kernel<<<dim3((capacity + 3) / 4), dim3(256), 0, s>>>(p, candidate, plan);
  return check_launch("commit_plan_protect_kernel");
}
