/*
 * C ABI of libpla_gfx950.so: gated delta-rule (GDN / KDA) decode, MTP verify,
 * accepted-prefix commit and chunk-64 prefill for AMD MI355X (gfx950).
 *
 * Every entry point takes plain device pointers, sizes and element strides and
 * a hipStream_t (as void*); nothing is retained after the call returns, no
 * entry point allocates, synchronises or copies to the host, so every call is
 * hipGraph-capturable.  Return value: 0 on success, non-zero on a rejected
 * argument or a launch error; pla_last_error() then describes it.  Argument
 * rejections happen before any kernel is launched, so no state is written.
 *
 * Each declaration cites the interface of the reference (t-head/pla) that it
 * replaces.
 */
#ifndef PLA_GFX950_H
#define PLA_GFX950_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* element type codes */
enum {
  PLA_F32 = 0,
  PLA_BF16 = 1,
  PLA_F16 = 2
};

/* gate_mode of the k-last entry points */
enum {
  PLA_GATE_SOFTPLUS = 0,    /* g = -exp(A_log) * softplus_{beta,threshold}(a + dt_bias)           */
  PLA_GATE_LOWER_BOUND = 1, /* g = lower_bound * sigmoid(exp(A_log) * (a + dt_bias)), KDA only     */
  PLA_GATE_LOG_DECAY = 2    /* `a` already holds the float32 log-decay g; A_log/dt_bias ignored    */
};

/* Library identification: "pla_gfx950 <version> gfx950". */
const char* pla_version(void);

/* Message of the last failing call on this thread ("" if none). */
const char* pla_last_error(void);

/*
 * Packed one-token decode over an indexed k-last state pool.
 * Replaces k_last_packed_launcher_t
 * (src/decode/k-last/fused_sigmoid_gating_cuda_k_last_packed.cpp:53-80) and the
 * kernel fused_sigmoid_gating_delta_kernel_packed
 * (src/decode/k-last/fused_sigmoid_gating_k_last_packed_kernel.cuh:59-384).
 *
 *   mixed_qkv  [tokens, 2*H*128 + HV*128] act dtype, row pitch stride_qkv elements
 *   a          [tokens, HV] (GDN) or [tokens, HV*128] (KDA), pitch stride_a
 *   b          [tokens, HV], pitch stride_b
 *   A_log      [HV] of alog_dtype;  dt_bias [HV] or [HV*128] act dtype
 *   o          [tokens, HV, 128] act dtype, dense
 *   h0         state pool of state_dtype (PLA_F32, or PLA_BF16: widened on load, the FP32 result
 *              rounded to nearest even on store), slot pitch h0_slot_stride elements,
 *              slot = [HV,128(V),128(K)]
 *   cu_seqlens [B+1] int32 or NULL (then request n owns token n)
 *   h0_indices [B] int32; invalid slot (<0 when is_sglang, <=0 otherwise) => zeros in o,
 *              no state access;  a request of length 0 touches nothing.
 * rows_per_wave: 0 = pick from the gfx950 tuning table, else 8, 16 or 32.
 */
int pla_k_last_packed_launch(
    const void* A_log, int alog_dtype, const void* a, const void* dt_bias,
    float softplus_beta, float softplus_threshold,
    const void* mixed_qkv, const void* b, void* o, void* h0, int state_dtype,
    const int32_t* cu_seqlens, const int32_t* h0_indices,
    float scale, int T_max,
    int64_t stride_a, int64_t stride_qkv, int64_t stride_b, int64_t h0_slot_stride,
    int B, int H, int HV, int K, int V,
    int use_qk_l2norm, int is_sglang, int is_kda, int act_dtype,
    int rows_per_wave, void* stream);

/*
 * Non-packed decode and MTP / speculative verify.
 * Replaces k_last_launcher_t
 * (src/decode/k-last/fused_sigmoid_gating_cuda_k_last.cpp:161-199) and the kernel
 * fused_sigmoid_gating_delta_kernel
 * (src/decode/k-last/fused_sigmoid_gating_k_last_kernel.cuh:131-1058).
 *
 *   q,k [tokens,H,128], v [tokens,HV,128] act dtype with token pitches stride_q/k/v
 *   a: gate input (see gate_mode); with PLA_GATE_LOG_DECAY it is float32
 *   b: raw beta logits (act dtype), or float32 activated beta when beta_is_activated
 *   dt_bias: float32 when dt_bias_is_f32 else act dtype
 *   h0, cache: of state_dtype (PLA_F32 or PLA_BF16; snapshots are rounded like the pool)
 *   cache: SGLang intermediate-state buffer [rows, cache_steps, HV,128,128] or NULL;
 *          step t of request n is written to cache[cache_indices[n]*cache_steps + t]
 *          when is_sglang and cache_indices[n] >= 0
 *   parents: int64 [B, >=T] eagle-tree parent steps (needs cache), or NULL
 *   h0_indices: [B] (stride_h0_indices_seq == 0) or a 2-D [B,S] table with row pitch
 *          stride_h0_indices_seq (vLLM; requires !is_sglang): the start slot is column
 *          max(num_accepted[n]-1, 0) and step t is written to slot table[n][t] when > 0
 *   disable_state_update: do not write the final state back to the start slot
 */
int pla_k_last_launch(
    const void* A_log, int alog_dtype, const void* a, const void* dt_bias, int dt_bias_is_f32,
    float softplus_beta_or_lower_bound, float softplus_threshold, int gate_mode,
    const void* q, const void* k, const void* v, const void* b, int beta_is_activated,
    void* o, void* h0, int state_dtype, const int32_t* cu_seqlens, void* cache,
    const int32_t* h0_indices, const int32_t* cache_indices, int cache_steps,
    const int64_t* parents, int64_t stride_parent_seq, int64_t stride_parent_token,
    float scale, int T_max,
    int64_t stride_a, int64_t stride_q, int64_t stride_k, int64_t stride_v, int64_t stride_b,
    int64_t h0_slot_stride,
    int B, int H, int HV, int K, int V,
    int use_qk_l2norm, int disable_state_update,
    const int32_t* num_accepted, int64_t stride_h0_indices_seq, int is_sglang,
    int is_kda, int act_dtype, int rows_per_wave, void* stream);

/*
 * Accepted-prefix commit: replays accept_lens[n] recorded tokens of request n into
 * its FP32 state, in place.  Replaces launch_fold
 * (src/decode/kda_replayssm/kda_mtp_abi.h:165-176; kernel
 * src/decode/kda_replayssm/kda_mtp_fold.cu:256-545), all layers in one launch.
 *
 *   h0    [layers,slots,HV,128,128] float32, slot pitch h0_slot_stride, layer pitch h0_layer_stride
 *   rawk  [layers,slots,H,L,128]  act dtype (pre-normalisation; L2-normalised inside)
 *   rawv  [layers,slots,HV,L,128] act dtype
 *   gk    [layers,slots,HV,L,128] float32 log-decay;  beta [layers,slots,HV,L] float32
 *         (every tensor with its own slot and layer pitch, in elements; layers >= 1)
 *   slot_idx, accept_lens [B] int32.  slot <= null_block_id or accept_len <= 0 => untouched.
 *   track_idx, track_step [B] int32 or both NULL: the state after step track_step[n] (0-based) is also
 *         stored to slot track_idx[n] when that slot is > null_block_id.
 */
int pla_kda_fold_launch(
    float* h0, const void* rawv, const void* rawk, const float* gk, const float* beta,
    const int32_t* slot_idx, const int32_t* accept_lens,
    const int32_t* track_idx, const int32_t* track_step,
    int64_t h0_slot_stride, int64_t rawv_slot_stride, int64_t rawk_slot_stride,
    int64_t gk_slot_stride, int64_t beta_slot_stride,
    int layers, int64_t h0_layer_stride, int64_t rawv_layer_stride, int64_t rawk_layer_stride,
    int64_t gk_layer_stride, int64_t beta_layer_stride,
    int B, int H, int HV, int L, int null_block_id, int act_dtype, void* stream);

/*
 * Layer table of the paged (vLLM ReplaySSM) commit: device memory, PLA_LAYER_TABLE_ENTRIES int64 per layer
 * (the reference passes a table of layer descriptors the same way: `const int64_t* layers`,
 * src/decode/kda_replayssm/kda_mtp_abi.h:139-150).  Entries of layer l:
 *   0 checkpoint pool (float*, [slots,H,128,128]), 1 its slot pitch in floats,
 *   2 rawv, 3 rawk (bf16 [R,H,Q,128], dense), 4 gate (float [R,H,Q,128]), 5 beta (float [R,H,Q]),
 *   6 conv history (bf16*), 7-9 its slot / channel / tap pitches in elements,
 *   10 record windows (bf16*, [R,Q,channels,3]), 11-14 their row / step / channel / tap pitches, 15 unused.
 * Pools and records need 16-byte aligned bases, slot pitches a multiple of 4 floats.
 */
#define PLA_LAYER_TABLE_ENTRIES 16

/*
 * The fold of all layers driven by a commit plan over paged checkpoints with request-row records.  Replaces
 * launch_fold_native (src/decode/kda_replayssm/kda_mtp_abi.h:139-144): in every layer, request n replays
 * lengths[n] tokens of records row n from state[source[n]] and stores the result to
 * state[final_indices[n]]; when boundary_lengths[n] > 0 the state after that many tokens also goes to
 * state[boundary_indices[n]].  Destinations may equal the source slot.  Requests with lengths[n] <= 0 or a
 * source / final slot outside (null_block_id, slots) are skipped.
 */
int pla_kda_fold_native_launch(
    const int64_t* layer_table, int layers,
    const int32_t* source, const int32_t* lengths, const int32_t* final_indices,
    const int32_t* boundary_indices, const int32_t* boundary_lengths,
    int batch, int heads, int Q, int slots, int null_block_id, void* stream);

/*
 * The conv part of the same commit, all layers in one launch.  Replaces launch_conv_native
 * (src/decode/kda_replayssm/kda_mtp_abi.h:146-150): request n copies the record window after its
 * boundary_lengths[n]-th token into the conv history of slot boundary_indices[n] (when that length is
 * positive), then the window after its lengths[n]-th token into slot final_indices[n]; destinations
 * outside [0, slots) are skipped.  channels = 3 * H * 128, rows = record rows R.
 */
int pla_kda_conv_native_launch(
    const int64_t* layer_table, int layers, const int32_t* lengths, const int32_t* final_indices,
    const int32_t* boundary_indices, const int32_t* boundary_lengths,
    int batch, int channels, int Q, int rows, int slots, void* stream);

/*
 * Fused KDA decode step (one token per request): width-4 causal conv1d update + SiLU on the packed
 * q|k|v projection, q/k L2 norm, per-channel gate, delta-rule update of the indexed k-last FP32
 * state pool, optional gated RMSNorm of the output.  Replaces launch_kda_decode_mega
 * (src/decode/k-last/k_last_mega_abi.h:57-71; kernel
 * src/decode/k-last/fused_kda_decode_mega_kernel.cuh:138-729) argument for argument, with the
 * dtype enum replaced by PLA_BF16 / PLA_F16 and the stream passed as void*.
 *
 *   x_q, x_k, x_v   the three H*128-wide segments of a row of x [B, 3*H*128] (act dtype), row pitch x_row
 *   w_*_t           [4, H*128] float32 width-major conv weights per segment; bias_* [H*128] or NULL
 *   cs_q/k/v        the segments of conv_state [slots, 3*H*128, 3] in the SD layout: channel stride 1,
 *                   tap stride 3*H*128, slot pitch conv_slot (elements); shifted in place
 *   g [B,H,128], beta [B,H] (row pitch beta_row) raw gate / beta logits (act dtype);
 *   a_log [H], dt_bias [H*128] float32:  decay = exp(-exp(a_log) softplus(g + dt_bias)), or
 *                   exp(lower_bound sigmoid(exp(a_log) (g + dt_bias))) when use_lower_bound
 *   state [slots,H,128,128] float32 with slot pitch state_slot; state_indices [B] int32; a negative
 *                   slot writes zeros to the request's output row and touches neither pool
 *   out [B,H,128] act dtype, dense.  apply_onorm: out = o rsqrt(mean(o^2) + norm_eps) o_norm_weight
 *                   sigmoid(g_out), g_out [B,H,128] act dtype with row pitch onorm_row, weight [128] float32
 *   H must equal HV.  v is rounded to the activation dtype after SiLU (as the reference kernel does);
 *   q and k stay FP32.
 */
int pla_kda_decode_mega_launch(
    int act_dtype, int apply_onorm, int use_lower_bound,
    const float* a_log, const void* g, const float* dt_bias,
    const void* x_q, const void* x_k, const void* x_v, const void* beta,
    const float* w_q_t, const float* w_k_t, const float* w_v_t,
    const float* bias_q, const float* bias_k, const float* bias_v,
    void* cs_q, void* cs_k, void* cs_v,
    const void* g_out, const float* o_norm_weight, float norm_eps,
    float* state, const int32_t* state_indices, void* out,
    float scale, float lower_bound, int B, int H, int HV,
    int64_t x_row, int64_t beta_row, int64_t onorm_row,
    int64_t conv_slot, int64_t state_slot, void* stream);

/*
 * KDA speculative verify with replay records, ring mode (SGLang ReplaySSM).  Replaces launch_verify
 * (src/decode/kda_replayssm/kda_mtp_abi.h:316-330; kernel src/decode/kda_replayssm/kda_mtp_verify.cu,
 * host contract src/decode/kda_replayssm_sglang/kda_mtp_verify_host.cpp:50-243) with the stride structs
 * flattened and the index tensors passed as (pointer, is_int64).
 *
 *   x_q, x_k, x_v, g_in [T,H,128] bf16 (token strides strides[0..3]), beta_in [T,H] bf16 (strides[4])
 *   w_q, w_k, w_v   [H*128, 4] float32 conv weights, taps oldest first
 *   cs_q, cs_k, cs_v  conv states [slot, H*128, 3] bf16, read-only; strides[5..13] = (slot, channel, window) x 3
 *   ic_q, ic_k, ic_v  scratch windows [row, step, H*128, 3] bf16, written: the window after each token;
 *                   strides[14..25] = (row, step, channel, window) x 3
 *   a_log [H], dt_bias [H*128] float32: log-decay = lower_bound * sigmoid(exp(a_log) * (g + dt_bias))
 *   h0              [slots,H,128,128] float32 dense, read once, never written
 *   ring_rawv, ring_rawk [slots,H,L,128] bf16 (post-conv v and k, k before its L2 norm), ring_g
 *                   [slots,H,L,128] float32 log-decay, ring_beta [slots,H,L] float32: records of token t of
 *                   a request go to position t of its slot's rings
 *   out             [T,H,128] bf16 dense.  onorm_gate != NULL: out = o rsqrt(mean(o^2) + eps) weight
 *                   sigmoid(gate), gate [T,H,128] bf16 with token stride onorm_gate_stride
 *   slot_idx, scratch_idx, cu_seqlens: int32 or int64 ([N], [>=N], [N+1]); slot < 0: the request's
 *                   output rows are zeroed and nothing else is touched
 *   t_loop          draft tokens per request (1..32); ring_len = L >= t_loop
 */
int pla_kda_verify_dspark_launch(
    const void* x_q, const void* x_k, const void* x_v, const void* g_in, const void* beta_in,
    const float* w_q, const float* w_k, const float* w_v,
    const void* cs_q, const void* cs_k, const void* cs_v,
    const float* a_log, const float* dt_bias, const float* h0,
    void* out, void* ic_q, void* ic_k, void* ic_v,
    void* ring_rawv, void* ring_rawk, float* ring_g, float* ring_beta,
    const void* slot_idx, int slot_idx_wide, const void* scratch_idx, int scratch_idx_wide,
    const void* cu_seqlens, int cu_seqlens_wide,
    int H, int N, int t_loop, int ring_len, float scale, float lower_bound,
    const int64_t* strides,
    const void* onorm_gate, const float* onorm_weight, int64_t onorm_gate_stride, float onorm_eps,
    void* stream);

/*
 * The same verify over paged checkpoints with request-row records (vLLM ReplaySSM).  Replaces
 * launch_verify_native (src/decode/kda_replayssm/kda_mtp_abi.h:127-137; binding
 * src/decode/kda_replayssm_vllm/kda_replayssm_vllm.cpp:121-235).  Differences from the ring-mode entry:
 * records rawv / rawk / gate [R,H,Q,128], beta [R,H,Q] and windows ic_* [R,Q,.,3] are indexed by the
 * request row; the checkpoint pool has a slot pitch (state_slot_stride elements, slots entries); a slot
 * <= null_block_id (-1 or 0) is padding (zero output rows, nothing else written); a request whose query
 * interval is empty, longer than Q, not inside [0, tokens] or whose slot is >= slots is skipped entirely;
 * no fused output norm.  Q <= 32.
 */
int pla_kda_replay_verify_native_launch(
    const void* x_q, const void* x_k, const void* x_v, const void* g_in, const void* beta_in,
    const float* w_q, const float* w_k, const float* w_v,
    const void* cs_q, const void* cs_k, const void* cs_v,
    const float* a_log, const float* dt_bias, const float* h0,
    void* out, void* ic_q, void* ic_k, void* ic_v,
    void* rawv, void* rawk, float* gate, float* beta,
    const void* slot_idx, int slot_idx_wide, const void* cu_seqlens, int cu_seqlens_wide,
    int H, int N, int Q, float scale, float lower_bound, const int64_t* strides,
    int64_t state_slot_stride, int slots, int tokens, int null_block_id, void* stream);

/*
 * Device-side commit plan of the request-row replay: plan[c * capacity + b] for c = 0..3 = commit length,
 * final slot, boundary slot, boundary length of request b (zeroes for inactive, invalid and conflicting
 * requests).  Replaces launch_commit_plan (src/decode/kda_replayssm_vllm/commit_plan.h:7-14, kernels
 * commit_plan.cu:19-117).  Index vectors are dense int32 or int64 (is_int64 flags): sampled [sampler_rows],
 * source [batch], offsets [batch+1], mapping [batch] or NULL, computed [>= sampler rows] and blocks
 * [block_rows, block_cols] (strides in elements) or both NULL with block_size 0.  plan: int32 [4, capacity];
 * candidate: int32 scratch of the same size, a distinct buffer (it holds the requests' slot claims when the
 * capacity exceeds the 4096 requests whose claims fit into LDS).
 */
int pla_kda_commit_plan_launch(
    const void* sampled, int sampled_wide, const void* source, int source_wide, const void* offsets, int offsets_wide,
    const void* mapping, int mapping_wide, const void* computed, int computed_wide, const void* blocks, int blocks_wide,
    int batch, int capacity, int sampler_rows, int block_rows, int block_cols, int slots, int Q, int null_block_id,
    int token_capacity, int64_t block_row_stride, int64_t block_col_stride, int64_t block_size,
    int32_t* candidate, int32_t* plan, void* stream);

/*
 * Conv-window rollback of the commit: dst[layer, dst_idx[r], :, :] = src[layer, r, step_idx[r], :, :]
 * for every request r with step_idx[r] >= 0, 0 <= dst_idx[r] < dst_reqs, r < src_reqs and
 * step_idx[r] < src_steps.  Replaces launch_conv_scatter
 * (src/decode/kda_replayssm/kda_mtp_abi.h:177-186; kernel src/decode/kda_replayssm/kda_mtp_fold.cu:595-635).
 * src [layers, src_reqs, src_steps, dim, km1] with strides src_s0..4, dst [layers, dst_reqs, dim, km1]
 * with strides dst_s0..3 (elements of elem_bytes = 2 or 4); km1 = conv width - 1 (1..4).
 */
int pla_conv_window_scatter_launch(
    int elem_bytes, int km1, const void* src, void* dst,
    const void* dst_idx, int dst_idx_wide, const void* step_idx, int step_idx_wide,
    int layers, int dim, int reqs,
    int64_t src_s0, int64_t src_s1, int64_t src_s2, int64_t src_s3, int64_t src_s4,
    int64_t dst_s0, int64_t dst_s1, int64_t dst_s2, int64_t dst_s3,
    int src_reqs, int src_steps, int dst_reqs, void* stream);

/*
 * Workspace size in bytes (256-byte aligned buffer) needed by pla_gdn_prefill_launch for T physical
 * tokens in N sequences.  Chunk metadata is sized for the worst case T/64 + N chunks so that no
 * host copy of cu_seqlens is needed.
 */
int64_t pla_gdn_prefill_workspace_bytes(int T, int N, int H, int HV);

/*
 * GDN chunk-64 prefill over packed variable-length sequences (scalar gate per value head).
 * Replaces the FlashQLA stage launchers launch_*_cute
 * (src/prefill/flashqla/host/torch_extension_cute.cc:60-148: chunk_local_cumsum_qk_norm_gated,
 * kkt_solve, fused_fwd) with one call that runs all stages on `stream`.
 *
 *   q,k [T,H,128], v [T,HV,128] in the activation dtype (act_dtype: PLA_BF16 or PLA_F16) with token
 *       pitches stride_q/k/v (views into a packed Q|K|V row are fine; q and k rows 4-byte aligned - rows that
 *       are not 16-byte aligned are copied into the workspace first -, v rows 16-byte aligned: v % 16 == 0,
 *       stride_v % 8 == 0); a,b [T,HV] raw gate / beta
 *       logits in the same dtype (pitches stride_a/b) with
 *       A_log, dt_bias [HV] float32:  g = -exp(A_log) softplus(a + dt_bias), beta = sigmoid(b);
 *       or g_in, beta_in [T,HV] float32 (log-decay per token, activated beta) instead.
 *   normalize_qk: L2-normalise q and k (eps 1e-6 inside the root) and round to the activation dtype first.
 *   The matrix products take fp16 operands with FP32 accumulation: magnitudes above 65504 in v, the
 *       state or the intermediate products are outside the supported range.
 *   cu_seqlens [N+1] int32; tokens at and beyond cu_seqlens[N] are padding: their rows of o
 *       are set to zero and they never touch a state.  Empty sequences keep their state.
 *   h0 / ht: k-last FP32 state [slots,HV,128,128] read at h0_indices[n] (or n when the index
 *       array is NULL; zero state when h0 is NULL) and written at ht_indices[n].  h0 == ht with
 *       the same indices updates an indexed pool in place.
 *   o [T,HV,128] activation dtype, dense.   gcum_out / beta_out: optional [T,HV] float32 copies of the
 *       chunk-local cumulative log-decay and of beta (NULL: not written; no kernel reads them back).
 */
int pla_gdn_prefill_launch(
    const void* q, const void* k, const void* v, int64_t stride_q, int64_t stride_k, int64_t stride_v,
    const void* a, const void* b, int64_t stride_a, int64_t stride_b,
    const float* A_log, const float* dt_bias, const float* g_in, const float* beta_in,
    const int32_t* cu_seqlens, int N, int T, float scale, int normalize_qk,
    const float* h0, const int32_t* h0_indices, int64_t h0_slot_stride,
    float* ht, const int32_t* ht_indices, int64_t ht_slot_stride,
    void* o, void* workspace, int64_t workspace_bytes,
    float* gcum_out, float* beta_out,
    int H, int HV, int K, int V, int act_dtype, void* stream);

/*
 * pla_gdn_prefill_launch with the sequence offsets on the host as well: raw_cu_seqlens points to N + 1 int32
 * values in HOST memory that equal cu_seqlens (NULL: exactly pla_gdn_prefill_launch).  Replaces the
 * `raw_cu_seqlens` argument of the reference's public ops (pla/prefill/flashqla/ops.py: "trusted host copy of
 * cu_seqlens", which lets its planner decide without reading the device tensor back).  Here the host takes two
 * decisions from it, neither of which changes a bit of the results (they equal pla_gdn_prefill_launch's): by the rule
 * the device applies anyway, a call whose sequences are of nearly equal length runs in one stage, and with the offsets
 * at hand nothing is enqueued for a second one (two launches and four event operations less per call); and a call of
 * at most 64 ragged whole sequences with more than 128 chains sweeps the chains of its longest sequences as two
 * workgroups of 64 V columns each where idle CUs make that shorter (pla_gdn_prefill_halved_sequences) and, with
 * more chains than CUs, starts its chains longest first.  The values are read during the call and not kept.
 */
int pla_gdn_prefill_launch_raw(
    const void* q, const void* k, const void* v, int64_t stride_q, int64_t stride_k, int64_t stride_v,
    const void* a, const void* b, int64_t stride_a, int64_t stride_b,
    const float* A_log, const float* dt_bias, const float* g_in, const float* beta_in,
    const int32_t* cu_seqlens, int N, int T, float scale, int normalize_qk,
    const float* h0, const int32_t* h0_indices, int64_t h0_slot_stride,
    float* ht, const int32_t* ht_indices, int64_t ht_slot_stride,
    void* o, void* workspace, int64_t workspace_bytes,
    float* gcum_out, float* beta_out,
    int H, int HV, int K, int V, int act_dtype, void* stream, const int32_t* raw_cu_seqlens);

/*
 * The number of sequences whose chains pla_gdn_prefill_launch_raw would sweep as two workgroups each in its last
 * sweep, for these host offsets (0: none, or the call is not one of ragged whole sequences).  Host arithmetic only:
 * no GPU call.  No counterpart in the reference (its planner, pla/prefill/flashqla/private, decides on context-parallel
 * splits instead); for tests and for callers who log the plan.
 */
int pla_gdn_prefill_halved_sequences(const int32_t* raw_cu_seqlens, int N, int T, int H, int HV);

/*
 * pla_gdn_prefill_launch for callers that cannot allocate (code under hipGraph capture, tight serving
 * loops, harnesses that forbid hipMalloc): same arguments without the workspace pair, same results bit
 * for bit.  No counterpart in the reference.  The workspace is an array inside the library, one per GPU
 * (PLA_GDN_PREFILL_STATIC_BYTES, held until the process ends); the call allocates nothing, creates no
 * stream or event, and runs every kernel on `stream`.  Accepted: every shape whose
 * pla_gdn_prefill_workspace_bytes(T, N, H, HV) is within PLA_GDN_PREFILL_STATIC_BYTES (about 2 000 to
 * 3 300 tokens at H = 16, HV = 32, depending on the number of sequences); larger calls are rejected before any launch.  All calls on one GPU share that
 * GPU's array: calls that overlap in time on one GPU (two streams, two threads) race and must be
 * serialised by the caller.
 */
#define PLA_GDN_PREFILL_STATIC_BYTES (64ll << 20)
int pla_gdn_prefill_launch_static(
    const void* q, const void* k, const void* v, int64_t stride_q, int64_t stride_k, int64_t stride_v,
    const void* a, const void* b, int64_t stride_a, int64_t stride_b,
    const float* A_log, const float* dt_bias, const float* g_in, const float* beta_in,
    const int32_t* cu_seqlens, int N, int T, float scale, int normalize_qk,
    const float* h0, const int32_t* h0_indices, int64_t h0_slot_stride,
    float* ht, const int32_t* ht_indices, int64_t ht_slot_stride,
    void* o, float* gcum_out, float* beta_out,
    int H, int HV, int K, int V, int act_dtype, void* stream);

/* Workspace bytes (256-byte aligned) needed by pla_kda_prefill_launch. */
int64_t pla_kda_prefill_workspace_bytes(int T, int N, int H);

/*
 * KDA chunk-64 prefill over packed variable-length sequences (per-channel lower-bound gate).
 * Replaces _C.flashkda_fwd (pla/prefill/flashkdapro/ops.py:215-219) and the tc01 FLA stage
 * launchers fla_runtime::Launchers (src/prefill/flashkdapro/tc01/fla/launchers.h:38-78).
 *
 *   q,k,v,g [T,H,128] bf16 (token pitches stride_*; heads and channels contiguous), g the RAW gate;
 *   beta [T,H] bf16 raw logits (token pitch stride_beta); A_log [H], dt_bias [H*128] float32:
 *       log-decay = lower_bound * sigmoid(exp(A_log) * (g + dt_bias)),  beta = sigmoid(beta).
 *   q and k are L2-normalised (eps 1e-6 inside the root) and rounded to bf16 first.
 *   cu_seqlens [N+1] int32; rows of o at and beyond cu_seqlens[N] are zeroed.
 *   h0 / ht as in pla_gdn_prefill_launch (k-last FP32 [slots,H,128,128]).
 */
int pla_kda_prefill_launch(
    const void* q, const void* k, const void* v, const void* g, const void* beta,
    int64_t stride_q, int64_t stride_k, int64_t stride_v, int64_t stride_g, int64_t stride_beta,
    const float* A_log, const float* dt_bias, float lower_bound, float scale,
    const int32_t* cu_seqlens, int N, int T,
    const float* h0, const int32_t* h0_indices, int64_t h0_slot_stride,
    float* ht, const int32_t* ht_indices, int64_t ht_slot_stride,
    void* o, void* workspace, int64_t workspace_bytes,
    int H, int K, int V, int act_dtype, void* stream);

/*
 * pla_kda_prefill_launch with the sequence offsets on the host as well (N + 1 int32 values in HOST memory that
 * equal cu_seqlens; NULL: exactly pla_kda_prefill_launch).  Replaces the `raw_cu_seqlens` argument of the reference's
 * flashkda_fwd (pla/prefill/flashkdapro/ops.py: the trusted host copy of the offsets).  One host-side decision is
 * taken from it and changes no bit of the results: a call of at most 64 ragged whole sequences with more than 128
 * chains sweeps the chains of its longest sequences as two workgroups of 64 V columns each where idle CUs make that
 * shorter (pla_kda_prefill_halved_sequences tells how many) and, with more chains than CUs, starts its chains longest
 * first.  The values are read during the call and not kept.
 */
int pla_kda_prefill_launch_raw(
    const void* q, const void* k, const void* v, const void* g, const void* beta,
    int64_t stride_q, int64_t stride_k, int64_t stride_v, int64_t stride_g, int64_t stride_beta,
    const float* A_log, const float* dt_bias, float lower_bound, float scale,
    const int32_t* cu_seqlens, int N, int T,
    const float* h0, const int32_t* h0_indices, int64_t h0_slot_stride,
    float* ht, const int32_t* ht_indices, int64_t ht_slot_stride,
    void* o, void* workspace, int64_t workspace_bytes,
    int H, int K, int V, int act_dtype, void* stream, const int32_t* raw_cu_seqlens);

/* As pla_gdn_prefill_halved_sequences, for pla_kda_prefill_launch_raw.  Host arithmetic only. */
int pla_kda_prefill_halved_sequences(const int32_t* raw_cu_seqlens, int N, int T, int H);

/*
 * Rows of the 128-row state tile a wavefront owns (8, 16 or 32) that a k-last launch with
 * rows_per_wave = 0 takes for a shape: the row count the auto-tuner measured for the nearest batch size
 * of the same (kernel, heads, dtypes) if the built-in table holds the shape, else the size thresholds.
 * The table is compiled in from pla_amd/lut/ (the reference compiles its dispatch from
 * lut/tuned_result_<device>.csv: scripts/decode/generate_kernel_instantiations.py; tuner
 * scripts/decode/auto_tune.py).  kernel: 0 = k_last, 1 = k_last_packed, 2 = k_last_mtp; tree: 1 for the
 * eagle-tree mode; dtypes are PLA_* codes.  Host only, no GPU call.  Returns 0 for invalid arguments.
 */
int pla_tuned_rows_per_wave(int kernel, int tree, int act_dtype, int state_dtype, int H, int HV, int B);

#ifdef __cplusplus
}
#endif
#endif /* PLA_GFX950_H */
