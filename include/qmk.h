/*
 * qmk.h — C ABI of the gfx950 decode megakernel library (libqmk_hip.so).
 *
 * The library is the drop-in for the reference's per-route pybind module: one
 * launch executes a host-built instruction tensor (32 int32 words per
 * instruction, one queue per workgroup) over the caller's weight, KV-cache and
 * scratch tensors.  All pointers are raw DEVICE pointers owned by the caller;
 * the library allocates nothing, keeps no reference after the call returns and
 * launches asynchronously on the stream it is given.
 *
 * Reference interfaces each entry point stands in for (paths under
 * qimeng_megakernel/models/LLM/llama/llama3_2__1b/A100/single_batch/):
 *   qmk_decode_step   <- void mk(22 x const torch::Tensor&, int pos_id,
 *                        float attn_scale, float rms_norm_eps)
 *                        decode_kernel/mk.h:4-30, launcher decode_kernel/mk.cu:97-198,
 *                        python binding decode_kernel/pybind.cpp:8-39,
 *                        call site decode_schedule/mk_kernel.py:56-94
 *   qmk_decode_step_batch <- void mk(22 x const torch::Tensor&, int pos_id, int batch_size,
 *                        float attn_scale, float rms_norm_eps, optional position_ids, active_mask,
 *                        attn_partial_valid, attn_rms_out, mlp_rms_out, lm_head_rms_out) of the batch route:
 *                        …/A100/multi_batch/decode_kernel/mk.h:9-42, host checks mk.cu:52-216,
 *                        call site …/multi_batch/decode_schedule/mk_kernel.py:56-111
 *   qmk_query         <- KernelConfig (NUM_SMS, NUM_THREADS, SHARED_MEMORY_SIZE,
 *                        INSTRUCTION_WIDTH) decode_kernel/kernel_config.cuh:6-14
 *   qmk_status_*      <- the reference only printf()s launch errors
 *                        (decode_kernel/mk.cu:185-197) and traps on bad opcodes
 *                        (mk.cu:82-90); here both become return codes.
 */
#ifndef QMK_H_
#define QMK_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define QMK_ABI_VERSION 8
#define QMK_INSTRUCTION_WORDS 32

/* Return / status codes. 0 is success; everything else is an error. */
enum {
  QMK_OK = 0,
  QMK_ERR_NULL_ARG = 1,        /* args or a required pointer is NULL            */
  QMK_ERR_ABI = 2,             /* args->struct_size does not match this library */
  QMK_ERR_SHAPE = 3,           /* a dimension is out of the supported range     */
  QMK_ERR_POSITION = 4,        /* pos_id outside the KV cache / RoPE table      */
  QMK_ERR_TOO_MANY_QUEUES = 5, /* more queues than co-resident workgroups       */
  QMK_ERR_NO_DEVICE = 6,       /* no gfx950 device / HIP runtime error          */
  QMK_ERR_LAUNCH = 7,          /* hipLaunchKernel failed                        */
  QMK_ERR_MODEL = 8,           /* unknown model id                              */
  QMK_ERR_SCRATCH = 9,         /* qmk_decode_step_static: the launch needs more than the
                                  library's static scratch array holds          */
  /* device-side (reported through qmk_status_fetch) */
  QMK_DEV_BAD_OPCODE = 32,     /* opcode outside 0..7 (batch route: 0..10)      */
  QMK_DEV_BAD_OPERAND = 33,    /* an operand would index out of bounds          */
  QMK_DEV_WAIT_TIMEOUT = 34    /* a counter never reached its expected value    */
};

/* Model shapes compiled into the library. */
enum {
  QMK_MODEL_LLAMA_3_2_1B = 0,  /* H 2048, F 8192, 32 q / 8 kv heads, d 64 */
  QMK_MODEL_QWEN1_5_MOE_A2_7B = 2, /* H 2048, 16 q / 16 kv heads, d 128, QKV bias; the MoE op set
                                  (…/qwen/qwen1_5_moe_a2_7b/A100/single_batch/decode_kernel/mk.h); expert
                                  count, top-k and FFN widths are launch parameters (qmk_decode_step_moe) */
  QMK_MODEL_QWEN3_1_7B = 1,    /* H 2048, F 6144, 16 q / 8 kv heads, d 128, per-head QK RMSNorm
                                  (the Qwen3 op set: …/qwen/qwen3__0_6b/A100/single_batch/
                                  decode_kernel/mk.h, decode_schedule/mk_kernel.py:52-110)     */
  QMK_MODEL_QWEN3_30B_A3B = 3  /* H 2048, 32 q / 4 kv heads, d 128 (attention output 4096 wide), per-head QK
                                  RMSNorm, no QKV bias: the Qwen3 op set's attention in front of the MoE op
                                  set (qmk_decode_step_moe), without a shared expert and with renormalised
                                  top-k weights (norm_topk_prob: …/qwen1_5_moe_a2_7b/A100/single_batch/
                                  decode_schedule/fused/operations.py:405).  The reference has no route
                                  for this shape: it is its two routes put together                  */
};

/* qmk_query selectors. */
enum {
  QMK_QUERY_ABI_VERSION = 0,
  QMK_QUERY_CU_COUNT = 1,          /* compute units of the current device        */
  QMK_QUERY_THREADS = 2,           /* threads per workgroup                      */
  QMK_QUERY_LDS_BYTES = 3,         /* static LDS per workgroup                   */
  QMK_QUERY_MAX_QUEUES = 4,        /* largest co-resident grid on this device    */
  QMK_QUERY_INSTRUCTION_WORDS = 5,
  QMK_QUERY_MAX_PARTIALS = 6       /* largest split-KV fan-out the kernel merges */
};

/* Rows of `barriers` per layer that QMK_FLAG_XCD_COUNTERS needs (with 48 slots). */
#define QMK_XCD_COUNTER_ROWS 54

/* Flags. */
#define QMK_FLAG_TAGGED 4u         /* the vectors that every workgroup hands to others inside a
                                      launch (q and the appended K/V row, the residual stream after
                                      the O-proj and after the down projection, silu_out) also travel through
                                      `workspace` as 8-byte units {32-bit payload, 32-bit tag}, the
                                      tag naming launch and layer.  A consumer polls the units it
                                      needs until they carry the tag it expects, and the producer
                                      neither waits for its stores to be acknowledged nor counts an
                                      arrival: one memory round trip per hand-over instead of four.
                                      Needs `workspace` (qmk_workspace_bytes), at most 63 layers and
                                      a schedule whose down projection is not split along K; not
                                      combinable with QMK_FLAG_KEEP_BARRIERS.  The caller's buffers
                                      receive the same values as without the flag; counter rows 0,
                                      3, 4 and 5 carry no count.  (The split-KV partials stay on
                                      counters.  Where the O-projection merges them itself, the
                                      model has at most 8 KV heads, QMK_FLAG_XCD_COUNTERS is not
                                      set and rows 2..5 hold 256 words, their arrivals go to eight
                                      128-byte lines from word 0 of row 2 on, every arrival to all
                                      eight, and an O-projection workgroup polls the line of its
                                      own XCD: rows 3.. are then written in part.)                */
#define QMK_FLAG_KEEP_BARRIERS 1u  /* leave the final counter values in `barriers`
                                      (the reference's behaviour); by default the
                                      last workgroup to retire clears them so the
                                      host needs no barriers.zero_() per step.   */
#define QMK_FLAG_XCD_COUNTERS 2u   /* the all-to-all edges of a layer (attention -> O-proj when the
                                      O-proj merges the partials itself, O-proj -> up/gate,
                                      up/gate -> down, down -> next QKV / LM head) count
                                      arrivals on eight sub-counters, one 128-byte line per
                                      XCD, kept in rows 10.. of each layer of `barriers`;
                                      consumers poll the eight lines and sum them (the attention
                                      edge: every arrival goes to all eight lines and a consumer
                                      polls the line of its own XCD).  Needs
                                      num_layer_barriers * barrier_slots >= 10 * barrier_slots
                                      + 2048 ints (32 counter lines, then 32 flag lines), a 128-byte aligned `barriers` with a layer
                                      stride that is a multiple of 128 bytes, and a schedule
                                      that does not split the down projection along K.  Rows
                                      2..5 of the reference protocol stay zero in this mode. */

/*
 * One decode step.  Tensor order and meaning follow mk(...) of the reference
 * (decode_kernel/mk.h:4-30).  "bf16" is the raw 16-bit pattern.
 */
typedef struct QmkArgs {
  uint32_t struct_size;            /* = sizeof(QmkArgs)                           */
  uint32_t model;                  /* QMK_MODEL_*                                 */
  uint32_t flags;                  /* QMK_FLAG_*                                  */
  uint32_t spin_limit;             /* counter polls before QMK_DEV_WAIT_TIMEOUT; 0 = default */

  const int32_t* instructions;     /* int32 [num_queues, num_insts, 32]           */
  void* hidden_states;             /* bf16 [H]            in/out residual stream  */
  void* q_post_rope;               /* bf16 [Hq*D]                                 */
  void* k_cache;                   /* bf16 [L, 1, max_seq_len, Hkv, D]            */
  void* v_cache;                   /* bf16 [L, 1, max_seq_len, Hkv, D]            */
  void* attn_out;                  /* bf16 [Hq*D]                                 */
  float* attn_lse_intermediates;   /* f32  [Hq, max_splits]      log2 domain      */
  float* attn_out_intermediates;   /* f32  [Hq, max_splits, D]                    */
  void* silu_out;                  /* bf16 [F]                                    */
  void* logits;                    /* bf16 [vocab_size]                           */
  const void* attn_norm_weights;   /* bf16 [L, H]                                 */
  const void* qkv_weights;         /* bf16 [L, (Hq+2Hkv)*D, H]                    */
  const float* rope_cos;           /* f32  [rope_rows, D]  pair-interleaved       */
  const float* rope_sin;           /* f32  [rope_rows, D]                         */
  const void* o_proj_weights;      /* bf16 [L, H, H]                              */
  const void* mlp_norm_weights;    /* bf16 [L, H]                                 */
  const void* up_proj_weights;     /* bf16 [L, F, H]                              */
  const void* gate_proj_weights;   /* bf16 [L, F, H]                              */
  const void* down_proj_weights;   /* bf16 [L, H, F]                              */
  const void* lm_head_norm_weights;/* bf16 [H]                                    */
  const void* lm_head_weights;     /* bf16 [vocab_size, H]                        */
  int32_t* barriers;               /* int32 [num_layers, num_layer_barriers, barrier_slots] */

  int32_t num_queues;              /* instructions.size(0) = workgroups launched  */
  int32_t num_insts;               /* instructions.size(1)                        */
  int32_t num_layers;              /* barriers.size(0)                            */
  int32_t num_layer_barriers;      /* barriers.size(1)  (>= 8)                    */
  int32_t barrier_slots;           /* barriers.size(2)  (>= Hq + 2*Hkv)           */
  int32_t max_seq_len;             /* k_cache.size(2)                             */
  int32_t max_splits;              /* attn_lse_intermediates.size(1)              */
  int32_t vocab_size;              /* logits.size(0)                              */
  int32_t rope_rows;               /* rope_cos.size(0)                            */
  int32_t pos_id;                  /* index of the token being decoded            */
  float attn_scale;                /* 1/sqrt(D)                                   */
  float rms_norm_eps;

  /* Final counter values implied by the scheduler's tile geometry.  0 selects
   * the reference's (16-row tiles, 2048-wide K slices): 4, 128, 128, 512.       */
  int32_t qkv_blocks_per_head;     /* D / qkv_tile_n                              */
  int32_t oproj_blocks;            /* H / oproj_tile_n                            */
  int32_t upgate_blocks_per_bucket;/* split_k / upgate_tile_n                     */
  int32_t down_arrivals;           /* (H / down_tile_n) * (F / split_k)           */

  uint64_t* timeline;              /* optional u64 [num_queues, num_insts, 8] device
                                      buffer, per instruction: start, after-wait, end
                                      (100 MHz ticks), opcode | layer << 8, and four
                                      op-specific intermediate stamps; NULL = off */
  void* stream;                    /* hipStream_t; NULL = the null stream         */
  void* workspace;                 /* QMK_FLAG_TAGGED and/or token_out: device buffer of
                                      workspace_bytes, 128-byte aligned, zeroed once when allocated
                                      and then left to the library (it carries a launch count from
                                      step to step); NULL otherwise                              */
  uint64_t workspace_bytes;        /* >= qmk_workspace_bytes(model)               */

  /* Greedy step chaining on the device (both NULL = off, the reference's behaviour, where the host
   * runs argmax and the embedding lookup between launches: models/LLM/decode.py:1386-1397).  With
   * both set, the last workgroup to retire writes the index of the first maximal bf16 logit to
   * *token_out and copies that token's embedding row into hidden_states, so the next step can be
   * launched without any host work in between.  Needs `workspace`, at most 1024 queues, and is not
   * combinable with QMK_FLAG_KEEP_BARRIERS. */
  const void* embed_tokens;        /* bf16 [vocab_size, H]                        */
  int64_t* token_out;              /* one element                                 */

  /* Qwen3 op set only (NULL for the Llama shape): the three tensors its mk(...) takes in addition. */
  void* qkv_raw;                   /* bf16 [(Hq+2Hkv)*D]  QKV before norm and RoPE */
  const void* q_norm_weights;      /* bf16 [L, D]  per-head RMSNorm of q, pair-interleaved like the q rows */
  const void* k_norm_weights;      /* bf16 [L, D]                                 */
} QmkArgs;

/* Launch one decode step asynchronously on args->stream.  Returns QMK_OK or a
 * host-side QMK_ERR_*.  Device-side errors surface through qmk_status_fetch. */
int qmk_decode_step(const QmkArgs* args);

/*
 * qmk_decode_step without any allocation on the caller's side or the library's: no counterpart in
 * the reference.  It is for callers that cannot allocate device memory -- code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  Everything is as in
 * qmk_decode_step (same struct, same kernels, same results bit for bit), except that
 * args->workspace and args->workspace_bytes are ignored: the tagged units, the greedy candidates
 * and the launch count live in a static device array of the library (94 208 bytes per GPU, held
 * until the process ends; its address is looked up once per device on the first call of any entry
 * point there).  Limits of that array: at most 1024 queues when token_out is set and at most 63
 * layers with QMK_FLAG_TAGGED -- beyond them the call returns QMK_ERR_SCRATCH and launches nothing.
 * All calls on one GPU share the array, which keeps the previous call's contents: the launch count
 * carries on from call to call (stale units never carry a current tag; candidates are rewritten by
 * every queue of a launch before they are read), and qmk_status_fetch clears the array when it
 * reports a device-side error.  Calls that overlap on one GPU (two streams) race on it: serialise
 * them, or use qmk_decode_step with one workspace per stream.
 * Under HIP graph capture: the first call of any entry point on a device looks the device up (occupancy
 * queries, hipGetSymbolAddress, a blocking clear of the status words), none of which may be captured, so
 * call qmk_query(QMK_QUERY_MAX_QUEUES) once per device before the capture begins; from then on a call
 * is one kernel launch and nothing else.
 */
int qmk_decode_step_static(const QmkArgs* args);

/*
 * One decode step of the batch route: 2..16 rows decoded together (1 is accepted), each at its own
 * position.  Ten opcodes (…/multi_batch/decode_schedule/instructions/instruction_defs.py:11-211):
 * RMSNorm rows 1/6/9, GEMMs 2/5/7/8/10 over 16-row blocks on the matrix cores, split-KV attention 3 and
 * its reduction 4 per batch row.  Tensors are the batch-1 ones with a leading batch dimension, in the
 * order of mk(...) (…/multi_batch/decode_kernel/mk.h:9-42).  Two layer geometries are compiled for this
 * route: Llama-3.2-1B, and Qwen3-1.7B with the Qwen3 op set (opcode 2 leaves the raw QKV rows, opcode 3
 * applies the per-head RMSNorm and RoPE to its row's q and k and appends the cache row).
 * Flags: QMK_FLAG_KEEP_BARRIERS, and QMK_FLAG_XCD_COUNTERS in this route's form: the blocks of the
 * O-projection, the up/gate and the down projection (counter rows 4, 6, 7) are counted on words 0, 32 .. 224 of
 * their row (the sender's workgroup index modulo 8 chooses: one 128-byte line per XCD) instead of all on word 0, and
 * the instructions that wait for them add the eight words up; a norm row (counter rows 0, 5, 8) arrives on all eight
 * of those words of its row and a waiting workgroup polls the one of its own XCD; the head counters of row 1 and the
 * row counters of row 3 move a line apart (word i -> 32 (i % 8) + i / 8).  Needs barrier_slots >= 256.  Hundreds of
 * arrivals from eight XCDs on one line are seen 2 us later than on eight.  No counterpart in the reference.
 */
typedef struct QmkBatchArgs {
  uint32_t struct_size;            /* = sizeof(QmkBatchArgs)                      */
  uint32_t model;                  /* QMK_MODEL_LLAMA_3_2_1B or QMK_MODEL_QWEN3_1_7B */
  uint32_t flags;                  /* QMK_FLAG_KEEP_BARRIERS, QMK_FLAG_XCD_COUNTERS */
  uint32_t spin_limit;             /* counter polls before QMK_DEV_WAIT_TIMEOUT; 0 = default */

  const int32_t* instructions;     /* int32 [num_queues, num_insts, 32]           */
  void* hidden_states;             /* bf16 [B, H]         in/out residual stream  */
  void* q_post_rope;               /* bf16 [B, Hq*D]                              */
  void* k_cache;                   /* bf16 [L, B, max_seq_len, Hkv, D]            */
  void* v_cache;                   /* bf16 [L, B, max_seq_len, Hkv, D]            */
  void* attn_out;                  /* bf16 [B, Hq*D]                              */
  float* attn_lse_intermediates;   /* f32  [B, Hq, max_splits]   log2 domain      */
  float* attn_out_intermediates;   /* f32  [B, Hq, max_splits, D]                 */
  void* silu_out;                  /* bf16 [B, F]                                 */
  void* logits;                    /* bf16 [B, vocab_size]                        */
  const void* attn_norm_weights;   /* bf16 [L, H]                                 */
  const void* qkv_weights;         /* bf16 [L, (Hq+2Hkv)*D, H]                    */
  const float* rope_cos;           /* f32  [rope_rows, D]  pair-interleaved       */
  const float* rope_sin;           /* f32  [rope_rows, D]                         */
  const void* o_proj_weights;      /* bf16 [L, H, H]                              */
  const void* mlp_norm_weights;    /* bf16 [L, H]                                 */
  const void* up_proj_weights;     /* bf16 [L, F, H]                              */
  const void* gate_proj_weights;   /* bf16 [L, F, H]                              */
  const void* down_proj_weights;   /* bf16 [L, H, F]                              */
  const void* lm_head_norm_weights;/* bf16 [H]                                    */
  const void* lm_head_weights;     /* bf16 [vocab_size, H]                        */
  int32_t* barriers;               /* int32 [num_layers, num_layer_barriers (>= 10), barrier_slots (>= B*(Hq+2Hkv))] */

  int32_t num_queues;              /* instructions.size(0) = workgroups launched  */
  int32_t num_insts;               /* instructions.size(1)                        */
  int32_t num_layers;
  int32_t num_layer_barriers;
  int32_t barrier_slots;
  int32_t max_seq_len;             /* k_cache.size(2)                             */
  int32_t max_splits;              /* attn_lse_intermediates.size(2)              */
  int32_t vocab_size;              /* logits.size(1)                              */
  int32_t rope_rows;
  int32_t pos_id;                  /* position of every row when position_ids is NULL */
  int32_t batch_size;              /* B, 1..16                                    */
  int32_t kv_block_size;           /* tokens per split-KV block (the scheduler's attn_kv_block_size) */
  int32_t oproj_blocks;            /* final value of the O-proj counter = H / rows per O-proj block; 0 = H/16 */
  int32_t down_blocks;             /* ... of the down-projection counter; 0 = H/16.  Blocks of 16 rows are
                                      the reference's; this library also takes 8 (word tile_N_granularity
                                      of opcodes 5 and 8), which gives each of 256 workgroups one block */
  float attn_scale;
  float rms_norm_eps;

  const int32_t* position_ids;     /* int32 [B] or NULL                           */
  const uint8_t* active_mask;      /* u8/bool [B] or NULL: every row is active    */
  uint8_t* attn_partial_valid;     /* u8/bool [B, Hq, max_splits] or NULL         */
  void* attn_rms_out;              /* bf16 [B, H]  RMSNorm rows for the QKV GEMM  */
  void* mlp_rms_out;               /* bf16 [B, H]  ... for the up/gate GEMM       */
  void* lm_head_rms_out;           /* bf16 [B, H]  ... for the LM head            */

  uint64_t* timeline;              /* as in QmkArgs; NULL = off                   */
  void* stream;                    /* hipStream_t; NULL = the null stream         */

  /* Qwen3 op set only (QMK_MODEL_QWEN3_1_7B; NULL otherwise): as in QmkArgs, with a leading batch dimension
   * (…/qwen/qwen3__0_6b/A100/single_batch/decode_schedule/fused/operations.py:52-120 run per row). */
  void* qkv_raw;                   /* bf16 [B, (Hq+2Hkv)*D]  QKV before the per-head norm and RoPE */
  const void* q_norm_weights;      /* bf16 [L, D]  pair-interleaved like the q rows of qkv_weights */
  const void* k_norm_weights;      /* bf16 [L, D]                                 */

  /* Column window (…/multi_batch/decode_kernel/mk.h:44-115: mk_step runs the one column inst_idx of the instruction
   * tensor per launch, mk_step_loop all columns one launch after the other): the launch runs the columns
   * [first_inst, first_inst + inst_count) of `instructions`; inst_count = 0 runs all of them (first_inst must then
   * be 0).  A window that is not the whole tensor needs QMK_FLAG_KEEP_BARRIERS: the counters carry the step from one
   * launch to the next and the caller zeroes them before the first column, as the reference's callers do. */
  int32_t first_inst;
  int32_t inst_count;
} QmkBatchArgs;

/* Launch one step of the batch route asynchronously on args->stream.  Positions outside the KV
 * cache or the RoPE table are found on the device (QMK_DEV_BAD_OPERAND, instruction -1). */
int qmk_decode_step_batch(const QmkBatchArgs* args);

/*
 * One decode step of 1..4 requests ("rows") on the batch-1 kernel's row-streaming engine, for the batch sizes at which
 * the matrix-core tiles of qmk_decode_step_batch are mostly empty.  Same buffers as qmk_decode_step_batch (`step` is a
 * QmkBatchArgs: [B, ...] activations, KV cache [L, B, S, Hkv, D], position_ids, active_mask; its three RMSNorm row
 * buffers, attn_partial_valid, kv_block_size, oproj_blocks and down_blocks are not used, step.flags must be 0), but the
 * instruction stream is the BATCH-1 route's (…/single_batch/decode_schedule/instructions/instruction_defs.py:39-177):
 * opcodes 1, 4, 5, 6, 7 act on all rows at once — every weight row is streamed once and multiplied with every row's
 * activation vector — and opcode 2 names its row in the word behind its batch-1 operands (word 6).  The reference's batch
 * route (…/multi_batch/decode_kernel/mk.h:9-42) has no counterpart of this stream; a step is the batch-1 route run for
 * every active row, whose results it reproduces bit for bit.  Hand-over is the tagged one (one set of units per row in
 * `workspace`, qmk_rows_workspace_bytes(B) bytes, 128-byte aligned, zeroed once); the split-KV partials of a (row, KV
 * head) are merged by the group's last arrival (merge word 1, O-projection word 5 = 0; the row's count of merged heads
 * is kept on eight 128-byte lines at the end of the row's workspace, one per XCD, which the launch that retires clears)
 * or by every O-projection workgroup (merge word 2, word 5 = fan-out).  A row whose active flag is off is left alone;
 * its logits are set to -1e9.  After a device-side error the caller zeroes `workspace` and `barriers`.
 */
typedef struct QmkRowsArgs {
  uint32_t struct_size;            /* = sizeof(QmkRowsArgs)                       */
  int32_t qkv_blocks_per_head;     /* final value of a head's QKV counter = D / rows per QKV tile; 0 = D/16 */
  void* workspace;
  uint64_t workspace_bytes;
  QmkBatchArgs step;               /* step.struct_size = sizeof(QmkBatchArgs); batch_size 1..4 */
} QmkRowsArgs;

int qmk_decode_step_rows(const QmkRowsArgs* args);

/* Size of QmkRowsArgs.workspace; 0 when batch_size is out of range. */
uint64_t qmk_rows_workspace_bytes(int batch_size);

/*
 * One decode step of the MoE route at batch 1: opcodes 1-4 and 7 of the dense route (QKV with bias) and
 * 8-14 (…/qwen1_5_moe_a2_7b/A100/single_batch/decode_schedule/instructions/instruction_defs.py:24-151):
 * router logits, softmax top-k, shared expert up/gate and K-split down, routed experts up/gate and down,
 * combine + commit.  Tensors as in mk(...) of that route (decode_schedule/mk_kernel.py:95-205); its three
 * unused dense-MLP positions have no field here.  Counters [L, >= 15, >= 128].
 */
typedef struct QmkMoeArgs {
  uint32_t struct_size;            /* = sizeof(QmkMoeArgs)                        */
  uint32_t model;                  /* QMK_MODEL_QWEN1_5_MOE_A2_7B or QMK_MODEL_QWEN3_30B_A3B */
  uint32_t flags;                  /* QMK_FLAG_KEEP_BARRIERS, QMK_FLAG_TAGGED (whole steps, not with KEEP_BARRIERS) */
  uint32_t spin_limit;

  const int32_t* instructions;     /* int32 [num_queues, num_insts, 32]           */
  void* hidden_states;             /* bf16 [H]            in/out residual stream  */
  void* normed_hidden_states;      /* bf16 [H]   RMSNorm row published by opcode 8 */
  void* q_post_rope;               /* bf16 [Hq*D]                                 */
  void* k_cache;                   /* bf16 [L, 1, max_seq_len, Hkv, D]            */
  void* v_cache;
  void* attn_out;                  /* bf16 [Hq*D]                                 */
  float* attn_lse_intermediates;   /* f32  [Hq, max_splits]                       */
  float* attn_out_intermediates;   /* f32  [Hq, max_splits, D]                    */
  void* silu_out;                  /* bf16 [Fm]  what the last expert slot wrote  */
  void* logits;                    /* bf16 [vocab_size]                           */
  const void* attn_norm_weights;   /* bf16 [L, H]                                 */
  const void* qkv_weights;         /* bf16 [L, (Hq+2Hkv)*D, H]                    */
  const void* qkv_bias;            /* bf16 [L, (Hq+2Hkv)*D]; NULL for QMK_MODEL_QWEN3_30B_A3B */
  const float* rope_cos;           /* f32  [rope_rows, D]                         */
  const float* rope_sin;
  const void* o_proj_weights;      /* bf16 [L, H, Hq*D]                           */
  const void* mlp_norm_weights;    /* bf16 [L, H]                                 */
  const void* lm_head_norm_weights;/* bf16 [H]                                    */
  const void* lm_head_weights;     /* bf16 [vocab_size, H]                        */
  const void* router_weights;      /* bf16 [L, E, H]                              */
  float* router_logits_buf;        /* f32  [E]                                    */
  int64_t* expert_indices;         /* i64  [top_k]                                */
  float* expert_weights;           /* f32  [top_k]                                */
  /* the six shared-expert tensors: NULL for a model without a shared expert (shared_ffn = 0) */
  const void* shared_expert_gate_proj_weights; /* bf16 [L, Fs, H]                 */
  const void* shared_expert_up_proj_weights;   /* bf16 [L, Fs, H]                 */
  const void* shared_expert_down_proj_weights; /* bf16 [L, H, Fs]                 */
  void* shared_expert_silu_out;    /* bf16 [Fs]                                   */
  void* shared_out;                /* bf16 [H]                                    */
  const void* shared_expert_gate_weights;      /* bf16 [L, H]  the sigmoid gate   */
  const void* expert_gate_up_proj_weights;     /* bf16 [L, E, 2*Fm, H], gate rows first */
  const void* expert_down_proj_weights;        /* bf16 [L, E, H, Fm]              */
  void* routed_silu_buffer;        /* bf16 [top_k, Fm]                            */
  float* routed_out_f32;           /* f32  [H]   left cleared, as by the reference */
  void* routed_out;                /* bf16 [H]   unused by opcodes 8-14 (may be NULL) */
  int32_t* barriers;               /* int32 [num_layers, num_layer_barriers, barrier_slots] */

  int32_t num_queues;
  int32_t num_insts;
  int32_t num_layers;
  int32_t num_layer_barriers;      /* >= 15                                       */
  int32_t barrier_slots;           /* >= H/16 and >= Hq + 2 Hkv                   */
  int32_t max_seq_len;
  int32_t max_splits;
  int32_t vocab_size;
  int32_t rope_rows;
  int32_t pos_id;
  int32_t num_experts;             /* E, <= 512                                   */
  int32_t top_k;                   /* experts per token, <= 8                     */
  int32_t shared_ffn;              /* Fs, a multiple of 16; 0 = no shared expert: the stream then holds no opcodes 10/11
                                      and opcode 14 adds the routed experts only                                   */
  int32_t moe_ffn;                 /* Fm, a multiple of 16, <= 2048               */
  int32_t shared_k_slices;         /* K slices of the shared down projection (4 in the reference); 0 with shared_ffn = 0 */
  float attn_scale;
  float rms_norm_eps;

  uint64_t* timeline;
  void* stream;
  void* workspace;                 /* qmk_moe_workspace_bytes(top_k, shared_k_slices) bytes, 128-byte aligned: the
                                      terms of the two in-place accumulations of the reference (shared_out over
                                      the K slices, routed_out_f32 over the expert slots), one slot per producer,
                                      added by opcode 14 in the reference VM's order; the layer's gate scalar; and
                                      the tagged units of QMK_FLAG_TAGGED (zeroed once when allocated, and again
                                      after a launch that reported a device error)                              */
  uint64_t workspace_bytes;

  /* Qwen3 op set only (QMK_MODEL_QWEN3_30B_A3B; NULL otherwise), as in QmkArgs. */
  void* qkv_raw;                   /* bf16 [(Hq+2Hkv)*D]  QKV before norm and RoPE */
  const void* q_norm_weights;      /* bf16 [L, D]                                 */
  const void* k_norm_weights;      /* bf16 [L, D]                                 */
  int32_t norm_topk_prob;          /* 1: opcode 9 divides the top-k probabilities by their sum (fp32, added in slot
                                      order); 0: raw probabilities, as the reference's decode route leaves them   */
  int32_t routed_upgate_tile;      /* outputs per tile of opcode 12 (its tile_N_granularity word): 16 (0 = 16), or 8
                                      where that deals the tiles evenly (Fm = 768: 768 tiles for 256 queues)        */
  int32_t oproj_tile;              /* rows per tile of opcode 4 (its tile_N_granularity word): 16 (0 = 16), or 8, which
                                      gives each of 256 queues one tile of the 2048 rows; fixes the final value of the
                                      O-projection counter (H / oproj_tile)                                          */
  int32_t local_routing;           /* QMK_FLAG_TAGGED only.  0: the routed ops (12, 13) wait for the experts and weights that
                                      opcode 9 announces.  1: they take the routing decision themselves from the router's
                                      logits (the same function of the same values: the same experts and weights), and
                                      opcode 9 only reports it — for streams in which nothing runs beside the router and the
                                      top-k (no shared expert), where that hand-over would leave the whole device waiting;
                                      such a stream may place opcode 9 behind its queue's routed up/gate tiles          */
  int32_t qkv_tile;                /* rows per tile of opcode 1 (its tile_N_granularity word): 16 (0 = 16), or 8, 4 or 2 where
                                      16 deals the tiles unevenly (5120 rows: 320 tiles of 16 leave a quarter of 256 queues
                                      with two, 1280 tiles of 4 give each five); fixes the final value of a head's QKV
                                      counter (D / qkv_tile)                                                          */
  int32_t reserved0;               /* 0 */
} QmkMoeArgs;

int qmk_decode_step_moe(const QmkMoeArgs* args);

/* Size of QmkMoeArgs.workspace; 0 when an argument is out of range. */
uint64_t qmk_moe_workspace_bytes(int top_k, int shared_k_slices);

/*
 * One decode step of the MoE route for 1..4 requests ("rows") in ONE launch.  The reference has no MoE route for
 * batch sizes above one (its batch route, …/llama3_2__1b/A100/multi_batch/decode_kernel/mk.h:9-42, is dense); a step
 * is defined as the batch-1 route above run for every row on that row's own buffers, and every row's results are
 * those of the row decoded alone, bit for bit.  What the launch saves is traffic: attention weights, router and LM
 * head are read once per step, and each expert once for all the rows that picked it.
 *
 * `step` is a QmkMoeArgs in which every per-request buffer carries a leading row dimension — hidden_states [B, H],
 * k_cache [B, L, 1, S, Hkv, D], logits [B, vocab], expert_indices [B, top_k], routed_silu_buffer [B, top_k, Fm], … —
 * so row r's slice is a batch-1 buffer set; the weights, the RoPE tables, `instructions` and `barriers` exist once.
 * step.pos_id is ignored: row r decodes position_ids[r].  Models without a shared expert only (shared_ffn = 0:
 * QMK_MODEL_QWEN3_30B_A3B), QMK_FLAG_TAGGED required, Fm <= 1024, B x (E rounded up to 64) <= 512.
 * step.workspace: qmk_moe_rows_workspace_bytes(B) bytes (one set of tagged units per row), zeroed once.
 *
 * Instruction stream: opcodes 1, 4, 7, 8 as above, each for all rows; 2 and 9 with the row in the word behind
 * their batch-1 operands; and instead of 12/13/14
 *   [15, layer, part, nparts, tile]     gate/up rows of the layer's DISTINCT experts (the rows' picks merged on the
 *                                       device, ascending), dealt over the instruction's waves at run time
 *   [16, layer, n_start, n_end, tile]   down-projection rows [n_start*tile, n_end*tile) of every distinct expert and
 *                                       the commit of those rows for every request (tile 8 or 16, at most 16 rows).
 */
typedef struct QmkMoeRowsArgs {
  uint32_t struct_size;            /* = sizeof(QmkMoeRowsArgs)                    */
  int32_t batch_size;              /* B, 1..4                                     */
  const int32_t* position_ids;     /* int32 [B] on the device                     */
  int32_t* distinct_experts;       /* int32 [num_layers] on the device, or NULL: the number of distinct experts each
                                      layer streamed in this launch (what a step's algorithmic bytes are counted from) */
  QmkMoeArgs step;                 /* step.struct_size = sizeof(QmkMoeArgs)       */
} QmkMoeRowsArgs;

int qmk_decode_step_moe_rows(const QmkMoeRowsArgs* args);

/* Size of QmkMoeRowsArgs.step.workspace; 0 when batch_size is out of range. */
uint64_t qmk_moe_rows_workspace_bytes(int batch_size);

/* Size of QmkArgs.workspace for QMK_FLAG_TAGGED; 0 for an unknown model. */
uint64_t qmk_workspace_bytes(int model);

/* Device/library properties (QMK_QUERY_*); negative on error. */
int qmk_query(int what);

/* Synchronise `stream`, then return and clear the first device-side error the
 * kernels on the current device recorded since the last fetch (QMK_OK if none).
 * detail[0..3], when non-NULL, receive {workgroup, instruction index, opcode,
 * operand/slot}. */
int qmk_status_fetch(void* stream, int32_t detail[4]);

/* Static, human-readable name of a return/status code. */
const char* qmk_error_string(int code);

#ifdef __cplusplus
}
#endif
#endif /* QMK_H_ */
