// Device-side building blocks of the gfx950 decode megakernel: bf16 rounding,
// wave/workgroup reductions, the inter-workgroup counter protocol and the
// row-streaming GEMV primitives.  Wave size is 64 throughout.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "qmk.h"

namespace qmk {

// f(integral_constant<I>), ..., f(integral_constant<N-1>): an unrolled loop whose index is a constant.
template <int I, int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
  if constexpr (I < N) {
    f(std::integral_constant<int, I>{});
    static_for<I + 1, N>(f);
  }
}

constexpr int kThreads = 512;            // one workgroup per CU, 8 waves, 2 per SIMD
constexpr int kWaveSize = 64;
constexpr int kWaves = kThreads / kWaveSize;
constexpr int kInstWords = QMK_INSTRUCTION_WORDS;
constexpr int kMaxPartials = kInstWords - 7;   // reduction list capacity of one slot
constexpr int kMaxSelfMerge = 64;              // split-KV fan-out when every O-proj workgroup merges for itself
constexpr uint32_t kDefaultSpinLimit = 1u << 22;

using u16 = uint16_t;
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef uint32_t v4u __attribute__((ext_vector_type(4)));  // 16 bytes = 8 bf16

// Everything a workgroup needs; passed to the kernel by value.
struct Params {
  const int32_t* instructions;
  u16* hidden;
  u16* q_post_rope;
  u16* k_cache;
  u16* v_cache;
  u16* attn_out;
  float* attn_lse;
  float* attn_partial;
  u16* silu_out;
  u16* logits;
  const u16* attn_norm;
  u16* qkv_raw;         // Qwen3 op set only: QKV before the per-head norm and RoPE
  const u16* q_norm;    // Qwen3 op set only: per-head RMSNorm weights [L, D]
  const u16* k_norm;
  const u16* qkv_w;
  const float* rope_cos;
  const float* rope_sin;
  const u16* o_w;
  const u16* mlp_norm;
  const u16* up_w;
  const u16* gate_w;
  const u16* down_w;
  const u16* lm_norm;
  const u16* lm_w;
  int32_t* barriers;
  uint64_t* ws;         // workspace (tagged units, greedy candidates), else null
  const u16* embed;     // embedding table and destination of the greedy token, or null
  long long* token_out;
  uint64_t* timeline;
  int32_t* status;      // device status words: {code, workgroup, inst, opcode, operand}
  int32_t num_insts;
  int32_t first_inst, end_inst;   // batch route: the columns [first_inst, end_inst) of the instruction tensor run in this launch
  int32_t num_layers;
  int32_t num_layer_barriers;
  int32_t barrier_slots;
  int32_t max_seq_len;
  int32_t max_splits;
  int32_t vocab_size;
  int32_t pos_id;
  float attn_scale;
  float rms_norm_eps;
  int32_t qkv_blocks_per_head;
  int32_t oproj_blocks;
  int32_t upgate_blocks_per_bucket;
  int32_t down_arrivals;
  uint32_t spin_limit;
  uint32_t flags;
  // Batch route only.
  int32_t batch;                 // rows decoded together
  int32_t kv_block;              // tokens per split-KV block
  const int32_t* position_ids;   // [batch] or null: every row decodes pos_id
  const uint8_t* active_mask;    // [batch] or null: every row is active
  uint8_t* partial_valid;        // [batch, NQ, max_splits] or null
  u16* attn_rms_out;             // [batch, H] each
  u16* mlp_rms_out;
  u16* lm_rms_out;
  int32_t rope_rows;
  // MoE route only.
  const u16* qkv_bias;           // [L, QKV]
  const u16* router_w;           // [L, E, H]
  float* router_logits;          // [E]
  long long* expert_indices;     // [top_k]
  float* expert_weights;         // [top_k]
  u16* normed_hidden;            // [H]
  const u16* shared_gate_w;      // [L, Fs, H]
  const u16* shared_up_w;        // [L, Fs, H]
  const u16* shared_down_w;      // [L, H, Fs]
  const u16* shared_scale_w;     // [L, H]: the shared expert's sigmoid gate
  u16* shared_silu;              // [Fs]
  u16* shared_out;               // [H]
  const u16* expert_gate_up_w;   // [L, E, 2 Fm, H], gate rows first
  const u16* expert_down_w;      // [L, E, H, Fm]
  u16* routed_silu;              // [top_k, Fm]
  float* routed_out_f32;         // [H]
  u16* routed_out;               // [H]
  u16* shared_parts;             // workspace: [K slices, H] bf16 partial sums of the shared down projection
  float* routed_parts;           // workspace: [top_k, H] weighted contributions of the routed experts
  float* shared_gate;            // workspace: the layer's sigmoid gate of the shared expert
  int32_t num_experts;
  int32_t top_k;
  int32_t shared_ffn;            // Fs
  int32_t moe_ffn;               // Fm
  int32_t shared_k_slices;
  int32_t norm_topk;             // 1: the top-k weights are divided by their sum
  int32_t routed_tile;           // outputs per tile of the routed up/gate instructions (16, or 8)
  int32_t local_routing;         // tagged launches: 1 = the routed ops take the routing decision themselves from the logits
  // MoE route, several requests in one launch (qmk_rows_ops.h): every per-request buffer above is [batch, ...].
  int32_t ws_row_units;          // 8-byte units from one row's tagged workspace to the next
  int32_t* distinct_out;         // [L] or null: distinct experts each layer streamed in this launch
  int32_t kv_row_tokens;         // KV-cache tokens from one row's cache to the next ([B, L, 1, S, ..]: L*S; [L, B, S, ..]: S)
  int32_t kv_layer_tokens;       // ... from one layer to the next within a row's cache (S, or B*S)
};

// ---------------------------------------------------------------- bf16 ----
__device__ __forceinline__ float bf2f(u16 v) { return __uint_as_float(static_cast<uint32_t>(v) << 16); }

// Round-to-nearest-even, the rounding torch applies on .to(bfloat16).
// float -> bf16, round to nearest even (torch's .to(bfloat16)), as the hardware conversion v_cvt_pk_bf16_f32.  The
// integer form of the same rounding ((u + 0x7fff + ((u >> 16) & 1)) >> 16 with a select for NaN) is six instructions;
// norms, epilogues and merges round thousands of values per layer between two streaming phases, where instruction
// count is time: +1.4 % tok/s on the Llama-3.2-1B shape, +2.1 % Qwen3-1.7B, +2.1 % Qwen1.5-MoE, same bits.
__device__ __forceinline__ u16 f2bf(float f) { return __builtin_bit_cast(u16, static_cast<__bf16>(f)); }
// Two at once, low half first (the instruction converts a pair; written as two f2bf the compiler issues it twice).
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t f2bf2(float lo, float hi) {
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2_t{lo, hi}, bf16x2_t));
}
// 2^x for x <= 0 as one v_exp_f32 (results below the normal range flush to zero, which is what a
// softmax weight that small should be); 2^-inf = 0.
__device__ __forceinline__ float exp2_fast(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float round_bf16(float f) { return bf2f(f2bf(f)); }
__device__ __forceinline__ float bf_lo(uint32_t w) { return __uint_as_float(w << 16); }
__device__ __forceinline__ float bf_hi(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }

// 8 bf16 weights . 8 bf16 activations, fp32 accumulate (4 x v_dot2c_f32_bf16).
// The pairs are taken with shufflevector from the whole 16-byte vector: extracting
// one 32-bit lane first and bit-casting it to a bf16 pair makes this compiler
// reuse lane 0 for all four dot products.
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
__device__ __forceinline__ float dot8(const v4u& w, const v4u& x, float acc) {
  const bf16x8_t a = __builtin_bit_cast(bf16x8_t, w);
  const bf16x8_t b = __builtin_bit_cast(bf16x8_t, x);
  acc = __builtin_amdgcn_fdot2_f32_bf16(__builtin_shufflevector(a, a, 0, 1), __builtin_shufflevector(b, b, 0, 1), acc, false);
  acc = __builtin_amdgcn_fdot2_f32_bf16(__builtin_shufflevector(a, a, 2, 3), __builtin_shufflevector(b, b, 2, 3), acc, false);
  acc = __builtin_amdgcn_fdot2_f32_bf16(__builtin_shufflevector(a, a, 4, 5), __builtin_shufflevector(b, b, 4, 5), acc, false);
  acc = __builtin_amdgcn_fdot2_f32_bf16(__builtin_shufflevector(a, a, 6, 7), __builtin_shufflevector(b, b, 6, 7), acc, false);
  return acc;
}

// ---------------------------------------------------------- reductions ----
// Cross-lane reductions use DPP (data-parallel primitives on the VALU operand path), not
// ds_bpermute shuffles: a shuffle is a round trip through the LDS crossbar (~100 cycles when the
// result is needed at once), and six dependent ones per weight row add up.
template <int kCtrl, int kRowMask = 0xf>
__device__ __forceinline__ float dpp_f32(float identity, float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, identity), __builtin_bit_cast(int, v),
                                                                kCtrl, kRowMask, 0xf, false));
}
constexpr int kDppQuadXor1 = 0xB1;       // quad_perm:[1,0,3,2]
constexpr int kDppQuadXor2 = 0x4E;       // quad_perm:[2,3,0,1]
constexpr int kDppHalfMirror = 0x141;    // row_half_mirror: lane i <-> 7-i within 8 lanes
constexpr int kDppRowShr = 0x110;        // row_shr:n = 0x110 + n
constexpr int kDppRowBcast15 = 0x142;    // lane 15 of a row -> every lane of the next row
constexpr int kDppRowBcast31 = 0x143;    // lane 31 -> every lane of rows 2 and 3

// Sum over the 64 lanes; every lane gets the total.
__device__ __forceinline__ float wave_sum(float v) {
  v += dpp_f32<kDppRowShr + 1>(0.f, v);
  v += dpp_f32<kDppRowShr + 2>(0.f, v);
  v += dpp_f32<kDppRowShr + 4>(0.f, v);
  v += dpp_f32<kDppRowShr + 8>(0.f, v);           // lane 15 of each row: the row's total
  v += dpp_f32<kDppRowBcast15, 0xa>(0.f, v);      // rows 1 and 3 add the row before them
  v += dpp_f32<kDppRowBcast31, 0xc>(0.f, v);      // rows 2 and 3 add rows 0..1
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}

// Maximum over the 64 lanes; every lane gets it.
__device__ __forceinline__ float wave_max(float v) {
  constexpr float kNegInf = -__builtin_huge_valf();
  v = fmaxf(v, dpp_f32<kDppRowShr + 1>(kNegInf, v));
  v = fmaxf(v, dpp_f32<kDppRowShr + 2>(kNegInf, v));
  v = fmaxf(v, dpp_f32<kDppRowShr + 4>(kNegInf, v));
  v = fmaxf(v, dpp_f32<kDppRowShr + 8>(kNegInf, v));
  v = fmaxf(v, dpp_f32<kDppRowBcast15, 0xa>(kNegInf, v));
  v = fmaxf(v, dpp_f32<kDppRowBcast31, 0xc>(kNegInf, v));
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}

// Minimum of a signed integer over the 64 lanes; every lane gets it.
template <int kCtrl, int kRowMask = 0xf>
__device__ __forceinline__ int dpp_i32(int identity, int v) {
  return __builtin_amdgcn_update_dpp(identity, v, kCtrl, kRowMask, 0xf, false);
}
__device__ __forceinline__ int wave_min_i32(int v) {
  constexpr int kMax = 0x7fffffff;
  v = min(v, dpp_i32<kDppRowShr + 1>(kMax, v));
  v = min(v, dpp_i32<kDppRowShr + 2>(kMax, v));
  v = min(v, dpp_i32<kDppRowShr + 4>(kMax, v));
  v = min(v, dpp_i32<kDppRowShr + 8>(kMax, v));
  v = min(v, dpp_i32<kDppRowBcast15, 0xa>(kMax, v));
  v = min(v, dpp_i32<kDppRowBcast31, 0xc>(kMax, v));
  return __builtin_amdgcn_readlane(v, 63);
}

// Sum over each aligned group of 8 lanes; every lane of the group gets the group's total.
__device__ __forceinline__ float group8_sum(float v) {
  v += dpp_f32<kDppQuadXor1>(0.f, v);
  v += dpp_f32<kDppQuadXor2>(0.f, v);
  v += dpp_f32<kDppHalfMirror>(0.f, v);
  return v;
}

// Sum over the workgroup; `scratch` holds kWaves floats.  All threads get the total.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
  v = wave_sum(v);
  const int lane = threadIdx.x & (kWaveSize - 1), wave = threadIdx.x / kWaveSize;
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float t = 0.f;
#pragma unroll
  for (int w = 0; w < kWaves; ++w) t += scratch[w];
  return t;
}

// Maximum over the workgroup; `scratch` holds kWaves floats.  All threads get it.
__device__ __forceinline__ float block_max(float v, float* scratch) {
  v = wave_max(v);
  const int lane = threadIdx.x & (kWaveSize - 1), wave = threadIdx.x / kWaveSize;
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float t = scratch[0];
#pragma unroll
  for (int w = 1; w < kWaves; ++w) t = fmaxf(t, scratch[w]);
  return t;
}

// ------------------------------------------------- counters ("barriers") ----
__device__ __forceinline__ int32_t* counter_ptr(const Params& p, int layer, int row, int slot) {
  return p.barriers + (static_cast<size_t>(layer) * p.num_layer_barriers + row) * p.barrier_slots + slot;
}

// Record the first device-side error; later ones are dropped.
__device__ __forceinline__ void report_error(const Params& p, int code, int inst, int opcode, int operand) {
  if (atomicCAS(p.status, 0, code) == 0) {
    p.status[1] = blockIdx.x;
    p.status[2] = inst;
    p.status[3] = opcode;
    p.status[4] = operand;
  }
}

// One lane polls one counter until it reaches `expected`.  Returns false when
// the poll budget runs out (the producer is gone): the caller retires the
// workgroup so that the grid always drains.
__device__ __forceinline__ bool poll_counter(const int32_t* ctr, int expected, uint32_t limit) {
  uint32_t polls = 0;
  while (__hip_atomic_load(ctr, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < expected) {
    if (++polls > limit) return false;
    __builtin_amdgcn_s_sleep(2);
  }
  return true;
}

// ---- data that one workgroup writes and another reads within the same launch ----
// Each XCD has its own L2, so such data must not be served from (or parked in) a
// local cache.  Instead of writing back / invalidating whole caches around every
// counter, every access to the shared activation buffers is itself device-coherent:
// relaxed agent-scope atomics compile to loads and stores with the sc1 bit, which
// read from and write through to the memory side.  Weights and old KV rows, which no
// workgroup writes during a launch, use ordinary (cached, non-temporal) loads.
__device__ __forceinline__ uint32_t ld_shared32(const void* p) {
  return __hip_atomic_load(static_cast<const uint32_t*>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ uint64_t ld_shared64(const void* p) {
  return __hip_atomic_load(static_cast<const uint64_t*>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float ld_shared_f32(const float* p) { return __uint_as_float(ld_shared32(p)); }
__device__ __forceinline__ v4u ld_shared128(const void* p) {
  const uint64_t lo = ld_shared64(p), hi = ld_shared64(static_cast<const char*>(p) + 8);
  v4u r;
  r.x = static_cast<uint32_t>(lo); r.y = static_cast<uint32_t>(lo >> 32);
  r.z = static_cast<uint32_t>(hi); r.w = static_cast<uint32_t>(hi >> 32);
  return r;
}
// ---- tagged activations (QMK_FLAG_TAGGED) ----
// A hand-over through a counter costs four dependent trips to memory: the producer waits for its
// stores to be acknowledged, adds to the counter, the consumer's poll sees the count, and only
// then does the consumer fetch the data.  Here the data announces itself: every 8-byte unit of
// the workspace is {32-bit payload, 32-bit tag}, written with one 64-bit store, and the tag
// names the launch (a count kept in the workspace) and the layer.  The consumer polls the units
// it needs until they carry the tag it expects: one trip.  A unit is never overwritten before
// all its readers are done: its next writer depends, through the layer's data flow, on every one
// of them.  The split-KV partials do not travel this way: 256 workgroups re-reading 40-200 KiB
// each while they wait for the attention phase floods the fabric; for silu_out (16 KiB) the
// waiting time is short, and not waiting for store acknowledgements behind the next GEMV's row
// requests is worth more than the polling costs.  Offsets below are in units of 8 bytes.
constexpr int kWsGeneration = 0;            // launch count (first 128-byte line)
constexpr int kWsQ = 512;                   // q after RoPE: NQ*D/2 units (two bf16 each; room for 32 heads of 128)
constexpr int kWsK = kWsQ + 2048;           // appended K row: NKV*D/2 units
constexpr int kWsV = kWsK + 1024;           // appended V row (regions sized for 16 KV heads of 128)
constexpr int kWsHiddenMid = kWsV + 1024;   // residual stream after the O-proj: H/2 units
constexpr int kWsHiddenOut = kWsHiddenMid + 1024;  // residual stream after the down projection / the MoE combine step
constexpr int kWsSilu = kWsHiddenOut + 1024;        // silu_out: F/2 units (room for F = 8192)
constexpr int kWsCandidates = kWsSilu + 4096;       // one greedy candidate per workgroup: {logit bits, row}
constexpr int kMaxSamplingQueues = 1024;
constexpr int kWsUnits = kWsCandidates + kMaxSamplingQueues;
// MoE route only, behind the regions above (its workspace is sized by qmk_moe_workspace_bytes):
constexpr int kWsLogits = kWsUnits;                   // router logits, one fp32 per unit (room for 512 experts)
// One router logit per 128-byte line: 128 threads of every workgroup look at the logits from the end of the
// O-projection until the router has stored them, and the stores stand in the same queues as those looks.  Side by side
// (16 logits a line, 8 lines for 128 experts) a logit reached its readers 3 us after it was stored; a line each: +3.5 %
// tok/s on the Qwen3-30B-A3B shape.  (Eight copies of every vector, one per workgroup number modulo 8, did the same for
// the logits and cost 0.5-2 % everywhere else: the other vectors have 64-512 lines each.)
constexpr int kLogitStride = 16;
constexpr int kWsRoutedSilu = kWsLogits + 512 * kLogitStride;        // silu vectors of the routed experts: 1024 units (2048 values) per slot
constexpr int kWsRoutedParts = kWsRoutedSilu + 8 * 1024;   // weighted down-projection rows of the routed experts: H fp32 units per slot
constexpr int kWsSharedGate = kWsRoutedParts + 8 * 2048;   // the shared expert's sigmoid gate, fp32 (a line of its own)
constexpr int kWsTopK = kWsSharedGate + 16;                // the top-k's picks: slot j's expert and weight side by side at 16 j (a line per slot)
constexpr int kWsMoeUnits = kWsTopK + 8 * 16;

__device__ __forceinline__ bool tagged(const Params& p) { return (p.flags & QMK_FLAG_TAGGED) != 0; }
__device__ __forceinline__ uint32_t tag_of(uint32_t generation, int layer) { return (generation << 6) + static_cast<uint32_t>(layer) + 1u; }
__device__ __forceinline__ void st_tagged(uint64_t* unit, uint32_t payload, uint32_t tag) {
  __hip_atomic_store(unit, (static_cast<uint64_t>(tag) << 32) | payload, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// Poll one unit / two neighbouring units until they carry `tag`; false when the budget runs out.
__device__ __forceinline__ bool poll_tagged1(const uint64_t* unit, uint32_t tag, uint32_t limit, uint32_t& a) {
  uint32_t polls = 0;
  while (true) {
    const uint64_t x = ld_shared64(unit);
    if (static_cast<uint32_t>(x >> 32) == tag) {
      a = static_cast<uint32_t>(x);
      return true;
    }
    if (++polls > limit) return false;
    __builtin_amdgcn_s_sleep(1);
  }
}
__device__ __forceinline__ bool poll_tagged2(const uint64_t* units, uint32_t tag, uint32_t limit, uint32_t& a, uint32_t& b) {
  uint32_t polls = 0;
  while (true) {
    const uint64_t x = ld_shared64(units), y = ld_shared64(units + 1);
    if (static_cast<uint32_t>(x >> 32) == tag && static_cast<uint32_t>(y >> 32) == tag) {
      a = static_cast<uint32_t>(x);
      b = static_cast<uint32_t>(y);
      return true;
    }
    if (++polls > limit) return false;
    __builtin_amdgcn_s_sleep(1);
  }
}

__device__ __forceinline__ void st_shared32(void* p, uint32_t v) {
  __hip_atomic_store(static_cast<uint32_t*>(p), v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void st_shared_f32(float* p, float v) { st_shared32(p, __float_as_uint(v)); }
// 16-bit stores have no atomic form; the neighbouring element belongs to the same
// lane's next unit or to another wave, so the element is merged into its word by CAS.
__device__ __forceinline__ void st_shared16(u16* p, u16 v) {
  uint32_t* word = reinterpret_cast<uint32_t*>(reinterpret_cast<uintptr_t>(p) & ~uintptr_t(3));
  const bool high = (reinterpret_cast<uintptr_t>(p) & 2) != 0;
  uint32_t seen = ld_shared32(word);
  while (true) {
    const uint32_t want = high ? ((seen & 0x0000ffffu) | (static_cast<uint32_t>(v) << 16)) : ((seen & 0xffff0000u) | v);
    if (__hip_atomic_compare_exchange_strong(word, &seen, want, __ATOMIC_RELAXED, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) break;
  }
}

// All earlier vector-memory operations of this wave (the write-through stores above
// included) have been acknowledged.  Callers follow it with __syncthreads() and one
// publishing atomic.  s_waitcnt vmcnt(0), expcnt/lgkmcnt left alone.
__device__ __forceinline__ void release_stores() { __builtin_amdgcn_s_waitcnt(0x0F70); }
// Nothing to drop: consumers read shared data with device-coherent loads.
__device__ __forceinline__ void acquire_loads() {}

__device__ __forceinline__ void publish(int32_t* ctr, int amount) {
  __hip_atomic_fetch_add(ctr, amount, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// ---- per-XCD sub-counters for the all-to-all edges (QMK_FLAG_XCD_COUNTERS) ----
// 256 workgroups adding to one word make its cache line bounce between the eight
// XCD-local L2s; a barrier through a single counter costs ~3.8 us on MI355X, through
// eight per-XCD lines (one writer XCD each) ~1.5 us.  Workgroup b runs on XCD b % 8.
constexpr int kXcds = 8;
constexpr int kLineInts = 32;              // 128-byte line
constexpr int kHierFirstRow = 10;          // first row of the sub-counter region of a layer
constexpr int kHierEdges = 4;              // attention, O-proj, up/gate, down  (counter rows 2..5)

__device__ __forceinline__ bool xcd_counters(const Params& p) { return (p.flags & QMK_FLAG_XCD_COUNTERS) != 0; }

__device__ __forceinline__ int32_t* sub_counter(const Params& p, int layer, int row, int xcd) {
  return p.barriers + (static_cast<size_t>(layer) * p.num_layer_barriers + kHierFirstRow) * p.barrier_slots +
         ((row - 2) * kXcds + xcd) * kLineInts;
}

// The attention edge when the O-projection merges the partials itself: every split-KV instruction arrives once and
// EVERY O-proj workgroup polls the count.  Pollers and arrivals on one line stand in each other's way, so an arrival
// goes to eight lines, one per XCD, and a workgroup polls the line of its own XCD alone (32 pollers on a line instead of
// 256).  The lines: the edge's sub-counters with QMK_FLAG_XCD_COUNTERS; otherwise, if the launcher says so (a bit of
// Params::flags that no caller can set), the 256 words from word 0 of row 2 on — a tagged launch leaves counter rows
// 3, 4 and 5 unused.  The kernels that run several rows keep word 0 (their rows' counters lie 32 words apart).
constexpr uint32_t kFlagAttentionRows2To5 = 1u << 16;
// (host side) the choice for a batch-1 launch with these flags and this counter tensor.  The eightfold arrivals pay
// while a layer has few of them (measured: 16 arrivals +1.8 %, 32 +1.0 %, 64 -0.5 %): a model with more than
// eight KV heads keeps word 0 in a tagged launch.
inline uint32_t attention_lines_flag(uint32_t flags, int num_layer_barriers, int barrier_slots, int kv_heads) {
  if ((flags & QMK_FLAG_TAGGED) && !(flags & QMK_FLAG_XCD_COUNTERS) && kv_heads <= 8 && num_layer_barriers >= 6 &&
      4 * barrier_slots >= kXcds * kLineInts)
    return kFlagAttentionRows2To5;
  return 0u;
}

// The kernels that run several rows: a row's attention output is complete when the last split-KV arrival of each of
// its KV-head groups has merged the group and counted its heads, and every O-proj workgroup polls that count.  With
// this bit of Params::flags (the launchers of those kernels set it) the count lives on eight lines at the end of the
// row's tagged workspace, every arrival goes to all eight and a workgroup polls the line of its own XCD.  The lines
// are not per layer: a layer's arrivals all precede the next layer's, so layer l waits for (l + 1) x NQ; the
// workgroup that retires last clears them.
constexpr uint32_t kFlagRowAttentionLines = 1u << 17;
constexpr int kRowAttentionUnits = kXcds * kLineInts / 2;   // eight 128-byte lines, in 8-byte units
__device__ __forceinline__ int32_t* row_attention_line(uint64_t* row_ws, int row_units, int xcd) {
  return reinterpret_cast<int32_t*>(row_ws + row_units - kRowAttentionUnits) + xcd * kLineInts;
}

// Arrival on an all-to-all edge (counter row 2..5, slot 0).
__device__ __forceinline__ void arrive_all(const Params& p, int layer, int row, int amount) {
  publish(xcd_counters(p) ? sub_counter(p, layer, row, blockIdx.x & (kXcds - 1)) : counter_ptr(p, layer, row, 0), amount);
}

// Lanes 0..7 of a wave poll the eight sub-counters until their sum reaches `expected`.
// Must be called by at least the first 8 lanes of the wave; returns the same value in all of them.
__device__ __forceinline__ bool poll_sub_counters(const Params& p, int layer, int row, int expected, uint32_t limit) {
  const int32_t* mine = sub_counter(p, layer, row, threadIdx.x & (kXcds - 1));
  uint32_t polls = 0;
  while (true) {
    int v = __hip_atomic_load(mine, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    v += __shfl_xor(v, 1, kXcds);
    v += __shfl_xor(v, 2, kXcds);
    v += __shfl_xor(v, 4, kXcds);
    if (v >= expected) return true;
    if (++polls > limit) return false;
    __builtin_amdgcn_s_sleep(1);
  }
}

// 2048 lanes polling eight lines that 256 producers are still updating slow the producers
// down.  So only one workgroup per XCD (the "leader", workgroups 0..7) polls the sub-counters;
// when the edge is complete it raises a flag in its own XCD's line (word 1), which the other
// workgroups of that XCD poll out of their local L2.  A follower whose leader does not show up
// (its queue may not contain a consumer of this edge) falls back to polling the sub-counters
// itself after kFollowerPolls tries, and raises the flag for its neighbours too.
constexpr uint32_t kFollowerPolls = 256;

__device__ __forceinline__ bool wait_edge_xcd(const Params& p, int layer, int row, int expected, uint32_t limit) {
  const int xcd = blockIdx.x & (kXcds - 1);
  // The flag has a line of its own (second half of the region): only workgroups of this XCD ever
  // touch it, so it lives in this XCD's L2 and polling it stays off the fabric.
  int32_t* flag = sub_counter(p, layer, row, xcd) + kHierEdges * kXcds * kLineInts;
  const bool leader = blockIdx.x < kXcds || gridDim.x < 2 * kXcds;
  bool ready = false;
  if (!leader) {
    for (uint32_t k = 0; k < kFollowerPolls; ++k) {
      if (__hip_atomic_load(flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0) {
        ready = true;
        break;
      }
      __builtin_amdgcn_s_sleep(1);
    }
  }
  if (!ready) {
    ready = poll_sub_counters(p, layer, row, expected, limit);
    if (ready && (threadIdx.x & (kXcds - 1)) == 0) __hip_atomic_store(flag, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  return ready;
}

// ------------------------------------------------------- row streaming ----
// A wave reads one weight row of CH*512 bf16 as CH fully coalesced 1 KiB loads;
// lane l owns columns (j*64 + l)*8 .. +7 of chunk j.
template <int CH>
struct RowRegs {
  v4u v[CH];
};

template <int CH>
__device__ __forceinline__ void load_row(RowRegs<CH>& r, const u16* row, int lane) {
  const v4u* p = reinterpret_cast<const v4u*>(row) + lane;
#pragma unroll
  for (int j = 0; j < CH; ++j) r.v[j] = __builtin_nontemporal_load(p + j * kWaveSize);
}

template <int CH>
__device__ __forceinline__ float dot_row(const RowRegs<CH>& r, const v4u (&x)[CH]) {
  float a = 0.f;
#pragma unroll
  for (int j = 0; j < CH; ++j) a = dot8(r.v[j], x[j], a);
  return a;
}

// Lane l's activation chunks from a bf16 vector in LDS (same column ownership as load_row).
template <int CH>
__device__ __forceinline__ void load_x_from_lds(v4u (&x)[CH], const u16* lds_vec, int lane) {
  const v4u* p = reinterpret_cast<const v4u*>(lds_vec) + lane;
#pragma unroll
  for (int j = 0; j < CH; ++j) x[j] = p[j * kWaveSize];
}

}  // namespace qmk
