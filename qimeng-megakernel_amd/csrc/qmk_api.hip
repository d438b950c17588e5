// The persistent decode megakernel for gfx950 and its C ABI (include/qmk.h).
//
// One workgroup per instruction queue walks its queue in order; each
// instruction is one fused transformer op on a slice of the output.  Ordering
// across workgroups uses monotone global counters (release/acquire at agent
// scope).  The grid must be co-resident — the launcher checks it — and every
// wait has a poll budget, so the grid drains even if a producer is missing.
//
// Replaces mk_kernel / mk of the reference
// (qimeng_megakernel/models/LLM/llama/llama3_2__1b/A100/single_batch/decode_kernel/mk.cu:29-198).
#include <hip/hip_runtime.h>

#include <mutex>

#include "qmk.h"
#include "qmk_mb_ops.h"
#include "qmk_moe_ops.h"
#include "qmk_ops.h"
#include "qmk_rows_ops.h"

// Workspace of qmk_decode_step_static: the tagged units, the greedy candidates and the launch count
// that qmk_decode_step keeps in the caller's QmkArgs.workspace, here in an array of the library's own
// (94 208 bytes per device, held until the process ends), so that the entry point allocates nothing.
// In host code the name is only a handle for hipGetSymbolAddress: the kernels get the device address
// that call returned (DeviceInfo::scratch), once per device.
static __device__ __align__(256) unsigned long long scratch[qmk::kWsUnits];

namespace qmk {

constexpr int kStatusWords = 8;
constexpr int kMaxDevices = 16;

// {code, workgroup, instruction, opcode, operand}; written only on errors.
__device__ int32_t g_status[kStatusWords];

// The launch's Params as an instruction sees them: read from the kernel-argument segment through a pointer the
// compiler cannot look behind, so what an op needs of them is loaded (scalar loads) inside that op and forgotten
// after it.  Read through the kernel's own by-value parameter, every field is loaded once at the top, outlives the
// whole instruction loop, and — 100 pointers against 100 scalar registers — is parked in vector-register lanes:
// one v_readlane per use, an eighth of all instructions of the MoE kernels (Qwen1.5-MoE shape +4.1 % tok/s,
// Qwen3-30B-A3B +3 %).  The dense kernels park a quarter as many, and there it depends on the op: the up/gate GEMV
// loses 2 % this way (its first row requests wait for the scalar loads), the O-projection gains; which ops of a
// dense kernel read the segment is M::PARAMS_FROM_SEGMENT, measured op by op (Llama-3.2-1B +0.7 %, Qwen3-1.7B +2.7 %
// against all by value).
// What this rests on, checked where it can be: every interpreter kernel takes exactly one argument, a trivially
// copyable Params by value, so the explicit-argument part of the kernel-argument segment is that struct at offset 0
// (explicit arguments come first in the segment, in declaration order, at their natural alignment; the hidden
// arguments follow).  The launcher passes the same struct type, so sizeof agrees by construction.
static_assert(std::is_trivially_copyable<Params>::value && std::is_standard_layout<Params>::value, "Params is copied byte for byte into the kernel-argument segment");
static_assert(alignof(Params) <= 16, "the segment's base alignment covers the struct's");
__device__ __forceinline__ const Params& params_of_this_instruction() {
  auto args = __builtin_amdgcn_kernarg_segment_ptr();   // (a pointer into the constant address space)
  asm volatile("" : "+s"(args));
  return *(const Params*)args;   // the only kernel argument: offset 0 of the segment
}

template <class M>
__global__ __launch_bounds__(kThreads, 1) void decode_megakernel(const Params p_launch) {
  const Params& p = p_launch;
  __shared__ Smem<M> s;
  if (threadIdx.x < 8) s.ctl[threadIdx.x] = 0;
  if (threadIdx.x == 0) {
    s.generation = tagged(p) ? ld_shared32(p.ws + kWsGeneration) : 0u;
    s.best_val = -INFINITY;
    s.best_idx = 0x7fffffff;
  }
  __syncthreads();

  const int32_t* queue = p.instructions + static_cast<size_t>(blockIdx.x) * p.num_insts * kInstWords;
  bool ok = true;
  // Two instructions are visible at a time (the second one for requests made on its behalf); the
  // words of instruction i+2 are asked for while instruction i runs.
  int32_t word = (threadIdx.x < kInstWords && p.num_insts > 0) ? queue[threadIdx.x] : 0;
  int32_t word1 = (threadIdx.x < kInstWords && p.num_insts > 1) ? queue[kInstWords + threadIdx.x] : 0;
  Carried carry;
  bool carried = false, parked = false, after_attention = false;
  forget(carry);
  const int num_insts = p.num_insts;
  for (int i = 0; i < num_insts && ok; ++i) {
    if (threadIdx.x < kInstWords) {
      s.inst[threadIdx.x] = word;
      s.next[threadIdx.x] = word1;
      word = word1;
      word1 = (i + 2 < num_insts) ? queue[(i + 2) * kInstWords + threadIdx.x] : 0;
    }
    __syncthreads();
    const Params& from_segment = params_of_this_instruction();
    auto params_for = [&](int op) -> const Params& { return (M::PARAMS_FROM_SEGMENT & op) ? from_segment : p; };
    const int opcode = s.inst[0];
    int tid = threadIdx.x;
    asm volatile("" : "+v"(tid));
    const Ctx c{i, opcode, tid};
    unsigned long long t_start = 0;
    if (p.timeline != nullptr && threadIdx.x == 0) {
      t_start = wall_clock64();
      for (int k = 0; k < 4; ++k) s.stamps[k] = t_start;
    }
    // Only the O-proj hands rows to its successor: every other arm ends their life explicitly.
    switch (opcode) {
      case OP_NOOP: forget(carry); break;
      case OP_RMS_QKV_ROPE: [[clang::always_inline]] ok = op_rms_qkv_rope<M>(params_for(kSegmentQkv), s, c); forget(carry); break;
      case OP_ATTN_SPLITKV: [[clang::always_inline]] ok = op_attn_splitkv<M>(params_for(kSegmentAttention), s, c); forget(carry); break;
      case OP_ATTN_REDUCE: [[clang::always_inline]] ok = op_attn_reduce<M>(p, s, c); forget(carry); break;
      case OP_OPROJ_RESIDUAL:
        carried = M::CARRY_AFTER_ATTENTION || !after_attention;
        parked = !after_attention;   // a workgroup that has just run the attention has no wait to fill
        [[clang::always_inline]] ok = op_oproj_residual<M>(params_for(kSegmentOproj), s, c, carry, carried, parked);
        break;
      case OP_RMS_UPGATE_SILU: [[clang::always_inline]] ok = op_rms_upgate_silu<M>(params_for(kSegmentUpGate), s, c, carry, carried, parked); forget(carry); break;
      case OP_DOWN_RESIDUAL: [[clang::always_inline]] ok = op_down_residual<M>(params_for(kSegmentDown), s, c); forget(carry); break;
      case OP_RMS_LMHEAD: [[clang::always_inline]] ok = op_rms_lmhead<M>(params_for(kSegmentLmHead), s, c); forget(carry); break;
      default:
        if (threadIdx.x == 0) report_error(p, QMK_DEV_BAD_OPCODE, i, opcode, 0);
        ok = false;
        forget(carry);
        break;
    }
    if (opcode != OP_OPROJ_RESIDUAL) carried = parked = false;
    after_attention = opcode == OP_ATTN_SPLITKV || opcode == OP_ATTN_REDUCE;

    if (p.timeline != nullptr && threadIdx.x == 0) {
      uint64_t* rec = p.timeline + (static_cast<size_t>(blockIdx.x) * p.num_insts + i) * 8;
      rec[0] = t_start;
      rec[1] = s.ctl[2] ? s.t_wait : t_start;
      rec[2] = wall_clock64();
      rec[3] = static_cast<uint64_t>(opcode) | (static_cast<uint64_t>(static_cast<uint32_t>(s.inst[1])) << 8);
      for (int k = 0; k < 4; ++k) rec[4 + k] = s.stamps[k];
      s.ctl[2] = 0;
    }
    __syncthreads();  // s.inst and s.x are reused by the next instruction
  }
  if (!ok || (p.flags & QMK_FLAG_KEEP_BARRIERS)) return;

  // Retire.  The workgroup that arrives last owns the counters alone (every
  // other queue is finished, so nobody polls any more) and clears them for the
  // next step.  The arrival counter is the last word of layer 0's last row.
  // Greedy chaining: the workgroup's candidate {order-preserving logit bits, row} is in memory
  // before the arrival below, so the last workgroup finds all of them.
  const bool sampling = p.token_out != nullptr;
  if (sampling && threadIdx.x == 0) {
    const uint32_t bits = __float_as_uint(s.best_val);
    const uint32_t key = (bits & 0x80000000u) ? ~bits : (bits | 0x80000000u);  // larger float <=> larger key
    __hip_atomic_store(p.ws + kWsCandidates + blockIdx.x, (static_cast<uint64_t>(key) << 32) | static_cast<uint32_t>(s.best_idx),
                       __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  release_stores();  // our publishing atomics have landed before we say we are done
  __syncthreads();
  int32_t* done = counter_ptr(p, 0, p.num_layer_barriers - 1, p.barrier_slots - 1);
  if (threadIdx.x == 0) {
    const int prev = __hip_atomic_fetch_add(done, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    s.ctl[1] = (prev == static_cast<int>(gridDim.x) - 1);
  }
  __syncthreads();
  if (s.ctl[1]) {
    const int total = p.num_layers * p.num_layer_barriers * p.barrier_slots;
    for (int i = threadIdx.x; i < total; i += kThreads)
      __hip_atomic_store(p.barriers + i, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    // The next launch tags its activations with the next count (26 bits: the tag keeps 6 for the layer).
    if (tagged(p) && threadIdx.x == 0) st_shared32(p.ws + kWsGeneration, (s.generation + 1u) & 0x03ffffffu);
    if (sampling) {
      // Largest logit, smallest row among equals (torch.argmax's choice): the key orders by logit,
      // the complemented row breaks ties towards the first row.
      uint64_t mine = 0;
      for (int q = threadIdx.x; q < static_cast<int>(gridDim.x); q += kThreads) {
        const uint64_t cand = ld_shared64(p.ws + kWsCandidates + q);
        const uint64_t ordered = (cand & 0xffffffff00000000ull) | (0xffffffffu - static_cast<uint32_t>(cand));
        mine = ordered > mine ? ordered : mine;
      }
      for (int off = 1; off < kWaveSize; off <<= 1) {
        const uint32_t lo = __shfl_xor(static_cast<uint32_t>(mine), off), hi = __shfl_xor(static_cast<uint32_t>(mine >> 32), off);
        const uint64_t other = (static_cast<uint64_t>(hi) << 32) | lo;
        mine = other > mine ? other : mine;
      }
      uint64_t* slots = reinterpret_cast<uint64_t*>(s.res);
      if ((threadIdx.x & (kWaveSize - 1)) == 0) slots[threadIdx.x >> 6] = mine;
      __syncthreads();
      uint64_t best = slots[0];
      for (int w = 1; w < kWaves; ++w) best = slots[w] > best ? slots[w] : best;
      const uint32_t token = 0xffffffffu - static_cast<uint32_t>(best);
      if (token < static_cast<uint32_t>(p.vocab_size)) {  // no LM-head instruction ran: leave both untouched
        if (threadIdx.x == 0) *p.token_out = static_cast<long long>(token);
        static_assert(M::H == kThreads * 4, "one thread copies four embedding elements");
        const uint2 row = *reinterpret_cast<const uint2*>(p.embed + static_cast<size_t>(token) * M::H + threadIdx.x * 4);
        *reinterpret_cast<uint2*>(p.hidden + threadIdx.x * 4) = row;
      }
    }
  }
}

// The batch route's interpreter: same queue walk, the ten opcodes of qmk_mb_ops.h, the reference's
// counter protocol per batch row (…/A100/multi_batch/decode_kernel/mk.cu).  Per-row positions and
// activity are read once per launch.
template <class M>
__global__ __launch_bounds__(kThreads, 1) void decode_megakernel_batch(const Params p) {
  __shared__ mb::Smem<M> s;
  if (threadIdx.x < 8) s.ctl[threadIdx.x] = 0;
  if (threadIdx.x < mb::kMaxBatch) {   // one wave: the zeroing above has happened for all of them
    const int b = threadIdx.x;
    int pos = 0, on = 0;
    if (b < p.batch) {
      pos = p.position_ids != nullptr ? p.position_ids[b] : p.pos_id;
      on = p.active_mask != nullptr ? (p.active_mask[b] != 0) : 1;
      if (pos < 0 || pos >= p.max_seq_len || pos >= p.rope_rows) {
        s.ctl[0] = 1;
        report_error(p, QMK_DEV_BAD_OPERAND, -1, 0, b);
        pos = 0;
      }
    }
    s.pos[b] = pos;
    s.active[b] = on;
  }
  __syncthreads();
  bool ok = s.ctl[0] == 0;

  const int32_t* queue = p.instructions + static_cast<size_t>(blockIdx.x) * p.num_insts * kInstWords;
  // A launch runs the columns [first_inst, end_inst) of the tensor: all of them, or the window of a column-by-column run
  // (…/multi_batch/decode_kernel/mk.h:44-115: mk_step, mk_step_loop).
  int32_t word = (threadIdx.x < kInstWords && p.first_inst < p.end_inst) ? queue[p.first_inst * kInstWords + threadIdx.x] : 0;
  for (int i = p.first_inst; i < p.end_inst && ok; ++i) {
    if (threadIdx.x < kInstWords) {
      s.inst[threadIdx.x] = word;
      word = (i + 1 < p.end_inst) ? queue[(i + 1) * kInstWords + threadIdx.x] : 0;
    }
    __syncthreads();
    const int opcode = s.inst[0];
    int tid = threadIdx.x;
    asm volatile("" : "+v"(tid));
    const Ctx c{i, opcode, tid};
    unsigned long long t_start = 0;
    if (p.timeline != nullptr && threadIdx.x == 0) {
      t_start = wall_clock64();
      for (int k = 0; k < 4; ++k) s.stamps[k] = t_start;
    }
    switch (opcode) {
      case mb::OP_NOOP: break;
      case mb::OP_ATTN_RMS:
      case mb::OP_MLP_RMS:
      case mb::OP_LM_RMS: [[clang::always_inline]] ok = mb::op_rms_row<M>(p, s, c); break;
      case mb::OP_QKV: [[clang::always_inline]] ok = mb::op_qkv<M>(p, s, c); break;
      case mb::OP_SPLITKV: [[clang::always_inline]] ok = mb::op_splitkv<M>(p, s, c); break;
      case mb::OP_REDUCE: [[clang::always_inline]] ok = mb::op_reduce<M>(p, s, c); break;
      case mb::OP_OPROJ: [[clang::always_inline]] ok = mb::op_oproj<M>(p, s, c); break;
      case mb::OP_UPGATE: [[clang::always_inline]] ok = mb::op_upgate<M>(p, s, c); break;
      case mb::OP_DOWN: [[clang::always_inline]] ok = mb::op_down<M>(p, s, c); break;
      case mb::OP_LMHEAD: [[clang::always_inline]] ok = mb::op_lmhead<M>(p, s, c); break;
      default:
        if (threadIdx.x == 0) report_error(p, QMK_DEV_BAD_OPCODE, i, opcode, 0);
        ok = false;
        break;
    }
    if (p.timeline != nullptr && threadIdx.x == 0) {
      uint64_t* rec = p.timeline + (static_cast<size_t>(blockIdx.x) * p.num_insts + i) * 8;
      rec[0] = t_start;
      rec[1] = s.ctl[2] ? s.t_wait : t_start;
      rec[2] = wall_clock64();
      rec[3] = static_cast<uint64_t>(opcode) | (static_cast<uint64_t>(static_cast<uint32_t>(s.inst[1])) << 8);
      for (int k = 0; k < 4; ++k) rec[4 + k] = s.stamps[k];
      s.ctl[2] = 0;
    }
    __syncthreads();  // s.inst and the staging areas are reused by the next instruction
  }
  if (!ok || (p.flags & QMK_FLAG_KEEP_BARRIERS)) return;

  // Retire: the workgroup that arrives last owns the counters alone and clears them for the next
  // step.  The arrival counter is the last word of layer 0's last row (row 9 carries no counter).
  release_stores();
  __syncthreads();
  int32_t* done = counter_ptr(p, 0, p.num_layer_barriers - 1, p.barrier_slots - 1);
  if (threadIdx.x == 0) {
    const int prev = __hip_atomic_fetch_add(done, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    s.ctl[1] = (prev == static_cast<int>(gridDim.x) - 1);
  }
  __syncthreads();
  if (s.ctl[1]) {
    const int total = p.num_layers * p.num_layer_barriers * p.barrier_slots;
    for (int i = threadIdx.x; i < total; i += kThreads)
      __hip_atomic_store(p.barriers + i, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}

// The MoE route's interpreter: the dense route's attention and LM head (opcodes 1-4, 7) and the MoE
// block (8-14) on the reference's counters (…/qwen1_5_moe_a2_7b/A100/single_batch/decode_kernel/mk.cu).
template <class M>
__global__ __launch_bounds__(kThreads, 1) void decode_megakernel_moe(const Params p_launch) {
  const Params& p = p_launch;
  __shared__ Smem<M> s;
  if (threadIdx.x < 8) s.ctl[threadIdx.x] = 0;
  if (threadIdx.x == 0) {
    s.route_layer = -1;
    s.generation = tagged(p) ? ld_shared32(p.ws + kWsGeneration) : 0u;
    s.best_val = -INFINITY;
    s.best_idx = 0x7fffffff;
  }
  __syncthreads();
  const int32_t* queue = p.instructions + static_cast<size_t>(blockIdx.x) * p.num_insts * kInstWords;
  bool ok = true;
  int32_t word = (threadIdx.x < kInstWords && p.num_insts > 0) ? queue[threadIdx.x] : 0;
  int32_t word1 = (threadIdx.x < kInstWords && p.num_insts > 1) ? queue[kInstWords + threadIdx.x] : 0;
  Carried carry;
  forget(carry);
  const int num_insts = p.num_insts;
  for (int i = 0; i < num_insts && ok; ++i) {
    if (threadIdx.x < kInstWords) {
      s.inst[threadIdx.x] = word;
      s.next[threadIdx.x] = word1;
      word = word1;
      word1 = (i + 2 < num_insts) ? queue[(i + 2) * kInstWords + threadIdx.x] : 0;
    }
    __syncthreads();
    const Params& p = params_of_this_instruction();
    const int opcode = s.inst[0];
    int tid = threadIdx.x;
    asm volatile("" : "+v"(tid));
    const Ctx c{i, opcode, tid};
    unsigned long long t_start = 0;
    if (p.timeline != nullptr && threadIdx.x == 0) {
      t_start = wall_clock64();
      for (int k = 0; k < 4; ++k) s.stamps[k] = t_start;
    }
    bool carried = false, parked = false;
    // Every op inlined, whatever its size: an op left out of line takes `p` by reference, and the kernel
    // arguments then live in private memory for all ops (vector loads from scratch instead of scalar loads).
    switch (opcode) {
      case OP_NOOP: break;
      case OP_RMS_QKV_ROPE: [[clang::always_inline]] ok = op_rms_qkv_rope<M>(p, s, c); break;
      case OP_ATTN_SPLITKV: [[clang::always_inline]] ok = op_attn_splitkv<M>(p, s, c); break;
      case OP_ATTN_REDUCE: [[clang::always_inline]] ok = op_attn_reduce<M>(p, s, c); break;
      case OP_OPROJ_RESIDUAL: [[clang::always_inline]] ok = op_oproj_residual<M>(p, s, c, carry, carried, parked); break;
      case OP_RMS_LMHEAD: [[clang::always_inline]] ok = op_rms_lmhead<M>(p, s, c); break;
      case moe::OP_ROUTER: [[clang::always_inline]] ok = moe::op_router<M>(p, s, c); break;
      case moe::OP_TOPK: [[clang::always_inline]] ok = moe::op_topk<M>(p, s, c); break;
      case moe::OP_SHARED_UPGATE: [[clang::always_inline]] ok = moe::op_shared_upgate<M>(p, s, c); break;
      case moe::OP_SHARED_DOWN: [[clang::always_inline]] ok = moe::op_shared_down<M>(p, s, c); break;
      case moe::OP_ROUTED_UPGATE: [[clang::always_inline]] ok = moe::op_routed_upgate<M>(p, s, c); break;
      case moe::OP_ROUTED_DOWN: [[clang::always_inline]] ok = moe::op_routed_down<M>(p, s, c); break;
      case moe::OP_COMBINE: [[clang::always_inline]] ok = moe::op_combine<M>(p, s, c); break;
      default:
        if (threadIdx.x == 0) report_error(p, QMK_DEV_BAD_OPCODE, i, opcode, 0);
        ok = false;
        break;
    }
    forget(carry);
    if (p.timeline != nullptr && threadIdx.x == 0) {
      uint64_t* rec = p.timeline + (static_cast<size_t>(blockIdx.x) * p.num_insts + i) * 8;
      rec[0] = t_start;
      rec[1] = s.ctl[2] ? s.t_wait : t_start;
      rec[2] = wall_clock64();
      rec[3] = static_cast<uint64_t>(opcode) | (static_cast<uint64_t>(static_cast<uint32_t>(s.inst[1])) << 8);
      for (int k = 0; k < 4; ++k) rec[4 + k] = s.stamps[k];
      s.ctl[2] = 0;
    }
    __syncthreads();
  }
  if (!ok || (p.flags & QMK_FLAG_KEEP_BARRIERS)) return;
  // Retire: the last workgroup clears the counters (arrival counter: last word of layer 0's last row, which
  // is row 14 and carries no counter of the protocol).
  release_stores();
  __syncthreads();
  int32_t* done = counter_ptr(p, 0, p.num_layer_barriers - 1, p.barrier_slots - 1);
  if (threadIdx.x == 0) {
    const int prev = __hip_atomic_fetch_add(done, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    s.ctl[1] = (prev == static_cast<int>(gridDim.x) - 1);
  }
  __syncthreads();
  if (s.ctl[1]) {
    const int total = p.num_layers * p.num_layer_barriers * p.barrier_slots;
    for (int i = threadIdx.x; i < total; i += kThreads)
      __hip_atomic_store(p.barriers + i, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    // The next launch tags its activations with the next count (26 bits: the tag keeps 6 for the layer).
    if (tagged(p) && threadIdx.x == 0) st_shared32(p.ws + kWsGeneration, (s.generation + 1u) & 0x03ffffffu);
  }
}


// The MoE route for several requests in one launch (qmk_rows_ops.h): the same queue walk; opcodes 1, 4, 7, 8 for all
// rows at once, 2 and 9 as the batch-1 ops on a row's view of the buffers, 15 and 16 over the layer's distinct experts.
// The parameters are the kernel's by-value argument throughout.
template <class M>
__global__ __launch_bounds__(kThreads, 1) void decode_megakernel_moe_rows(const Params p) {
  __shared__ rows::Smem<M> s;
  if (threadIdx.x < 8) s.b.ctl[threadIdx.x] = 0;
  if (threadIdx.x < rows::kMaxRows) {
    const int b = threadIdx.x;
    int pos = 0;
    if (b < p.batch) {
      pos = p.position_ids[b];
      if (pos < 0 || pos >= p.max_seq_len || pos >= p.rope_rows) {
        s.b.ctl[0] = 1;
        report_error(p, QMK_DEV_BAD_OPERAND, -1, 0, b);
        pos = 0;
      }
    }
    s.pos[b] = pos;
    s.live[b] = b < p.batch;
  }
  if (threadIdx.x == 0) {
    s.route_layer = -1;
    s.n_list = 0;
    s.b.route_layer = -1;
    s.b.generation = ld_shared32(p.ws + kWsGeneration);   // row 0's workspace keeps the launch count for all rows
    s.b.best_val = -INFINITY;
    s.b.best_idx = 0x7fffffff;
  }
  __syncthreads();
  bool ok = s.b.ctl[0] == 0;
  const int32_t* queue = p.instructions + static_cast<size_t>(blockIdx.x) * p.num_insts * kInstWords;
  int32_t word = (threadIdx.x < kInstWords && p.num_insts > 0) ? queue[threadIdx.x] : 0;
  int32_t word1 = (threadIdx.x < kInstWords && p.num_insts > 1) ? queue[kInstWords + threadIdx.x] : 0;
  const int num_insts = p.num_insts;
  for (int i = 0; i < num_insts && ok; ++i) {
    if (threadIdx.x < kInstWords) {
      s.b.inst[threadIdx.x] = word;
      s.b.next[threadIdx.x] = word1;
      word = word1;
      word1 = (i + 2 < num_insts) ? queue[(i + 2) * kInstWords + threadIdx.x] : 0;
    }
    __syncthreads();
    const int opcode = s.b.inst[0];
    int tid = threadIdx.x;
    asm volatile("" : "+v"(tid));
    const Ctx c{i, opcode, tid};
    unsigned long long t_start = 0;
    if (p.timeline != nullptr && threadIdx.x == 0) {
      t_start = wall_clock64();
      for (int k = 0; k < 4; ++k) s.b.stamps[k] = t_start;
    }
    switch (opcode) {
      case OP_NOOP: break;
      case OP_RMS_QKV_ROPE: [[clang::always_inline]] ok = rows::op_qkv<M>(p, s, c); break;
      case OP_ATTN_SPLITKV: {
        const int row = s.b.inst[6];   // the word behind the batch-1 operands
        if (row < 0 || row >= p.batch) {
          ok = rows::bad_operand(p, s, c, 6);
        } else {
          const Params pr = rows::row_view<M>(p, row, s.pos[row]);
          [[clang::always_inline]] ok = op_attn_splitkv<rows::Inner<M>>(pr, s.b, c);
        }
        break;
      }
      case OP_OPROJ_RESIDUAL: [[clang::always_inline]] ok = rows::op_oproj<M>(p, s, c); break;
      case OP_RMS_LMHEAD: [[clang::always_inline]] ok = rows::op_lmhead<M>(p, s, c); break;
      case moe::OP_ROUTER: [[clang::always_inline]] ok = rows::op_router<M>(p, s, c); break;
      case moe::OP_TOPK: {
        const int row = s.b.inst[2];
        if (row < 0 || row >= p.batch) {
          ok = rows::bad_operand(p, s, c, 2);
        } else {
          const Params pr = rows::row_view<M>(p, row, s.pos[row]);
          [[clang::always_inline]] ok = moe::op_topk<rows::Inner<M>>(pr, s.b, c);
        }
        break;
      }
      case rows::OP_ROUTED_UPGATE_ROWS: [[clang::always_inline]] ok = rows::op_routed_upgate<M>(p, s, c); break;
      case rows::OP_ROUTED_DOWN_COMMIT_ROWS: [[clang::always_inline]] ok = rows::op_routed_down_commit<M>(p, s, c); break;
      default:
        if (threadIdx.x == 0) report_error(p, QMK_DEV_BAD_OPCODE, i, opcode, 0);
        ok = false;
        break;
    }
    if (p.timeline != nullptr && threadIdx.x == 0) {
      uint64_t* rec = p.timeline + (static_cast<size_t>(blockIdx.x) * p.num_insts + i) * 8;
      rec[0] = t_start;
      rec[1] = s.b.ctl[2] ? s.b.t_wait : t_start;
      rec[2] = wall_clock64();
      rec[3] = static_cast<uint64_t>(opcode) | (static_cast<uint64_t>(static_cast<uint32_t>(s.b.inst[1])) << 8);
      for (int k = 0; k < 4; ++k) rec[4 + k] = s.b.stamps[k];
      s.b.ctl[2] = 0;
    }
    __syncthreads();
  }
  if (!ok) return;
  // Retire: the last workgroup clears the counters and advances the launch count the tags are derived from.
  release_stores();
  __syncthreads();
  int32_t* done = counter_ptr(p, 0, p.num_layer_barriers - 1, p.barrier_slots - 1);
  if (threadIdx.x == 0) {
    const int prev = __hip_atomic_fetch_add(done, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    s.b.ctl[1] = (prev == static_cast<int>(gridDim.x) - 1);
  }
  __syncthreads();
  if (s.b.ctl[1]) {
    const int total = p.num_layers * p.num_layer_barriers * p.barrier_slots;
    for (int i = threadIdx.x; i < total; i += kThreads)
      __hip_atomic_store(p.barriers + i, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (p.flags & kFlagRowAttentionLines)   // the rows' attention counts, which ran through the layers
      for (int i = threadIdx.x; i < p.batch * kXcds * kLineInts; i += kThreads)
        __hip_atomic_store(row_attention_line(rows::ws_of(p, i / (kXcds * kLineInts)), p.ws_row_units, 0) + i % (kXcds * kLineInts), 0,
                           __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (threadIdx.x == 0) st_shared32(p.ws + kWsGeneration, (s.b.generation + 1u) & 0x03ffffffu);
  }
}

// The dense route for 1..4 requests in one launch on the batch-1 row-streaming engine (qmk_rows_ops.h): opcodes 1, 4, 5,
// 6, 7 of the batch-1 route for all rows at once, 2 as the batch-1 op on a row's view of the buffers.  Buffers in the
// batch route's layout ([B, ...]; KV cache [L, B, S, Hkv, D]); a row whose active flag is off is a hole: nothing of it is
// read or written but its logits, which are set to -1e9 as the batch route does.
template <class M>
__global__ __launch_bounds__(kThreads, 1) void decode_megakernel_rows(const Params p) {
  __shared__ rows::Smem<M> s;
  if (threadIdx.x < 8) s.b.ctl[threadIdx.x] = 0;
  if (threadIdx.x < rows::kMaxRows) {
    const int b = threadIdx.x;
    int pos = 0, on = 0;
    if (b < p.batch) {
      pos = p.position_ids != nullptr ? p.position_ids[b] : p.pos_id;
      on = p.active_mask != nullptr ? (p.active_mask[b] != 0) : 1;
      if (on && (pos < 0 || pos >= p.kv_row_tokens || pos >= p.rope_rows)) {
        s.b.ctl[0] = 1;
        report_error(p, QMK_DEV_BAD_OPERAND, -1, 0, b);
      }
      if (pos < 0 || pos >= p.kv_row_tokens || pos >= p.rope_rows) pos = 0;
    }
    s.pos[b] = pos;
    s.live[b] = on;
  }
  if (threadIdx.x == 0) {
    s.route_layer = -1;
    s.n_list = 0;
    s.b.generation = ld_shared32(p.ws + kWsGeneration);
    s.b.best_val = -INFINITY;
    s.b.best_idx = 0x7fffffff;
  }
  __syncthreads();
  bool ok = s.b.ctl[0] == 0;
  const int32_t* queue = p.instructions + static_cast<size_t>(blockIdx.x) * p.num_insts * kInstWords;
  int32_t word = (threadIdx.x < kInstWords && p.num_insts > 0) ? queue[threadIdx.x] : 0;
  int32_t word1 = (threadIdx.x < kInstWords && p.num_insts > 1) ? queue[kInstWords + threadIdx.x] : 0;
  const int num_insts = p.num_insts;
  Carried carry;
  bool carried = false, parked = false, after_attention = false;
  forget(carry);
  for (int i = 0; i < num_insts && ok; ++i) {
    if (threadIdx.x < kInstWords) {
      s.b.inst[threadIdx.x] = word;
      s.b.next[threadIdx.x] = word1;
      word = word1;
      word1 = (i + 2 < num_insts) ? queue[(i + 2) * kInstWords + threadIdx.x] : 0;
    }
    __syncthreads();
    const int opcode = s.b.inst[0];
    int tid = threadIdx.x;
    asm volatile("" : "+v"(tid));
    const Ctx c{i, opcode, tid};
    unsigned long long t_start = 0;
    if (p.timeline != nullptr && threadIdx.x == 0) {
      t_start = wall_clock64();
      for (int k = 0; k < 4; ++k) s.b.stamps[k] = t_start;
    }
    switch (opcode) {
      // Only the O-projection hands rows to its successor: every other arm ends their life explicitly.
      case OP_NOOP: forget(carry); break;
      case OP_RMS_QKV_ROPE: [[clang::always_inline]] ok = rows::op_qkv<M>(p, s, c); forget(carry); break;
      case OP_ATTN_SPLITKV: {
        const int row = s.b.inst[6];   // the word behind the batch-1 operands
        if (row < 0 || row >= p.batch) {
          ok = rows::bad_operand(p, s, c, 6);
        } else if (s.live[row]) {
          const Params pr = rows::row_view<M>(p, row, s.pos[row]);
          [[clang::always_inline]] ok = op_attn_splitkv<rows::Inner<M>>(pr, s.b, c);
        }
        forget(carry);
        break;
      }
      case OP_OPROJ_RESIDUAL:
        carried = M::CARRY_AFTER_ATTENTION || !after_attention;
        parked = !after_attention;   // a workgroup that has just run the attention has no wait to fill
        [[clang::always_inline]] ok = rows::op_oproj<M, rows::AsksAhead<M>::value>(p, s, c, carry, carried, parked);
        break;
      case OP_RMS_UPGATE_SILU: [[clang::always_inline]] ok = rows::op_upgate<M>(p, s, c, carry, carried, parked); forget(carry); break;
      case OP_DOWN_RESIDUAL: [[clang::always_inline]] ok = rows::op_down<M>(p, s, c); forget(carry); break;
      case OP_RMS_LMHEAD: [[clang::always_inline]] ok = rows::op_lmhead<M>(p, s, c); forget(carry); break;
      default:
        if (threadIdx.x == 0) report_error(p, QMK_DEV_BAD_OPCODE, i, opcode, 0);
        ok = false;
        forget(carry);
        break;
    }
    if (opcode != OP_OPROJ_RESIDUAL) carried = parked = false;
    after_attention = opcode == OP_ATTN_SPLITKV;
    if (p.timeline != nullptr && threadIdx.x == 0) {
      uint64_t* rec = p.timeline + (static_cast<size_t>(blockIdx.x) * p.num_insts + i) * 8;
      rec[0] = t_start;
      rec[1] = s.b.ctl[2] ? s.b.t_wait : t_start;
      rec[2] = wall_clock64();
      rec[3] = static_cast<uint64_t>(opcode) | (static_cast<uint64_t>(static_cast<uint32_t>(s.b.inst[1])) << 8);
      for (int k = 0; k < 4; ++k) rec[4 + k] = s.b.stamps[k];
      s.b.ctl[2] = 0;
    }
    __syncthreads();
  }
  if (!ok) return;
  release_stores();
  __syncthreads();
  int32_t* done = counter_ptr(p, 0, p.num_layer_barriers - 1, p.barrier_slots - 1);
  if (threadIdx.x == 0) {
    const int prev = __hip_atomic_fetch_add(done, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    s.b.ctl[1] = (prev == static_cast<int>(gridDim.x) - 1);
  }
  __syncthreads();
  if (s.b.ctl[1]) {
    const int total = p.num_layers * p.num_layer_barriers * p.barrier_slots;
    for (int i = threadIdx.x; i < total; i += kThreads)
      __hip_atomic_store(p.barriers + i, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (p.flags & kFlagRowAttentionLines)   // the rows' attention counts, which ran through the layers
      for (int i = threadIdx.x; i < p.batch * kXcds * kLineInts; i += kThreads)
        __hip_atomic_store(row_attention_line(rows::ws_of(p, i / (kXcds * kLineInts)), p.ws_row_units, 0) + i % (kXcds * kLineInts), 0,
                           __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (threadIdx.x == 0) st_shared32(p.ws + kWsGeneration, (s.b.generation + 1u) & 0x03ffffffu);
  }
}

static_assert(std::is_same<decltype(&decode_megakernel<Llama1B>), void (*)(const Params)>::value &&
                  std::is_same<decltype(&decode_megakernel<Qwen3_1p7B>), void (*)(const Params)>::value &&
                  std::is_same<decltype(&decode_megakernel_moe<QwenMoeA2_7B>), void (*)(const Params)>::value &&
                  std::is_same<decltype(&decode_megakernel_moe<Qwen3MoeA3B>), void (*)(const Params)>::value,
              "the kernels that read the kernel-argument segment have one by-value Params argument and nothing else");

struct DeviceInfo {
  bool ready = false;
  int cu_count = 0;
  int max_queues = 0;
  int max_queues_batch = 0;
  int max_queues_batch_qwen3 = 0;
  int max_queues_moe = 0;
  int max_queues_moe_rows = 0;
  int max_queues_rows = 0;
  int32_t* status = nullptr;
  uint64_t* scratch = nullptr;   // this device's copy of the file-scope `scratch` array
  bool static_in_use = false;    // a launch since the last status fetch used that array as its workspace
};
DeviceInfo g_devices[kMaxDevices];
std::mutex g_mutex;

int device_info(DeviceInfo** out) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return QMK_ERR_NO_DEVICE;
  std::lock_guard<std::mutex> lock(g_mutex);
  DeviceInfo& d = g_devices[dev];
  if (!d.ready) {
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, dev) != hipSuccess) return QMK_ERR_NO_DEVICE;
    int per_cu = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, decode_megakernel<Llama1B>, kThreads, 0) != hipSuccess)
      return QMK_ERR_NO_DEVICE;
    int per_cu_batch = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu_batch, decode_megakernel_batch<Llama1B>, kThreads, 0) != hipSuccess)
      return QMK_ERR_NO_DEVICE;
    int per_cu_batch3 = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu_batch3, decode_megakernel_batch<Qwen3_1p7B>, kThreads, 0) != hipSuccess)
      return QMK_ERR_NO_DEVICE;
    int per_cu_moe = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu_moe, decode_megakernel_moe<QwenMoeA2_7B>, kThreads, 0) != hipSuccess)
      return QMK_ERR_NO_DEVICE;
    int per_cu_moe3 = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu_moe3, decode_megakernel_moe<Qwen3MoeA3B>, kThreads, 0) != hipSuccess)
      return QMK_ERR_NO_DEVICE;
    per_cu_moe = per_cu_moe3 < per_cu_moe ? per_cu_moe3 : per_cu_moe;
    int per_cu_rows = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu_rows, decode_megakernel_moe_rows<Qwen3MoeA3B>, kThreads, 0) != hipSuccess)
      return QMK_ERR_NO_DEVICE;
    void* sym = nullptr;
    if (hipGetSymbolAddress(&sym, HIP_SYMBOL(g_status)) != hipSuccess) return QMK_ERR_NO_DEVICE;
    if (hipMemset(sym, 0, sizeof(int32_t) * kStatusWords) != hipSuccess) return QMK_ERR_NO_DEVICE;
    void* scratch_ptr = nullptr;
    if (hipGetSymbolAddress(&scratch_ptr, HIP_SYMBOL(scratch)) != hipSuccess || scratch_ptr == nullptr) return QMK_ERR_NO_DEVICE;
    d.cu_count = prop.multiProcessorCount;
    d.max_queues = per_cu * prop.multiProcessorCount;
    d.max_queues_batch = per_cu_batch * prop.multiProcessorCount;
    d.max_queues_batch_qwen3 = per_cu_batch3 * prop.multiProcessorCount;
    d.max_queues_moe = per_cu_moe * prop.multiProcessorCount;
    d.max_queues_moe_rows = per_cu_rows * prop.multiProcessorCount;
    int per_cu_dense_rows = 0, per_cu_dense_rows3 = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu_dense_rows, decode_megakernel_rows<rows::Llama1BRows>, kThreads, 0) != hipSuccess ||
        hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu_dense_rows3, decode_megakernel_rows<rows::Qwen3_1p7BRows>, kThreads, 0) != hipSuccess)
      return QMK_ERR_NO_DEVICE;
    d.max_queues_rows = (per_cu_dense_rows3 < per_cu_dense_rows ? per_cu_dense_rows3 : per_cu_dense_rows) * prop.multiProcessorCount;
    d.status = static_cast<int32_t*>(sym);
    d.scratch = static_cast<uint64_t*>(scratch_ptr);
    d.ready = true;
  }
  *out = &d;
  return QMK_OK;
}

}  // namespace qmk

using namespace qmk;

namespace {

// `static_scratch`: the workspace is the library's own array of the current device instead of
// a->workspace (qmk_decode_step_static).
template <class M>
int decode_step(const QmkArgs* a, bool static_scratch) {
  const void* required[] = {a->instructions, a->hidden_states, a->q_post_rope, a->k_cache, a->v_cache, a->attn_out,
                            a->attn_lse_intermediates, a->attn_out_intermediates, a->silu_out, a->logits,
                            a->attn_norm_weights, a->qkv_weights, a->rope_cos, a->rope_sin, a->o_proj_weights,
                            a->mlp_norm_weights, a->up_proj_weights, a->gate_proj_weights, a->down_proj_weights,
                            a->lm_head_norm_weights, a->lm_head_weights, a->barriers};
  for (const void* ptr : required)
    if (ptr == nullptr) return QMK_ERR_NULL_ARG;
  if (M::QK_NORM && (a->qkv_raw == nullptr || a->q_norm_weights == nullptr || a->k_norm_weights == nullptr)) return QMK_ERR_NULL_ARG;
  if (a->num_queues < 1 || a->num_insts < 0 || a->num_layers < 1 || a->num_layer_barriers < 8 ||
      a->barrier_slots < M::NQ + 2 * M::NKV || a->max_seq_len < 1 || a->max_splits < 1 || a->vocab_size < 1 ||
      a->rope_rows < 1)
    return QMK_ERR_SHAPE;
  if (a->pos_id < 0 || a->pos_id >= a->max_seq_len || a->pos_id >= a->rope_rows) return QMK_ERR_POSITION;
  if (a->flags & QMK_FLAG_XCD_COUNTERS) {
    const long layer_ints = static_cast<long>(a->num_layer_barriers) * a->barrier_slots;
    const long needed = static_cast<long>(kHierFirstRow) * a->barrier_slots + 2 * kHierEdges * kXcds * kLineInts;  // counter lines + flag lines
    const bool aligned = reinterpret_cast<uintptr_t>(a->barriers) % 128 == 0 && (layer_ints * 4) % 128 == 0 &&
                         (static_cast<long>(kHierFirstRow) * a->barrier_slots * 4) % 128 == 0;
    if (layer_ints < needed || !aligned) return QMK_ERR_SHAPE;
  }

  const bool sampling = a->token_out != nullptr || a->embed_tokens != nullptr;
  if (sampling && (a->token_out == nullptr || a->embed_tokens == nullptr)) return QMK_ERR_NULL_ARG;
  if ((a->flags & QMK_FLAG_TAGGED) || sampling) {
    if (static_scratch) {
      // What the array has room for: one candidate per queue, six bits of layer in a tag.
      if (qmk_workspace_bytes(static_cast<int>(a->model)) > sizeof(scratch)) return QMK_ERR_SCRATCH;
      if ((a->flags & QMK_FLAG_TAGGED) && a->num_layers > 63) return QMK_ERR_SCRATCH;
      if (sampling && a->num_queues > kMaxSamplingQueues) return QMK_ERR_SCRATCH;
      if (a->flags & QMK_FLAG_KEEP_BARRIERS) return QMK_ERR_SHAPE;
    } else {
      if (a->workspace == nullptr) return QMK_ERR_NULL_ARG;
      if ((a->flags & QMK_FLAG_KEEP_BARRIERS) || reinterpret_cast<uintptr_t>(a->workspace) % 128 != 0 ||
          a->workspace_bytes < qmk_workspace_bytes(static_cast<int>(a->model)))
        return QMK_ERR_SHAPE;
      if ((a->flags & QMK_FLAG_TAGGED) && a->num_layers > 63) return QMK_ERR_SHAPE;
      if (sampling && a->num_queues > kMaxSamplingQueues) return QMK_ERR_SHAPE;
    }
  }

  DeviceInfo* dev = nullptr;
  if (int rc = device_info(&dev); rc != QMK_OK) return rc;
  if (a->num_queues > dev->max_queues) return QMK_ERR_TOO_MANY_QUEUES;
  if (a->num_insts == 0) return QMK_OK;

  Params p{};
  p.instructions = a->instructions;
  p.hidden = static_cast<u16*>(a->hidden_states);
  p.q_post_rope = static_cast<u16*>(a->q_post_rope);
  p.k_cache = static_cast<u16*>(a->k_cache);
  p.v_cache = static_cast<u16*>(a->v_cache);
  p.attn_out = static_cast<u16*>(a->attn_out);
  p.attn_lse = a->attn_lse_intermediates;
  p.attn_partial = a->attn_out_intermediates;
  p.silu_out = static_cast<u16*>(a->silu_out);
  p.logits = static_cast<u16*>(a->logits);
  p.attn_norm = static_cast<const u16*>(a->attn_norm_weights);
  p.qkv_w = static_cast<const u16*>(a->qkv_weights);
  p.qkv_raw = static_cast<u16*>(a->qkv_raw);
  p.q_norm = static_cast<const u16*>(a->q_norm_weights);
  p.k_norm = static_cast<const u16*>(a->k_norm_weights);
  p.rope_cos = a->rope_cos;
  p.rope_sin = a->rope_sin;
  p.o_w = static_cast<const u16*>(a->o_proj_weights);
  p.mlp_norm = static_cast<const u16*>(a->mlp_norm_weights);
  p.up_w = static_cast<const u16*>(a->up_proj_weights);
  p.gate_w = static_cast<const u16*>(a->gate_proj_weights);
  p.down_w = static_cast<const u16*>(a->down_proj_weights);
  p.lm_norm = static_cast<const u16*>(a->lm_head_norm_weights);
  p.lm_w = static_cast<const u16*>(a->lm_head_weights);
  p.barriers = a->barriers;
  p.ws = static_scratch ? dev->scratch : static_cast<uint64_t*>(a->workspace);
  if (static_scratch) {
    std::lock_guard<std::mutex> lock(g_mutex);
    dev->static_in_use = true;
  }
  p.embed = static_cast<const u16*>(a->embed_tokens);
  p.token_out = reinterpret_cast<long long*>(a->token_out);
  p.timeline = a->timeline;
  p.status = dev->status;
  p.num_insts = a->num_insts;
  p.num_layers = a->num_layers;
  p.num_layer_barriers = a->num_layer_barriers;
  p.barrier_slots = a->barrier_slots;
  p.max_seq_len = a->max_seq_len;
  p.max_splits = a->max_splits;
  p.vocab_size = a->vocab_size;
  p.pos_id = a->pos_id;
  p.attn_scale = a->attn_scale;
  p.rms_norm_eps = a->rms_norm_eps;
  // Reference geometry: 16-row tiles everywhere, down projection in 2048-wide K slices.
  p.qkv_blocks_per_head = a->qkv_blocks_per_head > 0 ? a->qkv_blocks_per_head : M::D / 16;
  p.oproj_blocks = a->oproj_blocks > 0 ? a->oproj_blocks : M::H / 16;
  p.upgate_blocks_per_bucket = a->upgate_blocks_per_bucket > 0 ? a->upgate_blocks_per_bucket : 2048 / 16;
  p.down_arrivals = a->down_arrivals > 0 ? a->down_arrivals : (M::H / 16) * (M::F / 2048);
  p.spin_limit = a->spin_limit > 0 ? a->spin_limit : kDefaultSpinLimit;
  p.flags = a->flags | attention_lines_flag(a->flags, a->num_layer_barriers, a->barrier_slots, M::NKV);

  hipLaunchKernelGGL(decode_megakernel<M>, dim3(a->num_queues), dim3(kThreads), 0,
                     static_cast<hipStream_t>(a->stream), p);
  return hipGetLastError() == hipSuccess ? QMK_OK : QMK_ERR_LAUNCH;
}

}  // namespace

namespace {
int decode_step_any(const QmkArgs* a, bool static_scratch) {
  if (a == nullptr) return QMK_ERR_NULL_ARG;
  if (a->struct_size != sizeof(QmkArgs)) return QMK_ERR_ABI;
  switch (a->model) {
    case QMK_MODEL_LLAMA_3_2_1B: return decode_step<Llama1B>(a, static_scratch);
    case QMK_MODEL_QWEN3_1_7B: return decode_step<Qwen3_1p7B>(a, static_scratch);
    default: return QMK_ERR_MODEL;
  }
}
}  // namespace

extern "C" int qmk_decode_step(const QmkArgs* a) { return decode_step_any(a, false); }

// The same launch with the library's own workspace: no allocation anywhere on the way (the array
// lives in the code object; its address was looked up when the device was first used).
extern "C" int qmk_decode_step_static(const QmkArgs* a) { return decode_step_any(a, true); }

template <class M>
static int decode_step_batch(const QmkBatchArgs* a) {
  const void* required[] = {a->instructions, a->hidden_states, a->q_post_rope, a->k_cache, a->v_cache, a->attn_out,
                            a->attn_lse_intermediates, a->attn_out_intermediates, a->silu_out, a->logits,
                            a->attn_norm_weights, a->qkv_weights, a->rope_cos, a->rope_sin, a->o_proj_weights,
                            a->mlp_norm_weights, a->up_proj_weights, a->gate_proj_weights, a->down_proj_weights,
                            a->lm_head_norm_weights, a->lm_head_weights, a->barriers,
                            a->attn_rms_out, a->mlp_rms_out, a->lm_head_rms_out};
  for (const void* ptr : required)
    if (ptr == nullptr) return QMK_ERR_NULL_ARG;
  if (M::QK_NORM && (a->qkv_raw == nullptr || a->q_norm_weights == nullptr || a->k_norm_weights == nullptr)) return QMK_ERR_NULL_ARG;
  if (a->batch_size < 1 || a->batch_size > mb::kMaxBatch) return QMK_ERR_SHAPE;
  if (a->num_queues < 1 || a->num_insts < 0 || a->num_layers < 1 || a->num_layer_barriers < 10 ||
      a->barrier_slots < a->batch_size * (M::NQ + 2 * M::NKV) || a->max_seq_len < 1 || a->max_splits < 1 ||
      a->vocab_size < 1 || a->rope_rows < 1 || a->kv_block_size < 1 || a->oproj_blocks < 0 || a->down_blocks < 0)
    return QMK_ERR_SHAPE;
  if (a->flags & ~(QMK_FLAG_KEEP_BARRIERS | QMK_FLAG_XCD_COUNTERS)) return QMK_ERR_SHAPE;
  // eight sub-counters, a 128-byte line each, in the O-projection's, the up/gate's and the down projection's row
  if ((a->flags & QMK_FLAG_XCD_COUNTERS) && a->barrier_slots < kLineInts * mb::kSpread) return QMK_ERR_SHAPE;
  if (a->position_ids == nullptr && (a->pos_id < 0 || a->pos_id >= a->max_seq_len || a->pos_id >= a->rope_rows)) return QMK_ERR_POSITION;
  // the column window: all columns, or a part of them with counters that outlive the launch
  if (a->first_inst < 0 || a->inst_count < 0 || (a->inst_count == 0 && a->first_inst != 0) ||
      static_cast<long>(a->first_inst) + a->inst_count > a->num_insts)
    return QMK_ERR_SHAPE;
  const bool whole = a->inst_count == 0 || (a->first_inst == 0 && a->inst_count == a->num_insts);
  if (!whole && !(a->flags & QMK_FLAG_KEEP_BARRIERS)) return QMK_ERR_SHAPE;

  DeviceInfo* dev = nullptr;
  if (int rc = device_info(&dev); rc != QMK_OK) return rc;
  if (a->num_queues > (M::QK_NORM ? dev->max_queues_batch_qwen3 : dev->max_queues_batch)) return QMK_ERR_TOO_MANY_QUEUES;
  if (a->num_insts == 0) return QMK_OK;

  Params p{};
  p.instructions = a->instructions;
  p.hidden = static_cast<u16*>(a->hidden_states);
  p.q_post_rope = static_cast<u16*>(a->q_post_rope);
  p.k_cache = static_cast<u16*>(a->k_cache);
  p.v_cache = static_cast<u16*>(a->v_cache);
  p.attn_out = static_cast<u16*>(a->attn_out);
  p.attn_lse = a->attn_lse_intermediates;
  p.attn_partial = a->attn_out_intermediates;
  p.silu_out = static_cast<u16*>(a->silu_out);
  p.logits = static_cast<u16*>(a->logits);
  p.attn_norm = static_cast<const u16*>(a->attn_norm_weights);
  p.qkv_w = static_cast<const u16*>(a->qkv_weights);
  p.rope_cos = a->rope_cos;
  p.rope_sin = a->rope_sin;
  p.o_w = static_cast<const u16*>(a->o_proj_weights);
  p.mlp_norm = static_cast<const u16*>(a->mlp_norm_weights);
  p.up_w = static_cast<const u16*>(a->up_proj_weights);
  p.gate_w = static_cast<const u16*>(a->gate_proj_weights);
  p.down_w = static_cast<const u16*>(a->down_proj_weights);
  p.lm_norm = static_cast<const u16*>(a->lm_head_norm_weights);
  p.lm_w = static_cast<const u16*>(a->lm_head_weights);
  p.barriers = a->barriers;
  p.timeline = a->timeline;
  p.status = dev->status;
  p.num_insts = a->num_insts;
  p.first_inst = a->first_inst;
  p.end_inst = whole ? a->num_insts : a->first_inst + a->inst_count;
  p.num_layers = a->num_layers;
  p.num_layer_barriers = a->num_layer_barriers;
  p.barrier_slots = a->barrier_slots;
  p.max_seq_len = a->max_seq_len;
  p.max_splits = a->max_splits;
  p.vocab_size = a->vocab_size;
  p.pos_id = a->pos_id;
  p.attn_scale = a->attn_scale;
  p.rms_norm_eps = a->rms_norm_eps;
  p.spin_limit = a->spin_limit > 0 ? a->spin_limit : kDefaultSpinLimit;
  p.flags = a->flags;
  p.oproj_blocks = a->oproj_blocks > 0 ? a->oproj_blocks : M::H / mb::kTile;
  p.down_arrivals = a->down_blocks > 0 ? a->down_blocks : M::H / mb::kTile;
  p.batch = a->batch_size;
  p.kv_block = a->kv_block_size;
  p.position_ids = a->position_ids;
  p.active_mask = a->active_mask;
  p.partial_valid = a->attn_partial_valid;
  p.attn_rms_out = static_cast<u16*>(a->attn_rms_out);
  p.mlp_rms_out = static_cast<u16*>(a->mlp_rms_out);
  p.lm_rms_out = static_cast<u16*>(a->lm_head_rms_out);
  p.rope_rows = a->rope_rows;
  p.qkv_raw = static_cast<u16*>(a->qkv_raw);
  p.q_norm = static_cast<const u16*>(a->q_norm_weights);
  p.k_norm = static_cast<const u16*>(a->k_norm_weights);

  hipLaunchKernelGGL(decode_megakernel_batch<M>, dim3(a->num_queues), dim3(kThreads), 0, static_cast<hipStream_t>(a->stream), p);
  return hipGetLastError() == hipSuccess ? QMK_OK : QMK_ERR_LAUNCH;
}

extern "C" int qmk_decode_step_batch(const QmkBatchArgs* a) {
  if (a == nullptr) return QMK_ERR_NULL_ARG;
  if (a->struct_size != sizeof(QmkBatchArgs)) return QMK_ERR_ABI;
  if (a->model == QMK_MODEL_LLAMA_3_2_1B) return decode_step_batch<Llama1B>(a);
  if (a->model == QMK_MODEL_QWEN3_1_7B) return decode_step_batch<Qwen3_1p7B>(a);
  return QMK_ERR_MODEL;
}

extern "C" uint64_t qmk_moe_workspace_bytes(int top_k, int shared_k_slices) {
  if (top_k < 1 || top_k > moe::kMaxTopK || shared_k_slices < 0 || shared_k_slices > 16) return 0;   // 0 slices: no shared expert
  const uint64_t shared = static_cast<uint64_t>(shared_k_slices) * QwenMoeA2_7B::H * sizeof(u16);
  // the down projections' terms, the gate scalar's line, then the tagged units of the residual stream and q/k/v
  static_assert(QwenMoeA2_7B::H <= 2048 && Qwen3MoeA3B::H <= 2048 && moe::kMaxTopK <= 8 && moe::kMaxK <= 2048, "the tagged MoE regions");
  return ((shared + 127) / 128) * 128 + static_cast<uint64_t>(top_k) * QwenMoeA2_7B::H * sizeof(float) + 128 +
         static_cast<uint64_t>(kWsMoeUnits) * sizeof(uint64_t);
}

namespace {

template <class M>
void fill_moe_params(const QmkMoeArgs* a, DeviceInfo* dev, Params& p);

// Rows per tile of opcode 1 that QmkMoeArgs may name: the powers of two from 2 (one RoPE pair) to 16; 0 stands for 16.
static bool qkv_tile_ok(int tile) { return tile == 0 || tile == 2 || tile == 4 || tile == 8 || tile == 16; }

template <class M>
int decode_step_moe(const QmkMoeArgs* a) {
  const void* required[] = {a->instructions, a->hidden_states, a->normed_hidden_states, a->q_post_rope, a->k_cache, a->v_cache,
                            a->attn_out, a->attn_lse_intermediates, a->attn_out_intermediates, a->silu_out, a->logits,
                            a->attn_norm_weights, a->qkv_weights, a->rope_cos, a->rope_sin, a->o_proj_weights,
                            a->mlp_norm_weights, a->lm_head_norm_weights, a->lm_head_weights, a->router_weights,
                            a->router_logits_buf, a->expert_indices, a->expert_weights, a->expert_gate_up_proj_weights,
                            a->expert_down_proj_weights, a->routed_silu_buffer, a->routed_out_f32, a->barriers, a->workspace};
  for (const void* ptr : required)
    if (ptr == nullptr) return QMK_ERR_NULL_ARG;
  if (M::QKV_BIAS && a->qkv_bias == nullptr) return QMK_ERR_NULL_ARG;
  if (M::QK_NORM && (a->qkv_raw == nullptr || a->q_norm_weights == nullptr || a->k_norm_weights == nullptr)) return QMK_ERR_NULL_ARG;
  const bool shared = a->shared_ffn != 0;   // a model without a shared expert: shared_ffn = shared_k_slices = 0, no opcodes 10/11
  if (shared && (a->shared_expert_gate_proj_weights == nullptr || a->shared_expert_up_proj_weights == nullptr ||
                 a->shared_expert_down_proj_weights == nullptr || a->shared_expert_silu_out == nullptr || a->shared_out == nullptr ||
                 a->shared_expert_gate_weights == nullptr))
    return QMK_ERR_NULL_ARG;
  if (a->num_queues < 1 || a->num_insts < 0 || a->num_layers < 1 || a->num_layer_barriers < 15 ||
      a->barrier_slots < M::H / 16 || a->barrier_slots < M::NQ + 2 * M::NKV || a->max_seq_len < 1 || a->max_splits < 1 ||
      a->vocab_size < 1 || a->rope_rows < 1)
    return QMK_ERR_SHAPE;
  if (a->num_experts < 1 || a->num_experts > moe::kMaxExperts || a->top_k < 1 || a->top_k > moe::kMaxTopK || a->top_k > a->num_experts ||
      a->moe_ffn < 16 || a->moe_ffn % 16 || a->moe_ffn > moe::kMaxK)
    return QMK_ERR_SHAPE;
  if (shared ? (a->shared_ffn < 16 || a->shared_ffn % 16 || a->shared_k_slices < 1 || a->shared_k_slices > 16)
             : (a->shared_ffn != 0 || a->shared_k_slices != 0))
    return QMK_ERR_SHAPE;
  const int routed_tile = a->routed_upgate_tile == 0 ? moe::kTile : a->routed_upgate_tile;
  if ((routed_tile != 8 && routed_tile != 16) || a->moe_ffn % routed_tile) return QMK_ERR_SHAPE;
  if (a->norm_topk_prob != 0 && a->norm_topk_prob != 1) return QMK_ERR_SHAPE;
  const int oproj_tile = a->oproj_tile == 0 ? moe::kTile : a->oproj_tile;
  if ((oproj_tile != 8 && oproj_tile != 16) || (a->local_routing != 0 && a->local_routing != 1)) return QMK_ERR_SHAPE;
  if (!qkv_tile_ok(a->qkv_tile) || a->reserved0 != 0) return QMK_ERR_SHAPE;
  if (a->flags & ~(QMK_FLAG_KEEP_BARRIERS | QMK_FLAG_TAGGED)) return QMK_ERR_SHAPE;
  // tagged units carry the launch count, which the retiring launch advances, and six bits of layer
  if ((a->flags & QMK_FLAG_TAGGED) && ((a->flags & QMK_FLAG_KEEP_BARRIERS) || a->num_layers > 63)) return QMK_ERR_SHAPE;
  if (a->pos_id < 0 || a->pos_id >= a->max_seq_len || a->pos_id >= a->rope_rows) return QMK_ERR_POSITION;
  if (reinterpret_cast<uintptr_t>(a->workspace) % 128 != 0 || a->workspace_bytes < qmk_moe_workspace_bytes(a->top_k, a->shared_k_slices))
    return QMK_ERR_SHAPE;

  DeviceInfo* dev = nullptr;
  if (int rc = device_info(&dev); rc != QMK_OK) return rc;
  if (a->num_queues > dev->max_queues_moe) return QMK_ERR_TOO_MANY_QUEUES;
  if (a->num_insts == 0) return QMK_OK;

  Params p{};
  fill_moe_params<M>(a, dev, p);
  p.flags |= attention_lines_flag(a->flags, a->num_layer_barriers, a->barrier_slots, M::NKV);
  const uint64_t shared_bytes = ((static_cast<uint64_t>(a->shared_k_slices) * M::H * sizeof(u16) + 127) / 128) * 128;
  p.shared_parts = static_cast<u16*>(a->workspace);
  p.routed_parts = reinterpret_cast<float*>(static_cast<char*>(a->workspace) + shared_bytes);
  p.shared_gate = p.routed_parts + static_cast<size_t>(a->top_k) * M::H;
  p.ws = reinterpret_cast<uint64_t*>(reinterpret_cast<char*>(p.shared_gate) + 128);

  hipLaunchKernelGGL(decode_megakernel_moe<M>, dim3(a->num_queues), dim3(kThreads), 0, static_cast<hipStream_t>(a->stream), p);
  return hipGetLastError() == hipSuccess ? QMK_OK : QMK_ERR_LAUNCH;
}

// The fields of Params that come straight from a QmkMoeArgs (everything but the workspace's regions).
template <class M>
void fill_moe_params(const QmkMoeArgs* a, DeviceInfo* dev, Params& p) {
  const int routed_tile = a->routed_upgate_tile == 0 ? moe::kTile : a->routed_upgate_tile;
  const int oproj_tile = a->oproj_tile == 0 ? moe::kTile : a->oproj_tile;
  p.instructions = a->instructions;
  p.hidden = static_cast<u16*>(a->hidden_states);
  p.q_post_rope = static_cast<u16*>(a->q_post_rope);
  p.k_cache = static_cast<u16*>(a->k_cache);
  p.v_cache = static_cast<u16*>(a->v_cache);
  p.attn_out = static_cast<u16*>(a->attn_out);
  p.attn_lse = a->attn_lse_intermediates;
  p.attn_partial = a->attn_out_intermediates;
  p.silu_out = static_cast<u16*>(a->silu_out);
  p.logits = static_cast<u16*>(a->logits);
  p.attn_norm = static_cast<const u16*>(a->attn_norm_weights);
  p.qkv_w = static_cast<const u16*>(a->qkv_weights);
  p.qkv_bias = static_cast<const u16*>(a->qkv_bias);
  p.qkv_raw = static_cast<u16*>(a->qkv_raw);
  p.q_norm = static_cast<const u16*>(a->q_norm_weights);
  p.k_norm = static_cast<const u16*>(a->k_norm_weights);
  p.rope_cos = a->rope_cos;
  p.rope_sin = a->rope_sin;
  p.o_w = static_cast<const u16*>(a->o_proj_weights);
  p.mlp_norm = static_cast<const u16*>(a->mlp_norm_weights);
  p.lm_norm = static_cast<const u16*>(a->lm_head_norm_weights);
  p.lm_w = static_cast<const u16*>(a->lm_head_weights);
  p.barriers = a->barriers;
  p.timeline = a->timeline;
  p.status = dev->status;
  p.num_insts = a->num_insts;
  p.num_layers = a->num_layers;
  p.num_layer_barriers = a->num_layer_barriers;
  p.barrier_slots = a->barrier_slots;
  p.max_seq_len = a->max_seq_len;
  p.max_splits = a->max_splits;
  p.vocab_size = a->vocab_size;
  p.pos_id = a->pos_id;
  p.attn_scale = a->attn_scale;
  p.rms_norm_eps = a->rms_norm_eps;
  p.qkv_blocks_per_head = M::D / (a->qkv_tile == 0 ? moe::kTile : a->qkv_tile);
  p.oproj_blocks = M::H / oproj_tile;
  p.down_arrivals = M::H / 16;           // what completes a layer here: the combine step's tiles
  p.spin_limit = a->spin_limit > 0 ? a->spin_limit : kDefaultSpinLimit;
  p.flags = a->flags;
  p.router_w = static_cast<const u16*>(a->router_weights);
  p.router_logits = a->router_logits_buf;
  p.expert_indices = reinterpret_cast<long long*>(a->expert_indices);
  p.expert_weights = a->expert_weights;
  p.normed_hidden = static_cast<u16*>(a->normed_hidden_states);
  p.shared_gate_w = static_cast<const u16*>(a->shared_expert_gate_proj_weights);
  p.shared_up_w = static_cast<const u16*>(a->shared_expert_up_proj_weights);
  p.shared_down_w = static_cast<const u16*>(a->shared_expert_down_proj_weights);
  p.shared_scale_w = static_cast<const u16*>(a->shared_expert_gate_weights);
  p.shared_silu = static_cast<u16*>(a->shared_expert_silu_out);
  p.shared_out = static_cast<u16*>(a->shared_out);
  p.expert_gate_up_w = static_cast<const u16*>(a->expert_gate_up_proj_weights);
  p.expert_down_w = static_cast<const u16*>(a->expert_down_proj_weights);
  p.routed_silu = static_cast<u16*>(a->routed_silu_buffer);
  p.routed_out_f32 = a->routed_out_f32;
  p.routed_out = static_cast<u16*>(a->routed_out);
  p.num_experts = a->num_experts;
  p.top_k = a->top_k;
  p.shared_ffn = a->shared_ffn;
  p.moe_ffn = a->moe_ffn;
  p.shared_k_slices = a->shared_k_slices;
  p.norm_topk = a->norm_topk_prob;
  p.routed_tile = routed_tile;
  p.local_routing = a->local_routing;
}

// Units from one row's tagged workspace to the next in a launch of several rows: a batch-1 launch's units, in whole lines.
constexpr int kWsRowUnits = ((kWsMoeUnits + 15) / 16) * 16 + kRowAttentionUnits;   // ... and the row's attention lines

template <class M>
int decode_step_moe_rows(const QmkMoeRowsArgs* r) {
  const QmkMoeArgs* a = &r->step;
  const int B = r->batch_size;
  if (B < 1 || B > rows::kMaxRows) return QMK_ERR_SHAPE;
  const void* required[] = {a->instructions, a->hidden_states, a->normed_hidden_states, a->q_post_rope, a->k_cache, a->v_cache,
                            a->attn_out, a->attn_lse_intermediates, a->attn_out_intermediates, a->silu_out, a->logits,
                            a->attn_norm_weights, a->qkv_weights, a->rope_cos, a->rope_sin, a->o_proj_weights,
                            a->mlp_norm_weights, a->lm_head_norm_weights, a->lm_head_weights, a->router_weights,
                            a->router_logits_buf, a->expert_indices, a->expert_weights, a->expert_gate_up_proj_weights,
                            a->expert_down_proj_weights, a->routed_silu_buffer, a->routed_out_f32, a->routed_out, a->barriers,
                            a->workspace, r->position_ids};
  for (const void* ptr : required)
    if (ptr == nullptr) return QMK_ERR_NULL_ARG;
  if (M::QKV_BIAS && a->qkv_bias == nullptr) return QMK_ERR_NULL_ARG;
  if (M::QK_NORM && (a->qkv_raw == nullptr || a->q_norm_weights == nullptr || a->k_norm_weights == nullptr)) return QMK_ERR_NULL_ARG;
  if (a->shared_ffn != 0 || a->shared_k_slices != 0) return QMK_ERR_SHAPE;   // the committing stream has no shared expert
  if (a->num_queues < 1 || a->num_insts < 0 || a->num_layers < 1 || a->num_layers > 63 || a->num_layer_barriers < 15 ||
      a->barrier_slots < B * M::NQ || a->max_seq_len < 1 || a->max_splits < 1 || a->vocab_size < 1 || a->rope_rows < 1)
    return QMK_ERR_SHAPE;
  // a wave per expert slot of a row's softmax, the rows side by side: rows x (experts in whole waves) threads
  if (a->num_experts < 1 || a->num_experts > moe::kMaxExperts || ((a->num_experts + kWaveSize - 1) / kWaveSize) * kWaveSize * B > kThreads ||
      a->top_k < 1 || a->top_k > moe::kMaxTopK || a->top_k > a->num_experts || a->moe_ffn < 16 || a->moe_ffn % 16 || a->moe_ffn > 1024)
    return QMK_ERR_SHAPE;
  if (a->norm_topk_prob != 0 && a->norm_topk_prob != 1) return QMK_ERR_SHAPE;
  const int oproj_tile = a->oproj_tile == 0 ? moe::kTile : a->oproj_tile;
  if (oproj_tile != 8 && oproj_tile != 16) return QMK_ERR_SHAPE;
  if (!qkv_tile_ok(a->qkv_tile) || a->reserved0 != 0) return QMK_ERR_SHAPE;
  if (a->flags != QMK_FLAG_TAGGED) return QMK_ERR_SHAPE;   // tagged hand-over, self-clearing counters: nothing else is built
  if (reinterpret_cast<uintptr_t>(a->workspace) % 128 != 0 || a->workspace_bytes < qmk_moe_rows_workspace_bytes(B)) return QMK_ERR_SHAPE;

  DeviceInfo* dev = nullptr;
  if (int rc = device_info(&dev); rc != QMK_OK) return rc;
  if (a->num_queues > dev->max_queues_moe_rows) return QMK_ERR_TOO_MANY_QUEUES;
  if (a->num_insts == 0) return QMK_OK;

  Params p{};
  fill_moe_params<M>(a, dev, p);
  p.local_routing = 1;
  p.flags |= kFlagRowAttentionLines;
  p.ws = static_cast<uint64_t*>(a->workspace);
  p.ws_row_units = kWsRowUnits;
  p.batch = B;
  p.position_ids = r->position_ids;
  p.distinct_out = r->distinct_experts;
  p.rope_rows = a->rope_rows;
  p.kv_row_tokens = a->num_layers * a->max_seq_len;   // caches [B, L, 1, S, Hkv, D]
  p.kv_layer_tokens = a->max_seq_len;
  p.pos_id = 0;
  hipLaunchKernelGGL(decode_megakernel_moe_rows<M>, dim3(a->num_queues), dim3(kThreads), 0, static_cast<hipStream_t>(a->stream), p);
  return hipGetLastError() == hipSuccess ? QMK_OK : QMK_ERR_LAUNCH;
}

}  // namespace

extern "C" int qmk_decode_step_moe(const QmkMoeArgs* a) {
  if (a == nullptr) return QMK_ERR_NULL_ARG;
  if (a->struct_size != sizeof(QmkMoeArgs)) return QMK_ERR_ABI;
  switch (a->model) {
    case QMK_MODEL_QWEN1_5_MOE_A2_7B: return decode_step_moe<QwenMoeA2_7B>(a);
    case QMK_MODEL_QWEN3_30B_A3B: return decode_step_moe<Qwen3MoeA3B>(a);
    default: return QMK_ERR_MODEL;
  }
}

// Units from one row's tagged workspace to the next in a dense launch of several rows.
constexpr int kWsDenseRowUnits = ((kWsUnits + 15) / 16) * 16 + kRowAttentionUnits;   // ... and the row's attention lines

extern "C" uint64_t qmk_rows_workspace_bytes(int batch_size) {
  if (batch_size < 1 || batch_size > rows::kMaxRows) return 0;
  return static_cast<uint64_t>(batch_size) * kWsDenseRowUnits * sizeof(uint64_t);
}

template <class M>
static int decode_step_rows(const QmkRowsArgs* r) {
  const QmkBatchArgs* a = &r->step;
  const int B = a->batch_size;
  if (B < 1 || B > rows::kMaxRows) return QMK_ERR_SHAPE;
  const void* required[] = {a->instructions, a->hidden_states, a->q_post_rope, a->k_cache, a->v_cache, a->attn_out,
                            a->attn_lse_intermediates, a->attn_out_intermediates, a->silu_out, a->logits,
                            a->attn_norm_weights, a->qkv_weights, a->rope_cos, a->rope_sin, a->o_proj_weights,
                            a->mlp_norm_weights, a->up_proj_weights, a->gate_proj_weights, a->down_proj_weights,
                            a->lm_head_norm_weights, a->lm_head_weights, a->barriers, r->workspace};
  for (const void* ptr : required)
    if (ptr == nullptr) return QMK_ERR_NULL_ARG;
  if (M::QK_NORM && (a->qkv_raw == nullptr || a->q_norm_weights == nullptr || a->k_norm_weights == nullptr)) return QMK_ERR_NULL_ARG;
  if (a->num_queues < 1 || a->num_insts < 0 || a->num_layers < 1 || a->num_layers > 63 || a->num_layer_barriers < 8 ||
      a->barrier_slots < B * M::NQ || a->max_seq_len < 1 || a->max_splits < 1 || a->vocab_size < 1 || a->rope_rows < 1)
    return QMK_ERR_SHAPE;
  if (a->flags != 0 || a->first_inst != 0 || a->inst_count != 0) return QMK_ERR_SHAPE;   // tagged hand-over and self-clearing counters always: whole steps only
  if (a->position_ids == nullptr && (a->pos_id < 0 || a->pos_id >= a->max_seq_len || a->pos_id >= a->rope_rows)) return QMK_ERR_POSITION;
  if (reinterpret_cast<uintptr_t>(r->workspace) % 128 != 0 || r->workspace_bytes < qmk_rows_workspace_bytes(B)) return QMK_ERR_SHAPE;

  DeviceInfo* dev = nullptr;
  if (int rc = device_info(&dev); rc != QMK_OK) return rc;
  if (a->num_queues > dev->max_queues_rows) return QMK_ERR_TOO_MANY_QUEUES;
  if (a->num_insts == 0) return QMK_OK;

  Params p{};
  p.instructions = a->instructions;
  p.hidden = static_cast<u16*>(a->hidden_states);
  p.q_post_rope = static_cast<u16*>(a->q_post_rope);
  p.k_cache = static_cast<u16*>(a->k_cache);
  p.v_cache = static_cast<u16*>(a->v_cache);
  p.attn_out = static_cast<u16*>(a->attn_out);
  p.attn_lse = a->attn_lse_intermediates;
  p.attn_partial = a->attn_out_intermediates;
  p.silu_out = static_cast<u16*>(a->silu_out);
  p.logits = static_cast<u16*>(a->logits);
  p.attn_norm = static_cast<const u16*>(a->attn_norm_weights);
  p.qkv_w = static_cast<const u16*>(a->qkv_weights);
  p.qkv_raw = static_cast<u16*>(a->qkv_raw);
  p.q_norm = static_cast<const u16*>(a->q_norm_weights);
  p.k_norm = static_cast<const u16*>(a->k_norm_weights);
  p.rope_cos = a->rope_cos;
  p.rope_sin = a->rope_sin;
  p.o_w = static_cast<const u16*>(a->o_proj_weights);
  p.mlp_norm = static_cast<const u16*>(a->mlp_norm_weights);
  p.up_w = static_cast<const u16*>(a->up_proj_weights);
  p.gate_w = static_cast<const u16*>(a->gate_proj_weights);
  p.down_w = static_cast<const u16*>(a->down_proj_weights);
  p.lm_norm = static_cast<const u16*>(a->lm_head_norm_weights);
  p.lm_w = static_cast<const u16*>(a->lm_head_weights);
  p.barriers = a->barriers;
  p.ws = static_cast<uint64_t*>(r->workspace);
  p.ws_row_units = kWsDenseRowUnits;
  p.timeline = a->timeline;
  p.status = dev->status;
  p.num_insts = a->num_insts;
  p.num_layers = a->num_layers;
  p.num_layer_barriers = a->num_layer_barriers;
  p.barrier_slots = a->barrier_slots;
  p.max_seq_len = a->max_seq_len;
  p.max_splits = a->max_splits;
  p.vocab_size = a->vocab_size;
  p.pos_id = a->pos_id;
  p.attn_scale = a->attn_scale;
  p.rms_norm_eps = a->rms_norm_eps;
  p.qkv_blocks_per_head = r->qkv_blocks_per_head > 0 ? r->qkv_blocks_per_head : M::D / 16;
  p.spin_limit = a->spin_limit > 0 ? a->spin_limit : kDefaultSpinLimit;
  p.flags = QMK_FLAG_TAGGED | kFlagRowAttentionLines;
  p.batch = B;
  p.position_ids = a->position_ids;
  p.active_mask = a->active_mask;
  p.rope_rows = a->rope_rows;
  p.kv_row_tokens = a->max_seq_len;            // caches [L, B, S, Hkv, D]
  p.kv_layer_tokens = B * a->max_seq_len;
  hipLaunchKernelGGL(decode_megakernel_rows<M>, dim3(a->num_queues), dim3(kThreads), 0, static_cast<hipStream_t>(a->stream), p);
  return hipGetLastError() == hipSuccess ? QMK_OK : QMK_ERR_LAUNCH;
}

extern "C" int qmk_decode_step_rows(const QmkRowsArgs* r) {
  if (r == nullptr) return QMK_ERR_NULL_ARG;
  if (r->struct_size != sizeof(QmkRowsArgs) || r->step.struct_size != sizeof(QmkBatchArgs)) return QMK_ERR_ABI;
  // the ops compiled for the smallest row count that holds the batch (same LDS and registers at every count: the
  // occupancy found for four holds)
  const int B = r->step.batch_size;
  if (r->step.model == QMK_MODEL_LLAMA_3_2_1B)
    return B <= 2 ? decode_step_rows<rows::Llama1BRowsN<2>>(r) : (B == 3 ? decode_step_rows<rows::Llama1BRowsN<3>>(r) : decode_step_rows<rows::Llama1BRows>(r));
  if (r->step.model == QMK_MODEL_QWEN3_1_7B)
    return B <= 2 ? decode_step_rows<rows::Qwen3_1p7BRowsN<2>>(r) : (B == 3 ? decode_step_rows<rows::Qwen3_1p7BRowsN<3>>(r) : decode_step_rows<rows::Qwen3_1p7BRows>(r));
  return QMK_ERR_MODEL;
}

extern "C" uint64_t qmk_moe_rows_workspace_bytes(int batch_size) {
  if (batch_size < 1 || batch_size > rows::kMaxRows) return 0;
  return static_cast<uint64_t>(batch_size) * kWsRowUnits * sizeof(uint64_t);
}

extern "C" int qmk_decode_step_moe_rows(const QmkMoeRowsArgs* r) {
  if (r == nullptr) return QMK_ERR_NULL_ARG;
  if (r->struct_size != sizeof(QmkMoeRowsArgs) || r->step.struct_size != sizeof(QmkMoeArgs)) return QMK_ERR_ABI;
  switch (r->step.model) {
    case QMK_MODEL_QWEN3_30B_A3B: return decode_step_moe_rows<Qwen3MoeA3B>(r);
    default: return QMK_ERR_MODEL;
  }
}

extern "C" uint64_t qmk_workspace_bytes(int model) {
  return (model == QMK_MODEL_LLAMA_3_2_1B || model == QMK_MODEL_QWEN3_1_7B) ? static_cast<uint64_t>(kWsUnits) * sizeof(uint64_t) : 0;
}

extern "C" int qmk_query(int what) {
  switch (what) {
    case QMK_QUERY_ABI_VERSION: return QMK_ABI_VERSION;
    case QMK_QUERY_THREADS: return kThreads;
    case QMK_QUERY_LDS_BYTES: return static_cast<int>(sizeof(Smem<Llama1B>));
    case QMK_QUERY_INSTRUCTION_WORDS: return kInstWords;
    case QMK_QUERY_MAX_PARTIALS: return kMaxPartials;
    default: break;
  }
  DeviceInfo* dev = nullptr;
  if (device_info(&dev) != QMK_OK) return -QMK_ERR_NO_DEVICE;
  if (what == QMK_QUERY_CU_COUNT) return dev->cu_count;
  if (what == QMK_QUERY_MAX_QUEUES) return dev->max_queues;
  return -QMK_ERR_SHAPE;
}

extern "C" int qmk_status_fetch(void* stream, int32_t detail[4]) {
  DeviceInfo* dev = nullptr;
  if (int rc = device_info(&dev); rc != QMK_OK) return rc;
  if (hipStreamSynchronize(static_cast<hipStream_t>(stream)) != hipSuccess) return QMK_ERR_NO_DEVICE;
  int32_t host[kStatusWords] = {0};
  if (hipMemcpy(host, dev->status, sizeof(host), hipMemcpyDeviceToHost) != hipSuccess) return QMK_ERR_NO_DEVICE;
  if (detail != nullptr)
    for (int i = 0; i < 4; ++i) detail[i] = host[1 + i];
  bool static_used;
  {
    std::lock_guard<std::mutex> lock(g_mutex);
    static_used = dev->static_in_use;
    dev->static_in_use = false;
  }
  if (host[0] != 0) {
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (hipMemsetAsync(dev->status, 0, sizeof(host), st) != hipSuccess) return QMK_ERR_NO_DEVICE;
    // Units of the aborted step must not pass for the next one's (the launch count did not advance).  Only when a
    // launch behind the last fetch used the library's own array, and on the caller's stream: a launch of another
    // route on another stream has a workspace of its own and is not disturbed.
    if (static_used && hipMemsetAsync(dev->scratch, 0, sizeof(scratch), st) != hipSuccess) return QMK_ERR_NO_DEVICE;
    if (hipStreamSynchronize(st) != hipSuccess) return QMK_ERR_NO_DEVICE;
  }
  return host[0];
}

extern "C" const char* qmk_error_string(int code) {
  switch (code) {
    case QMK_OK: return "ok";
    case QMK_ERR_NULL_ARG: return "null argument";
    case QMK_ERR_ABI: return "QmkArgs.struct_size does not match the library";
    case QMK_ERR_SHAPE: return "dimension out of range";
    case QMK_ERR_POSITION: return "pos_id outside the KV cache or RoPE table";
    case QMK_ERR_TOO_MANY_QUEUES: return "more instruction queues than co-resident workgroups";
    case QMK_ERR_NO_DEVICE: return "no usable HIP device";
    case QMK_ERR_LAUNCH: return "kernel launch failed";
    case QMK_ERR_MODEL: return "unknown model id";
    case QMK_ERR_SCRATCH: return "launch needs more than the library's static scratch array holds (queues > 1024 with token_out, layers > 63 with QMK_FLAG_TAGGED)";
    case QMK_DEV_BAD_OPCODE: return "device: unknown opcode";
    case QMK_DEV_BAD_OPERAND: return "device: instruction operand out of bounds";
    case QMK_DEV_WAIT_TIMEOUT: return "device: counter wait ran out of polls";
    default: return "unknown code";
  }
}
