// Opcodes 8-14 of the MoE decode route (batch 1) as workgroup-wide device functions for gfx950, and
// the layer geometry they are compiled for.  Opcodes 1-4 and 7 are the dense route's (qmk_ops.h), with
// the QKV bias added in the projection's epilogue.
//
// Semantics follow the reference's instruction VM, which is also what its kernel does
// (qimeng_megakernel/models/LLM/qwen/qwen1_5_moe_a2_7b/A100/single_batch/decode_schedule/instructions/
// python_vm.py:331-530; decode_kernel/router_softmax_topk.cu, moe_combine_commit.cu): fp32 router logits,
// softmax and top-k without renormalisation; silu(gate)*up evaluated in fp32 on the bf16-rounded GEMV
// results with one rounding; the shared down projection split along K with bf16 partial sums; routed
// contributions bf16(dot) * weight in fp32; hidden = bf16(hidden + routed + sigmoid(gate) * shared).
//
// Where the VM accumulates in place (shared_out over the K slices, routed_out_f32 over the expert
// slots), concurrent workgroups would add in arrival order, and neither bf16 nor fp32 addition is
// associative.  Here every producer leaves its term in a slot of its own in the caller's workspace and
// the combine step adds the terms in the VM's order: same bits as the VM, every run.
#pragma once

#include "qmk_ops.h"

namespace qmk {

// Qwen1.5-MoE-A2.7B layer geometry.  Expert count, top-k and the two FFN widths are launch parameters.
struct QwenMoeA2_7B {
  static constexpr int H = 2048;
  static constexpr int F = 8192;      // size of the LDS activation vector: >= every FFN width and H
  static constexpr int D = 128;
  static constexpr int NQ = 16;
  static constexpr int NKV = 16;
  static constexpr int GQA = NQ / NKV;
  static constexpr int QKV = (NQ + 2 * NKV) * D;
  static constexpr int AW = NQ * D;
  static constexpr int KV_BLOCK = 16;
  static constexpr int CARRY_ROWS = 0;
  static constexpr int PARK_ROWS = 0;
  static constexpr bool CARRY_AFTER_ATTENTION = false;
  static constexpr bool QK_NORM = false;
  static constexpr bool QKV_BIAS = true;
  static constexpr int REDUCE_HEADS = 4;   // attn_reduction_size of the route (model_config.py:27)
  static constexpr int PREV_ROW = 13;      // a layer is complete when its combine step is
  static constexpr int UPGATE_OUTPUTS_IN_FLIGHT = 4;   // per wave, in the expert up/gate ops (2 measured the same here)
};

// Qwen3-30B-A3B layer geometry: 32 query heads over 4 KV heads of 128 (the attention output is twice as
// wide as the residual stream), the Qwen3 op set's attention (opcode 1 leaves the raw QKV vector, the
// split-KV prologue applies the per-head RMSNorm of q and k and RoPE; no QKV bias) in front of the MoE
// block.  Expert count, top-k, FFN width, the absence of a shared expert and the renormalisation of the
// top-k weights are launch parameters.
struct Qwen3MoeA3B {
  static constexpr int H = 2048;
  static constexpr int F = 8192;      // size of the LDS activation vector: >= AW, every FFN width and H
  static constexpr int D = 128;
  static constexpr int NQ = 32;
  static constexpr int NKV = 4;
  static constexpr int GQA = NQ / NKV;
  static constexpr int QKV = (NQ + 2 * NKV) * D;
  static constexpr int AW = NQ * D;
  static constexpr int KV_BLOCK = 16;
  static constexpr int CARRY_ROWS = 0;
  static constexpr int PARK_ROWS = 0;
  static constexpr bool CARRY_AFTER_ATTENTION = false;
  static constexpr bool QK_NORM = true;
  static constexpr bool QKV_BIAS = false;
  static constexpr int REDUCE_HEADS = GQA;
  static constexpr int PREV_ROW = 13;
  // One output (two rows) per wave in flight: a queue has 24 outputs of a phase, and with all of a wave's rows
  // requested at once the hand-overs behind them wait for the whole burst (measured: 395 against 381 tok/s with 4).
  static constexpr int UPGATE_OUTPUTS_IN_FLIGHT = 1;
};

namespace moe {

enum Opcode {
  OP_ROUTER = 8,
  OP_TOPK = 9,
  OP_SHARED_UPGATE = 10,
  OP_SHARED_DOWN = 11,
  OP_ROUTED_UPGATE = 12,
  OP_ROUTED_DOWN = 13,
  OP_COMBINE = 14,
};
constexpr int ROW_ROUTER = 7, ROW_TOPK = 8, ROW_SHARED_UPGATE = 9, ROW_SHARED_DOWN = 10, ROW_ROUTED_UPGATE = 11, ROW_ROUTED_DOWN = 12,
              ROW_COMBINE = 13;
// An extension of this build, in the row behind the reference's fourteen: the routed up/gate tiles counted per expert
// slot as well, so that a slot's down projection can start when its own silu vector is complete (word tile_M_idx of
// opcode 13 = 1) instead of when all slots' are.
constexpr int ROW_ROUTED_UPGATE_SLOT = 14;
constexpr int kMaxK = 2048;       // longest dot product of these ops (a K slice, an expert's FFN width, H)
constexpr int kMaxExperts = 512;
constexpr int kMaxTopK = 8;
constexpr int kTile = 16;

// NR weight rows of K columns (a multiple of 8, <= kMaxK) as 16-byte pieces per lane.  `request_rows` asks
// for all pieces of the first `live` rows (the others read as zeros); `reduce_rows` multiplies them with the
// bf16 vector x in LDS and leaves every lane the sums.  Between the two a caller may wait for x: what it
// asked for lands meanwhile.  Indices are constants already in the source (static_for, not unrolled loops).
template <int NR>
struct RowSet {
  v4u w[NR][kMaxK / 512];
};
template <int NR>
__device__ __forceinline__ void request_rows(RowSet<NR>& set, const u16* const (&rows)[NR], int K, int lane, int live = NR) {
  static_for<0, NR>([&](auto r) {
    static_for<0, kMaxK / 512>([&](auto i) {
      const int col = lane * 8 + i * 512;
      set.w[r][i] = v4u{0, 0, 0, 0};
      if (r < live && col < K) set.w[r][i] = __builtin_nontemporal_load(reinterpret_cast<const v4u*>(rows[r] + col));
    });
  });
}
template <int NR>
__device__ __forceinline__ void reduce_rows(const RowSet<NR>& set, const u16* x, int K, int lane, float (&out)[NR]) {
  static_for<0, NR>([&](auto r) {
    float a = 0.f;
    static_for<0, kMaxK / 512>([&](auto i) {
      const int col = lane * 8 + i * 512;
      if (col < K) a = dot8(set.w[r][i], *reinterpret_cast<const v4u*>(x + col), a);
    });
    out[r] = wave_sum(a);
  });
}
template <int NR>
__device__ __forceinline__ void rows_dot(const u16* const (&rows)[NR], const u16* x, int K, int lane, float (&out)[NR]) {
  RowSet<NR> set;
  request_rows(set, rows, K, lane);
  reduce_rows(set, x, K, lane, out);
}

// n bf16 elements (a multiple of 4) of a vector that another workgroup wrote during this launch, into s.x.
template <class M>
__device__ __forceinline__ void stage_vector(Smem<M>& s, const Ctx& c, const u16* src, int n) {
  for (int i = c.tid * 4; i < n; i += kThreads * 4) *reinterpret_cast<uint64_t*>(s.x + i) = ld_shared64(src + i);
  __syncthreads();
}

template <class M>
__device__ __forceinline__ bool wait_one(const Params& p, Smem<M>& s, const Ctx& c, int layer, int row, int slot, int expected) {
  return wg_wait(p, s, c, 1, [&](int) { return counter_ptr(p, layer, row, slot); }, expected);
}

__device__ __forceinline__ void publish_done(const Params& p, const Ctx& c, int layer, int row, int slot, int amount) {
  release_stores();
  __syncthreads();
  if (c.tid == 0) publish(counter_ptr(p, layer, row, slot), amount);
}

// The layer's residual stream after the O-projection, normalised with the MLP norm weights, as bf16 in s.x.
// With counters: after the O-projection's last arrival (`oproj_seen`: a counter the caller has waited on
// already implies it), from the caller's buffer.  Tagged launch: from the units the O-projection workgroups
// announce their rows in, each thread polling its own two.
template <class M>
__device__ __forceinline__ bool residual_to_lds(const Params& p, Smem<M>& s, const Ctx& c, int layer, bool oproj_seen = false) {
  const u16* weight = p.mlp_norm + static_cast<size_t>(layer) * M::H;
  if (tagged(p)) return rms_to_lds<M>(p, s, c, p.ws + kWsHiddenMid, tag_of(s.generation, layer), weight);
  if (!oproj_seen && !wait_one(p, s, c, layer, ROW_OPROJ, 0, p.oproj_blocks)) return false;
  return rms_to_lds<M>(p, s, c, nullptr, 0u, weight);
}

// ===================================================================== 8 ==
// [8, layer, e_start, e_end, write_normed_hidden, tile_N_g]
// RMSNorm of the residual stream, fp32 router logits of experts [e_start, e_end); one instruction of a
// layer also publishes the normalised row for opcodes 10, 12 and 14   (python_vm.py:331-357).
template <class M>
__device__ __forceinline__ bool op_router(const Params& p, Smem<M>& s, const Ctx& c) {
  const int layer = s.inst[1], g = s.inst[5], e0 = s.inst[2] * g, e1 = min(s.inst[3] * g, p.num_experts);
  if (layer < 0 || layer >= p.num_layers) return bad_operand(p, s, c, 1);
  if (g < 1 || e0 < 0 || e1 < e0) return bad_operand(p, s, c, 2);
  const int lane = c.tid & 63, wave = c.tid >> 6;
  const u16* w = p.router_w + static_cast<size_t>(layer) * p.num_experts * M::H;
  // The wave's first expert row is asked for before the residual stream is looked at: it lands during the wait.
  RowSet<1> first;
  {
    const u16* const rows[1] = {w + static_cast<size_t>(min(e0 + wave, max(e1 - 1, 0))) * M::H};
    request_rows<1>(first, rows, M::H, lane, e0 + wave < e1 ? 1 : 0);
  }
  if (!residual_to_lds<M>(p, s, c, layer)) return false;
  for (int e = e0 + wave; e < e1; e += kWaves) {
    const u16* const rows[1] = {w + static_cast<size_t>(e) * M::H};
    float v[1];
    if (e == e0 + wave) reduce_rows<1>(first, s.x, M::H, lane, v);
    else rows_dot<1>(rows, s.x, M::H, lane, v);
    if (lane == 0) {
      st_shared_f32(p.router_logits + e, v[0]);
      // tagged launch: the routed up/gate workgroups take the routing decision themselves from these
      if (tagged(p)) st_tagged(p.ws + kWsLogits + e * kLogitStride, __float_as_uint(v[0]), tag_of(s.generation, layer));
    }
  }
  const bool publish_row = s.inst[4] != 0;
  if (publish_row) {
    for (int i = c.tid * 2; i < M::H; i += kThreads * 2) st_shared32(p.normed_hidden + i, *reinterpret_cast<const uint32_t*>(s.x + i));
    // ... and the shared expert's gate, sigmoid(gate_w . normed) in fp32, which every combine instruction of the
    // layer would otherwise recompute from the same row (python_vm.py:506-510)
    if (wave == kWaves - 1 && p.shared_ffn > 0) {
      const u16* const rows[1] = {p.shared_scale_w + static_cast<size_t>(layer) * M::H};
      float v[1];
      rows_dot<1>(rows, s.x, M::H, lane, v);
      if (lane == 0) {
        const float gate = 1.0f / (1.0f + expf(-v[0]));
        st_shared_f32(p.shared_gate, gate);
        if (tagged(p)) st_tagged(p.ws + kWsSharedGate, __float_as_uint(gate), tag_of(s.generation, layer));
      }
    }
  }
  release_stores();
  __syncthreads();
  if (c.tid == 0) {
    publish(counter_ptr(p, layer, ROW_ROUTER, 0), e1 - e0);
    if (publish_row) publish(counter_ptr(p, layer, ROW_ROUTER, 1), 1);
  }
  return true;
}

// ===================================================================== 9 ==
// [9, layer]   softmax over all router logits, the top_k largest probabilities and their experts, in
// decreasing order (ties: the lower expert first)   (python_vm.py:360-372); renormalised to sum 1 when the
// launch asks for it (fused/operations.py:405).
// Softmax over the E router logits (thread t brings expert t's; threads beyond E bring nothing) and the top_k picks:
// afterwards, for every slot j < top_k, picked[j] is the pick's probability and picked[kMaxTopK + j] its expert (as
// int bits), in decreasing order of probability, the lower expert first among equals — the order repeated arg-max
// with first-index ties produces.  Instead of top_k dependent sweeps every expert counts the experts that go before
// it; a count below top_k is the pick's slot.  False (uniformly) when a logit is NaN or infinite: no order to pick by.
// Uses s.res[0 .. 2 * kMaxExperts) and s.red.
template <class M>
__device__ __forceinline__ bool rank_experts(const Params& p, Smem<M>& s, const Ctx& c, float logit, float* picked) {
  const int t = c.tid, E = p.num_experts;
  const bool live = t < E;
  const float mx = block_max(live ? logit : -INFINITY, s.red);
  const float x = live ? expf(logit - mx) : 0.f;
  const int padded = (E + 3) & ~3;
  int* counts = reinterpret_cast<int*>(s.res) + kMaxExperts;      // behind the probabilities
  if (t < padded) {
    s.res[t] = live ? x : -1.f;   // padded to whole groups of four with values nobody goes behind
    counts[t] = 0;
  }
  const float sum = block_sum(x, s.red);   // its barriers also make s.res complete
  const bool ok = sum > 0.f && sum < INFINITY;
  QMK_STAMP(2);
  // The E x E comparisons are spread over the whole workgroup (one wave alone would spend 3-4 us on them): thread t
  // compares expert t % E' with a slice of the others and adds its count to the expert's.
  int parts = 1;
  while (2 * parts * padded <= kThreads) parts *= 2;
  const int mine = t % padded, part = t / padded;
  if (ok && part < parts && mine < E) {
    const float xm = s.res[mine];
    const int per = ((padded / 4 + parts - 1) / parts) * 4;        // a slice is whole groups of four
    const int e0 = part * per, e1 = min(e0 + per, padded);
    int before = 0;
    const float4* all = reinterpret_cast<const float4*>(s.res);
#pragma unroll 4
    for (int e = e0; e < e1; e += 4) {
      const float4 v = all[e >> 2];
      before += (v.x > xm || (v.x == xm && e < mine)) ? 1 : 0;
      before += (v.y > xm || (v.y == xm && e + 1 < mine)) ? 1 : 0;
      before += (v.z > xm || (v.z == xm && e + 2 < mine)) ? 1 : 0;
      before += (v.w > xm || (v.w == xm && e + 3 < mine)) ? 1 : 0;
    }
    if (before) atomicAdd(&counts[mine], before);
  }
  QMK_STAMP(3);
  __syncthreads();
  if (ok && live && counts[t] < p.top_k) {
    picked[counts[t]] = x / sum;
    picked[kMaxTopK + counts[t]] = __int_as_float(t);
  }
  __syncthreads();
  return ok;
}

template <class M>
__device__ __forceinline__ bool op_topk(const Params& p, Smem<M>& s, const Ctx& c) {
  const int layer = s.inst[1], E = p.num_experts;
  static_assert(kMaxExperts <= kThreads, "one thread per expert");
  if (layer < 0 || layer >= p.num_layers) return bad_operand(p, s, c, 1);
  const int t = c.tid;
  const bool tg = tagged(p);
  float logit = 0.f;
  if (tg) {
    // Tagged launch: the logits from their units, like every consumer of the routing decision; nobody inside the
    // launch reads what this instruction writes, so it neither drains its stores nor counts.
    uint32_t bits = 0;
    if (t < E && !poll_tagged1(p.ws + kWsLogits + t * kLogitStride, tag_of(s.generation, layer), p.spin_limit, bits)) {
      s.ctl[0] = 1;
      report_error(p, QMK_DEV_WAIT_TIMEOUT, c.inst_idx, c.opcode, t);
    }
    logit = __uint_as_float(bits);
    QMK_STAMP(0);
  } else {
    if (!wait_one(p, s, c, layer, ROW_ROUTER, 0, E)) return false;
    if (t < E) logit = ld_shared_f32(p.router_logits + t);
  }
  float* picked = &s.merge[0][0][0];
  const bool ranked = rank_experts<M>(p, s, c, logit, picked);   // (its barriers publish s.ctl[0])
  QMK_STAMP(1);
  if (s.ctl[0]) return false;
  if (!ranked) return bad_operand(p, s, c, 0);
  if (t == 0) {
    // norm_topk_prob: the picks' probabilities divided by their sum, added up in slot order (fp32)
    float total = 0.f;
    for (int j = 0; j < p.top_k; ++j) total += picked[j];
    for (int j = 0; j < p.top_k; ++j) {
      const int idx = __float_as_int(picked[kMaxTopK + j]);
      const float w = p.norm_topk ? picked[j] / total : picked[j];
      __hip_atomic_store(p.expert_indices + j, static_cast<long long>(idx), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      st_shared_f32(p.expert_weights + j, w);
      if (tg && !p.local_routing) {   // the routed ops poll these: one trip, no drain in between
        st_tagged(p.ws + kWsTopK + 16 * j, static_cast<uint32_t>(idx), tag_of(s.generation, layer));
        st_tagged(p.ws + kWsTopK + 16 * j + 1, __float_as_uint(w), tag_of(s.generation, layer));
      }
    }
  }
  if (tg) {
    __syncthreads();   // picked is read: s.merge and s.res may be reused
    return true;
  }
  release_stores();
  __syncthreads();
  if (c.tid == 0) __hip_atomic_store(counter_ptr(p, layer, ROW_TOPK, 0), 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  return true;
}

// Gate and up rows [r0, r0 + n) of one FFN against the normalised row in s.x; out[i] =
// bf16(silu(bf16(gate . x)) * bf16(up . x)), silu and the product in fp32 (python_vm.py:389-395, 455-459).
// The results wait in s.res; two neighbouring ones leave as one word to every destination given.
// `ready()` makes s.x the normalised residual stream (false: give up); the rows of the wave's first round are
// asked for before it is called.
template <class M, class Ready>
__device__ __forceinline__ bool upgate_rows(Smem<M>& s, const Ctx& c, const u16* gate_w, const u16* up_w, int r0, int n, u16* dst0, u16* dst1,
                                            Ready ready, uint64_t* units = nullptr, uint32_t tag = 0) {
  const int lane = c.tid & 63, wave = c.tid >> 6;
  constexpr int kOut = M::UPGATE_OUTPUTS_IN_FLIGHT;   // outputs (gate + up row each) of a wave in flight together: 8 KiB each
  RowSet<2 * kOut> set;
  auto request = [&](int i) {
    const u16* rows[2 * kOut];
    static_for<0, kOut>([&](auto k) {
      const int o = min(i + k * kWaves, n - 1);   // past the end: not asked for
      rows[2 * k] = gate_w + static_cast<size_t>(r0 + o) * M::H;
      rows[2 * k + 1] = up_w + static_cast<size_t>(r0 + o) * M::H;
    });
    const int left = i < n ? (n - 1 - i) / kWaves + 1 : 0;   // outputs of this round that exist
    request_rows(set, rows, M::H, lane, 2 * min(left, kOut));
  };
  request(wave);
  if (!ready()) return false;
  for (int i = wave; i < n; i += kOut * kWaves) {
    float v[2 * kOut];
    reduce_rows(set, s.x, M::H, lane, v);
    if (i + kOut * kWaves < n) request(i + kOut * kWaves);
    if (lane == 0) {
      static_for<0, kOut>([&](auto k) {
        const float g = round_bf16(v[2 * k]);
        if (i + k * kWaves < n) s.res[i + k * kWaves] = (g / (1.0f + expf(-g))) * round_bf16(v[2 * k + 1]);
      });
    }
  }
  __syncthreads();
  for (int pair = c.tid; pair < n / 2; pair += kThreads) {
    const uint32_t word = f2bf2(s.res[2 * pair], s.res[2 * pair + 1]);
    st_shared32(dst0 + r0 + 2 * pair, word);
    if (dst1 != nullptr) st_shared32(dst1 + r0 + 2 * pair, word);
    if (units != nullptr) st_tagged(units + (r0 + 2 * pair) / 2, word, tag);
  }
  return true;
}

// ==================================================================== 10 ==
// [10, layer, tile_M, n_start, n_end, init_shared_out, tile_M_g, tile_N_g]   (python_vm.py:375-396)
// shared_out needs no clearing here: its K-slice terms have slots of their own until the combine step.
template <class M>
__device__ __forceinline__ bool op_shared_upgate(const Params& p, Smem<M>& s, const Ctx& c) {
  const int layer = s.inst[1], n0 = s.inst[3], n1 = s.inst[4], tile = s.inst[7];
  if (layer < 0 || layer >= p.num_layers) return bad_operand(p, s, c, 1);
  if (tile != kTile || n0 < 0 || n1 < n0 || n1 * tile > p.shared_ffn || (n1 - n0) * tile > kResSlots) return bad_operand(p, s, c, 4);
  // The normalised row is recomputed here from the residual stream (the same function of the same values as
  // the row opcode 8 publishes, bit for bit) instead of being waited for: the shared expert starts with the
  // O-proj's last arrival, beside the router.
  const size_t base = static_cast<size_t>(layer) * p.shared_ffn * M::H;
  if (!upgate_rows(s, c, p.shared_gate_w + base, p.shared_up_w + base, n0 * tile, (n1 - n0) * tile, p.shared_silu, nullptr,
                   [&] { return residual_to_lds<M>(p, s, c, layer); }))
    return false;
  publish_done(p, c, layer, ROW_SHARED_UPGATE, 0, n1 - n0);
  return true;
}

// Rows [r0, r0 + n) of a down projection with K columns (row stride ld) against s.x[0..K); `leave(r, dot)`
// runs on lane 0 of the wave that owns row r.  `ready()` fills s.x (false: give up); the rows of the wave's
// first round are asked for before it is called.
template <class M, class Ready, class Leave>
__device__ __forceinline__ bool down_rows(Smem<M>& s, const Ctx& c, const u16* w, size_t ld, int K, int r0, int n, Ready ready, Leave leave) {
  const int lane = c.tid & 63, wave = c.tid >> 6;
  constexpr int kRows = 4;
  RowSet<kRows> set;
  auto request = [&](int i) {
    const u16* rows[kRows];
    static_for<0, kRows>([&](auto k) { rows[k] = w + static_cast<size_t>(r0 + min(i + k * kWaves, n - 1)) * ld; });
    request_rows(set, rows, K, lane, i < n ? min((n - 1 - i) / kWaves + 1, kRows) : 0);
  };
  request(wave);
  if (!ready()) return false;
  for (int i = wave; i < n; i += kRows * kWaves) {
    float v[kRows];
    reduce_rows(set, s.x, K, lane, v);
    if (i + kRows * kWaves < n) request(i + kRows * kWaves);
    if (lane == 0) {
      static_for<0, kRows>([&](auto k) {
        if (i + k * kWaves < n) leave(r0 + i + k * kWaves, v[k]);
      });
    }
  }
  return true;
}

// ==================================================================== 11 ==
// [11, layer, tile_M, n_start, n_end, split_K_idx, tile_M_g, tile_N_g, split_K_g]   (python_vm.py:399-418)
// One K slice of the shared down projection: bf16(W[r, k0:k1] . silu[k0:k1]) into this slice's slot.
template <class M>
__device__ __forceinline__ bool op_shared_down(const Params& p, Smem<M>& s, const Ctx& c) {
  const int layer = s.inst[1], n0 = s.inst[3], n1 = s.inst[4], slice = s.inst[5], tile = s.inst[7], kg = s.inst[8];
  if (layer < 0 || layer >= p.num_layers) return bad_operand(p, s, c, 1);
  if (tile != kTile || n0 < 0 || n1 < n0 || n1 * tile > M::H) return bad_operand(p, s, c, 4);
  if (slice < 0 || slice >= p.shared_k_slices || kg < 8 || (kg & 7) || kg > kMaxK || slice * kg >= p.shared_ffn) return bad_operand(p, s, c, 5);
  const int k0 = slice * kg, K = min(kg, p.shared_ffn - k0);
  const u16* w = p.shared_down_w + static_cast<size_t>(layer) * M::H * p.shared_ffn + k0;
  u16* mine = p.shared_parts + static_cast<size_t>(slice) * M::H;
  if (!down_rows(
          s, c, w, p.shared_ffn, K, n0 * tile, (n1 - n0) * tile,
          [&] {
            if (!wait_one(p, s, c, layer, ROW_SHARED_UPGATE, 0, p.shared_ffn / kTile)) return false;
            stage_vector(s, c, p.shared_silu + k0, K);
            return true;
          },
          [&](int r, float dot) { s.res[r - n0 * tile] = dot; }))
    return false;
  __syncthreads();
  for (int pair = c.tid; pair < (n1 - n0) * tile / 2; pair += kThreads)
    st_shared32(mine + n0 * tile + 2 * pair,
                f2bf2(s.res[2 * pair], s.res[2 * pair + 1]));
  release_stores();
  __syncthreads();
  if (c.tid < n1 - n0) publish(counter_ptr(p, layer, ROW_SHARED_DOWN, n0 + c.tid), 1);
  return true;
}

// The physical expert of a slot, read after the top-k edge; negative when it is not one.
__device__ __forceinline__ int expert_of(const Params& p, int slot) {
  const long long e = __hip_atomic_load(p.expert_indices + slot, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  return (e >= 0 && e < p.num_experts) ? static_cast<int>(e) : -1;
}

// Wait for the layer's top-k and fetch a slot's expert (negative: not an expert of the layer) and weight:
// through the counter and the caller's buffers, or, in a tagged launch, from the two neighbouring units the top-k
// instruction announces them in (one look for both; a line per slot).  False (uniformly) when the wait ran out of polls.
template <class M>
__device__ __forceinline__ bool routed_expert(const Params& p, Smem<M>& s, const Ctx& c, int layer, int slot, int& eid, float& weight) {
  if (!tagged(p)) {
    if (!wait_one(p, s, c, layer, ROW_TOPK, 0, 1)) return false;
    eid = expert_of(p, slot);
    weight = ld_shared_f32(p.expert_weights + slot);
    return true;
  }
  if (c.tid == 0) {
    uint32_t e = 0, w = 0;
    const uint32_t tag = tag_of(s.generation, layer);
    if (!poll_tagged2(p.ws + kWsTopK + 16 * slot, tag, p.spin_limit, e, w)) {   // expert and weight in one trip
      s.ctl[0] = 1;
      report_error(p, QMK_DEV_WAIT_TIMEOUT, c.inst_idx, c.opcode, slot);
    }
    s.ctl[4] = e < static_cast<uint32_t>(p.num_experts) ? static_cast<int>(e) : -1;
    s.ctl[5] = static_cast<int>(w);
    if (p.timeline != nullptr) {
      s.t_wait = wall_clock64();
      s.ctl[2] = 1;
    }
  }
  __syncthreads();
  eid = s.ctl[4];
  weight = __uint_as_float(static_cast<uint32_t>(s.ctl[5]));
  return s.ctl[0] == 0;
}

// Tagged launch: the routing decision taken by the consumer itself, from the router's logits as they announce
// themselves — the top-k instruction's own function of the same 32-bit values (rank_experts, then the same
// renormalisation in the same order), so the same experts and weights, bit for bit — instead of waiting for that
// instruction to announce it: one hand-over less between the O-projection and the expert rows, during which the
// whole device has nothing else to do.  The top-k instruction still leaves expert_indices / expert_weights for the
// caller, off the critical path.  False (uniformly) when the wait ran out of polls or the logits have no order.
// A workgroup takes the decision once per layer: its routed down-projection instruction finds what its routed
// up/gate instruction of the same layer left in LDS.
template <class M>
__device__ __forceinline__ bool routing_decision(const Params& p, Smem<M>& s, const Ctx& c, int layer, int slot, int& eid, float& weight) {
  static_assert(kMaxTopK <= 8, "the decision kept in LDS has eight slots");
  if (s.route_layer == layer) {   // (written before the barrier that ended an earlier instruction)
    eid = s.route_expert[slot];
    weight = s.route_weight[slot];
    if (p.timeline != nullptr && c.tid == 0) {
      s.t_wait = wall_clock64();
      s.ctl[2] = 1;
    }
    return true;
  }
  uint32_t bits = 0;
  if (c.tid < p.num_experts && !poll_tagged1(p.ws + kWsLogits + c.tid * kLogitStride, tag_of(s.generation, layer), p.spin_limit, bits)) {
    s.ctl[0] = 1;
    report_error(p, QMK_DEV_WAIT_TIMEOUT, c.inst_idx, c.opcode, c.tid);
  }
  if (p.timeline != nullptr && c.tid == 0) {
    s.t_wait = wall_clock64();
    s.ctl[2] = 1;
  }
  float* picked = &s.merge[0][0][0];
  const bool ranked = rank_experts<M>(p, s, c, __uint_as_float(bits), picked);   // (its barriers publish s.ctl[0])
  if (s.ctl[0]) return false;
  if (!ranked) return bad_operand(p, s, c, 2);
  float total = 0.f;
  for (int j = 0; j < p.top_k; ++j) total += picked[j];
  eid = __float_as_int(picked[kMaxTopK + slot]);
  weight = p.norm_topk ? picked[slot] / total : picked[slot];
  if (c.tid < p.top_k) {
    s.route_expert[c.tid] = __float_as_int(picked[kMaxTopK + c.tid]);
    s.route_weight[c.tid] = p.norm_topk ? picked[c.tid] / total : picked[c.tid];
  }
  if (c.tid == 0) s.route_layer = layer;
  __syncthreads();   // picked is read: s.merge and s.res may be reused
  return true;
}

// ==================================================================== 12 ==
// [12, layer, expert_slot, n_start, n_end, tile_M_g, tile_N_g]   (python_vm.py:421-464)
// The single buffer silu_out keeps what the last slot wrote, as after the VM's sequential run.
template <class M>
__device__ __forceinline__ bool op_routed_upgate(const Params& p, Smem<M>& s, const Ctx& c) {
  const int layer = s.inst[1], slot = s.inst[2], n0 = s.inst[3], n1 = s.inst[4], tile = s.inst[6];
  if (layer < 0 || layer >= p.num_layers) return bad_operand(p, s, c, 1);
  if (slot < 0 || slot >= p.top_k || slot >= p.barrier_slots - 1) return bad_operand(p, s, c, 2);
  if (tile != p.routed_tile || n0 < 0 || n1 < n0 || n1 * tile > p.moe_ffn || (n1 - n0) * tile > kResSlots) return bad_operand(p, s, c, 4);
  const bool tg = tagged(p);
  const uint32_t tag = tag_of(s.generation, layer);
  int eid;
  float unused;
  // A tagged launch has the normalised row long before the experts are known.
  if (tg && !residual_to_lds<M>(p, s, c, layer)) return false;
  if (!(tg && p.local_routing ? routing_decision<M>(p, s, c, layer, slot, eid, unused) : routed_expert<M>(p, s, c, layer, slot, eid, unused))) return false;
  if (eid < 0) return bad_operand(p, s, c, 2);
  const u16* w = p.expert_gate_up_w + (static_cast<size_t>(layer) * p.num_experts + eid) * 2 * p.moe_ffn * M::H;
  // tagged launch: the slot's down projections poll the silu values as units of their own
  uint64_t* units = tg ? p.ws + kWsRoutedSilu + slot * 1024 : nullptr;
  if (!upgate_rows(s, c, w, w + static_cast<size_t>(p.moe_ffn) * M::H, n0 * tile, (n1 - n0) * tile,
                   p.routed_silu + static_cast<size_t>(slot) * p.moe_ffn, slot == p.top_k - 1 ? p.silu_out : nullptr,
                   [&] { return tg || residual_to_lds<M>(p, s, c, layer, /*oproj_seen=*/true); }, units, tag))
    return false;
  if (tg) return true;   // nothing to wait for, nothing to count
  release_stores();
  __syncthreads();
  if (c.tid == 0) {
    publish(counter_ptr(p, layer, ROW_ROUTED_UPGATE_SLOT, slot), n1 - n0);
    publish(counter_ptr(p, layer, ROW_ROUTED_UPGATE, 0), n1 - n0);
  }
  return true;
}

// Opcode 13 with tile_M_idx = 2, an extension of this build for tagged launches of a model without a shared
// expert: ALL expert slots of the rows [r0, r0 + n) and the combine step in one instruction — the terms
// bf16(W_down[expert_j][r] . silu_j) * weight_j are added in slot order in fp32 and committed as opcode 14 commits
// them, hidden[r] = bf16(hidden[r] + routed[r])  (python_vm.py:467-530), so the stream needs no opcode 14 and the
// routed rows no hand-over of their own.  The decision of every slot comes from the workgroup's own ranking of the
// router's logits (local routing).
// Wave j takes expert slot j: it asks for its rows (kRows of kChunks x 512 columns per round: 8 x 2 holds all of an
// 8-row instruction for an expert width up to 1024; wider experts take 4 x 4 and more rounds), then every lane looks
// at exactly the units of silu_j its pieces of the rows multiply, all of them in one trip, and keeps them in
// registers: no LDS copy of the vectors, no barrier between the looks and the dot products, and a wave whose slot
// was finished early is not held up by a later one.
template <class M, int kRows, int kChunks>
__device__ __forceinline__ bool routed_down_commit(const Params& p, Smem<M>& s, const Ctx& c, int layer, int r0, int n) {
  const int lane = c.tid & 63, wave = c.tid >> 6;
  const int K = p.moe_ffn;
  const uint32_t tag = tag_of(s.generation, layer);
  int first_expert;
  float first_weight;
  if (!routing_decision<M>(p, s, c, layer, 0, first_expert, first_weight)) return false;   // leaves all slots in s.route_*
  const bool live = wave < p.top_k;
  const u16* const rows = p.expert_down_w + ((static_cast<size_t>(layer) * p.num_experts + (live ? s.route_expert[wave] : 0)) * M::H + r0) * K + lane * 8;
  v4u w[kRows][kChunks];
  auto request = [&](int r) {
    static_for<0, kRows>([&](auto k) {
      static_for<0, kChunks>([&](auto q) {
        w[k][q] = v4u{0, 0, 0, 0};
        if (live && r + k < n && lane * 8 + q * 512 < K)
          w[k][q] = __builtin_nontemporal_load(reinterpret_cast<const v4u*>(rows + static_cast<size_t>(r + k) * K + q * 512));
      });
    });
  };
  request(0);
  // the residual pair this thread commits, from the unit the O-projection announced it in (every up/gate workgroup
  // has seen its tag): asked for before the looks at the silu vector, not behind them
  uint32_t old = 0;
  if (c.tid < n / 2) old = static_cast<uint32_t>(ld_shared64(p.ws + kWsHiddenMid + (r0 + 2 * c.tid) / 2));
  v4u x[kChunks];   // columns lane*8 + q*512 .. +7 of silu_j: four units of two bf16 each; zeros past the row's end
  static_for<0, kChunks>([&](auto q) { x[q] = v4u{0, 0, 0, 0}; });
  if (live) {
    const uint64_t* units = p.ws + kWsRoutedSilu + wave * 1024 + lane * 4;
    uint32_t polls = 0;
    while (true) {
      uint64_t u[kChunks][4];
      static_for<0, kChunks>([&](auto q) {
        static_for<0, 4>([&](auto j) {
          u[q][j] = static_cast<uint64_t>(tag) << 32;
          if (lane * 8 + q * 512 < K) u[q][j] = ld_shared64(units + q * 256 + j);
        });
      });
      bool all = true;
      static_for<0, kChunks>([&](auto q) {
        static_for<0, 4>([&](auto j) { all = all && static_cast<uint32_t>(u[q][j] >> 32) == tag; });
        x[q] = v4u{static_cast<uint32_t>(u[q][0]), static_cast<uint32_t>(u[q][1]), static_cast<uint32_t>(u[q][2]), static_cast<uint32_t>(u[q][3])};
      });
      if (all) break;
      if (++polls > p.spin_limit) {
        s.ctl[0] = 1;   // seen by everybody after the barrier in front of the commit
        report_error(p, QMK_DEV_WAIT_TIMEOUT, c.inst_idx, c.opcode, wave);
        break;
      }
      __builtin_amdgcn_s_sleep(1);
    }
  }
  if (p.timeline != nullptr && c.tid == 0) {
    s.t_wait = wall_clock64();
    s.ctl[2] = 1;
  }
  for (int r = 0; r < n; r += kRows) {
    float v[kRows];
    static_for<0, kRows>([&](auto k) {
      float a = 0.f;
      static_for<0, kChunks>([&](auto q) { a = dot8(w[k][q], x[q], a); });
      v[k] = wave_sum(a);
    });
    if (r + kRows < n) request(r + kRows);
    if (lane == 0 && live) {
      const float weight = s.route_weight[wave];
      static_for<0, kRows>([&](auto k) {
        if (r + k < n) s.res[wave * n + r + k] = round_bf16(v[k]) * weight;
      });
    }
  }
  __syncthreads();
  if (s.ctl[0]) return false;
  if (c.tid < n / 2) {
    const int pair = c.tid, r = r0 + 2 * pair;
    float ro0 = 0.f, ro1 = 0.f;
    for (int j = 0; j < p.top_k; ++j) {
      ro0 += s.res[j * n + 2 * pair];
      ro1 += s.res[j * n + 2 * pair + 1];
    }
    const float h0 = (bf_lo(old) + ro0) + 0.f, h1 = (bf_hi(old) + ro1) + 0.f;   // opcode 14's expression without a shared term
    const uint32_t word = f2bf2(h0, h1);
    st_shared32(p.hidden + r, word);
    st_tagged(p.ws + kWsHiddenOut + r / 2, word, tag);
    st_shared_f32(p.routed_out_f32 + r, 0.f);
    st_shared_f32(p.routed_out_f32 + r + 1, 0.f);
  }
  return true;
}

// ==================================================================== 13 ==
// [13, layer, expert_slot, tile_M, n_start, n_end, tile_M_g, tile_N_g]   (python_vm.py:467-489)
// bf16(W_down[expert][r] . silu[slot]) * weight[slot], fp32, into the slot's own row of the workspace.
template <class M>
__device__ __forceinline__ bool op_routed_down(const Params& p, Smem<M>& s, const Ctx& c) {
  const int layer = s.inst[1], slot = s.inst[2], n0 = s.inst[4], n1 = s.inst[5], tile = s.inst[7];
  const bool own_slot_only = s.inst[3] == 1;   // tile_M_idx: 0 in the reference's streams
  if (layer < 0 || layer >= p.num_layers) return bad_operand(p, s, c, 1);
  if (slot < 0 || slot >= p.top_k || slot >= p.barrier_slots - 1) return bad_operand(p, s, c, 2);
  if (s.inst[3] == 2) {   // all slots of the rows and the commit: tagged launches with local routing, no shared expert
    if (!tagged(p) || !p.local_routing || p.shared_k_slices != 0 || slot != 0) return bad_operand(p, s, c, 3);
    if ((tile != kTile && tile != kTile / 2) || n0 < 0 || n1 <= n0 || n1 * tile > M::H || (n1 - n0) * tile > kTile) return bad_operand(p, s, c, 5);
    if ((p.moe_ffn & 7) || p.moe_ffn > kMaxK || p.top_k > kWaves) return bad_operand(p, s, c, 0);   // a wave per slot, <= 4 x 512 columns
    if (p.moe_ffn <= 1024) return routed_down_commit<M, 8, 2>(p, s, c, layer, n0 * tile, (n1 - n0) * tile);
    return routed_down_commit<M, 4, 4>(p, s, c, layer, n0 * tile, (n1 - n0) * tile);
  }
  if (s.inst[3] != 0 && s.inst[3] != 1) return bad_operand(p, s, c, 3);
  if (tile != kTile || n0 < 0 || n1 < n0 || n1 * tile > M::H) return bad_operand(p, s, c, 5);
  if (tagged(p) && (p.moe_ffn & 3)) return bad_operand(p, s, c, 0);   // whole unit pairs
  // The expert is known with the top-k edge, long before the routed up/gate rows are complete: its rows are
  // asked for in between.
  int eid;
  float weight;
  if (!(tagged(p) && p.local_routing ? routing_decision<M>(p, s, c, layer, slot, eid, weight) : routed_expert<M>(p, s, c, layer, slot, eid, weight))) return false;
  if (eid < 0) return bad_operand(p, s, c, 2);
  const u16* w = p.expert_down_w + (static_cast<size_t>(layer) * p.num_experts + eid) * M::H * p.moe_ffn;
  float* mine = p.routed_parts + static_cast<size_t>(slot) * M::H;
  const bool tg = tagged(p);
  const uint32_t tag = tag_of(s.generation, layer);
  uint64_t* out_units = p.ws + kWsRoutedParts + slot * 2048;
  if (!down_rows(
          s, c, w, p.moe_ffn, p.moe_ffn, n0 * tile, (n1 - n0) * tile,
          [&] {
            if (tg) {
              // the slot's silu vector from the units its up/gate workgroups announce it in: two units per poller
              const uint64_t* units = p.ws + kWsRoutedSilu + slot * 1024;
              uint32_t* words = reinterpret_cast<uint32_t*>(s.x);
              for (int u = 2 * c.tid; u < p.moe_ffn / 2; u += 2 * kThreads) {
                uint32_t a = 0, b = 0;
                if (!poll_tagged2(units + u, tag, p.spin_limit, a, b)) {
                  s.ctl[0] = 1;
                  report_error(p, QMK_DEV_WAIT_TIMEOUT, c.inst_idx, c.opcode, c.tid);
                }
                words[u] = a;
                words[u + 1] = b;
              }
              if (p.timeline != nullptr && c.tid == 0) {
                s.t_wait = wall_clock64();
                s.ctl[2] = 1;
              }
              __syncthreads();
              return s.ctl[0] == 0;
            }
            const int per_slot = p.moe_ffn / p.routed_tile;
            if (!(own_slot_only ? wait_one(p, s, c, layer, ROW_ROUTED_UPGATE_SLOT, slot, per_slot)
                                : wait_one(p, s, c, layer, ROW_ROUTED_UPGATE, 0, p.top_k * per_slot)))
              return false;
            stage_vector(s, c, p.routed_silu + static_cast<size_t>(slot) * p.moe_ffn, p.moe_ffn);
            return true;
          },
          [&](int r, float dot) {
            const float term = round_bf16(dot) * weight;
            if (tg) st_tagged(out_units + r, __float_as_uint(term), tag);   // the combine step polls these
            else st_shared_f32(mine + r, term);
          }))
    return false;
  if (tg) return true;
  release_stores();
  __syncthreads();
  if (c.tid < n1 - n0) publish(counter_ptr(p, layer, ROW_ROUTED_DOWN, n0 + c.tid), 1);
  return true;
}

// ==================================================================== 14 ==
// [14, layer, n_start, n_end, tile_N_g]   (python_vm.py:492-530)
// hidden[r] = bf16(hidden[r] + routed[r] + gate * shared[r]) for the rows of its tiles (gate: see opcode 8),
// with shared = the K-slice terms added in bf16 in slice order and routed = the slots' terms added in
// fp32 in slot order; leaves shared_out complete and routed_out_f32 cleared, as the VM does.
template <class M>
__device__ __forceinline__ bool op_combine(const Params& p, Smem<M>& s, const Ctx& c) {
  const int layer = s.inst[1], n0 = s.inst[2], n1 = s.inst[3], tile = s.inst[4];
  if (layer < 0 || layer >= p.num_layers) return bad_operand(p, s, c, 1);
  if (tile != kTile || n0 < 0 || n1 < n0 || n1 * tile > M::H || 2 * (n1 - n0) > kThreads) return bad_operand(p, s, c, 3);
  const int nb = n1 - n0;
  const bool tg = tagged(p);
  const uint32_t tag = tag_of(s.generation, layer);
  // Counters: the down projections of the instruction's blocks.  In a tagged launch the routed experts' rows are
  // units that announce themselves (polled below), so only the shared expert's K-slice counters are waited for.
  if (c.tid < 2 * nb && (!tg || c.tid < nb)) {
    const bool routed = c.tid >= nb;
    const int blk = n0 + (routed ? c.tid - nb : c.tid);
    // (without a shared expert shared_k_slices is 0 and that half of the pollers passes at once)
    if (!poll_counter(counter_ptr(p, layer, routed ? ROW_ROUTED_DOWN : ROW_SHARED_DOWN, blk), routed ? p.top_k : p.shared_k_slices, p.spin_limit)) {
      s.ctl[0] = 1;
      report_error(p, QMK_DEV_WAIT_TIMEOUT, c.inst_idx, c.opcode, c.tid);
    }
  }
  if (p.timeline != nullptr && c.tid == 0) {
    s.t_wait = wall_clock64();
    s.ctl[2] = 1;
  }
  __syncthreads();
  if (s.ctl[0]) return false;
  // left by the layer's publishing router instruction: behind the router counter that the top-k instruction waited
  // for, or, in a tagged launch, in a unit of its own
  float gate = 0.f;
  if (p.shared_k_slices > 0) {
    if (tg) {
      uint32_t bits = 0;
      if (!poll_tagged1(p.ws + kWsSharedGate, tag, p.spin_limit, bits)) {
        s.ctl[0] = 1;   // seen by everybody behind the barrier below
        report_error(p, QMK_DEV_WAIT_TIMEOUT, c.inst_idx, c.opcode, c.tid);
      }
      gate = __uint_as_float(bits);
    } else {
      gate = ld_shared_f32(p.shared_gate);
    }
  }
  constexpr int kMaxSlices = 16;   // the launcher's bound on shared_k_slices
  for (int pair = c.tid; pair < nb * tile / 2; pair += kThreads) {
    const int r = n0 * tile + 2 * pair;
    // every term is asked for before the first one is used: one trip to memory, not one per term
    uint32_t st[kMaxSlices];
    uint64_t rt[kMaxTopK];
#pragma unroll
    for (int k = 0; k < kMaxSlices; ++k) st[k] = k < p.shared_k_slices ? ld_shared32(p.shared_parts + static_cast<size_t>(k) * M::H + r) : 0u;
    // Tagged launch: the unit the O-projection announced this pair in.  Every up/gate workgroup has seen its
    // tag, and this instruction follows them through the down projections: no polling — and asked for before the
    // looks at the routed rows below, so that it does not cost a trip of its own behind them.
    const uint32_t old = tg ? static_cast<uint32_t>(ld_shared64(p.ws + kWsHiddenMid + r / 2)) : ld_shared32(p.hidden + r);
    if (tg) {
      // two units per slot, all slots in flight together, looked at until every one carries this layer's tag
      const uint64_t* units = p.ws + kWsRoutedParts + r;
      bool have[kMaxTopK];
#pragma unroll
      for (int j = 0; j < kMaxTopK; ++j) have[j] = j >= p.top_k, rt[j] = 0ull;
      for (uint32_t polls = 0;; ++polls) {
        uint64_t a[kMaxTopK], b[kMaxTopK];
#pragma unroll
        for (int j = 0; j < kMaxTopK; ++j)
          if (!have[j]) a[j] = ld_shared64(units + j * 2048), b[j] = ld_shared64(units + j * 2048 + 1);
        bool all = true;
#pragma unroll
        for (int j = 0; j < kMaxTopK; ++j) {
          if (!have[j] && static_cast<uint32_t>(a[j] >> 32) == tag && static_cast<uint32_t>(b[j] >> 32) == tag) {
            rt[j] = (a[j] & 0xffffffffull) | (b[j] << 32);
            have[j] = true;
          }
          all = all && have[j];
        }
        if (all) break;
        if (polls > p.spin_limit) {
          s.ctl[0] = 1;
          report_error(p, QMK_DEV_WAIT_TIMEOUT, c.inst_idx, c.opcode, c.tid);
          break;
        }
        __builtin_amdgcn_s_sleep(2);
      }
    } else {
#pragma unroll
      for (int j = 0; j < kMaxTopK; ++j) rt[j] = j < p.top_k ? ld_shared64(p.routed_parts + static_cast<size_t>(j) * M::H + r) : 0ull;
    }
    float sh0 = 0.f, sh1 = 0.f;
#pragma unroll
    for (int k = 0; k < kMaxSlices; ++k) {
      if (k < p.shared_k_slices) {
        sh0 = round_bf16(sh0 + bf_lo(st[k]));
        sh1 = round_bf16(sh1 + bf_hi(st[k]));
      }
    }
    float ro0 = 0.f, ro1 = 0.f;
#pragma unroll
    for (int j = 0; j < kMaxTopK; ++j) {
      if (j < p.top_k) {
        ro0 += __uint_as_float(static_cast<uint32_t>(rt[j]));
        ro1 += __uint_as_float(static_cast<uint32_t>(rt[j] >> 32));
      }
    }
    const float h0 = (bf_lo(old) + ro0) + gate * sh0, h1 = (bf_hi(old) + ro1) + gate * sh1;
    const uint32_t word = f2bf2(h0, h1);
    st_shared32(p.hidden + r, word);
    if (tg) st_tagged(p.ws + kWsHiddenOut + r / 2, word, tag);   // the next layer's QKV and O-projection, the LM head
    if (p.shared_k_slices > 0) st_shared32(p.shared_out + r, f2bf2(sh0, sh1));
    st_shared_f32(p.routed_out_f32 + r, 0.f);
    st_shared_f32(p.routed_out_f32 + r + 1, 0.f);
  }
  if (tg) {   // uniform: a poller that gave up has said so
    __syncthreads();
    if (s.ctl[0]) return false;
  }
  publish_done(p, c, layer, ROW_COMBINE, 0, nb);
  return true;
}

}  // namespace moe
}  // namespace qmk
