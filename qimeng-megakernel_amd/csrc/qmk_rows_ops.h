// The MoE decode route for 2..4 requests ("rows") in ONE launch per step, on the batch-1 kernel's row-streaming
// engine: a wave still reads whole weight rows as coalesced 16-byte pieces, but multiplies each piece with the
// activation vectors of all rows, so the attention half, the router and the LM head cross the memory system once
// per step instead of once per row, and every selected expert once for all the rows that chose it.
//
// The reference has no MoE route for batch sizes above one.  A step here is DEFINED as its batch-1 route
// (qimeng_megakernel/models/LLM/qwen/qwen1_5_moe_a2_7b/A100/single_batch/decode_schedule/instructions/python_vm.py:331-530,
// with the Qwen3 op set's attention, …/qwen/qwen3__0_6b/A100/single_batch/decode_schedule/fused/operations.py:52-120)
// run for every row on that row's own buffers, and every row keeps the batch-1 kernel's bits: each dot product is
// accumulated over the same pieces in the same order, the routed terms of a row are added in its own slot order.
//
// Layout: every per-request buffer of the batch-1 route gets a leading row dimension ([B, ...], KV cache
// [B, L, 1, S, NKV, D]), so row r's slice IS a batch-1 buffer set; weights exist once.  Hand-over between
// workgroups is the tagged one throughout (one workspace of self-announcing units per row); the only counters
// are the split-KV arrivals in front of the O-projection and the retirement count.
//
// Opcodes: 1, 4, 7, 8 as on the batch-1 route but for all rows at once; 2 (split-KV) and 9 (the reporting top-k)
// are the batch-1 ops run on a row's view of the buffers (the row is an extra operand word); 15 and 16 replace the
// per-slot instructions 12/13 — the rows' picks are merged, in every workgroup alike, into the list of DISTINCT
// experts in ascending order, and the routed work is dealt over that list at run time.
#pragma once

#include "qmk_moe_ops.h"

namespace qmk {
namespace rows {

constexpr int kMaxRows = 4;
constexpr int kMaxList = kMaxRows * moe::kMaxTopK;   // distinct experts of a layer at most
constexpr int kRowRes = 256;                         // GEMV results per row awaiting an epilogue
constexpr int kCommitRows = 16;                      // residual-stream rows one committing instruction takes at most

enum Opcode {
  OP_ROUTED_UPGATE_ROWS = 15,
  OP_ROUTED_DOWN_COMMIT_ROWS = 16,
};

// Width of a row's activation vector in LDS: the widest vector an op of the route stages (the attention output; for the
// dense models, whose geometries say so with DENSE_ROWS, the MLP's intermediate vector).
template <class M, class = void>
struct XWidth {
  static constexpr int value = M::AW > M::H ? M::AW : M::H;
};
template <class M>
struct XWidth<M, std::enable_if_t<M::DENSE_ROWS>> {
  static constexpr int value = M::F;
};

// The dense geometries as the rows kernel uses them: the number of rows the ops are compiled for (ROWS: 2, 3 or 4 — a
// launch of B rows runs on the smallest that holds them, so that two rows do not pay the norms, dot products and
// epilogues of four), and, as in the batch-1 kernel, the rows of the up/gate instruction behind it that an O-projection
// workgroup asks for while it waits through the attention phase and leaves in LDS (PARK_ROWS per wave; the batch-1 ops'
// result slots are not used here and make room for them).  Llama shape, last 200 steps of the 1024-token request, ms per
// step at 2 / 3 / 4 rows: none parked 0.645 / 0.690 / 0.738, two parked 0.629 / 0.677 / 0.736 (three at 2 rows: 0.625);
// rows also carried in registers, as the batch-1 kernel does (CARRY_ROWS): one 0.638 / 0.677 / 0.739, two 0.677 at 2 rows
// — beside the rows' activation vectors they cost more registers than they save time.  The Qwen3-1.7B shape, whose
// O-projection waits less, gains nothing from either (1.053 against 1.049 ms at 2 rows) and parks none.
template <int NR>
struct Llama1BRowsN : Llama1B {
  static constexpr int CARRY_ROWS = 0;
  static constexpr int PARK_ROWS = 2;
  static constexpr bool DENSE_ROWS = true;
  static constexpr int ROWS = NR;
  static constexpr int RES_SLOTS = 16;
};
template <int NR>
struct Qwen3_1p7BRowsN : Qwen3_1p7B {
  static constexpr int CARRY_ROWS = 0;
  static constexpr int PARK_ROWS = 0;
  static constexpr bool DENSE_ROWS = true;
  static constexpr int ROWS = NR;
};
using Llama1BRows = Llama1BRowsN<kMaxRows>;
using Qwen3_1p7BRows = Qwen3_1p7BRowsN<kMaxRows>;
// Rows the ops of a geometry are compiled for (kMaxRows unless the geometry says otherwise).
template <class M, class = void>
struct RowsOf {
  static constexpr int value = kMaxRows;
};
template <class M>
struct RowsOf<M, std::void_t<decltype(M::ROWS)>> {
  static constexpr int value = M::ROWS;
};

// The geometry as the batch-1 ops called from here see it: their LDS holds no parked rows (this kernel keeps its own).
template <class M>
struct Inner : M {
  static constexpr int PARK_ROWS = 0;
};
template <class M, class = void>
struct IsDense : std::false_type {};
template <class M>
struct IsDense<M, std::enable_if_t<M::DENSE_ROWS>> : std::true_type {};
// A dense geometry whose O-projection asks for rows of the up/gate instruction behind it.
template <class M>
struct AsksAhead {
  static constexpr bool value = IsDense<M>::value && (M::PARK_ROWS > 0 || M::CARRY_ROWS > 0);
};
// What only the MoE ops keep in LDS (absent from the dense kernels).
struct RoutingScratch {
  alignas(16) uint64_t key[kMaxRows][moe::kMaxExperts];  // ranking: {softmax numerator bits, ~expert} per row and expert (read two at a time)
  float terms[kMaxRows][moe::kMaxTopK][kCommitRows];     // committing instruction: weighted rows per (row, slot)
};
struct NoRoutingScratch {};

template <class M>
struct Smem {
  qmk::Smem<Inner<M>> b;                // what the batch-1 ops use when they run on a row's view (attention, top-k report)
  int32_t pos[kMaxRows];                // position each row decodes
  int32_t live[kMaxRows];               // the row exists and is active: a row that is not is a hole every op steps over
  float red[2][kMaxRows][kWaves];
  alignas(16) u16 x[AsksAhead<M>::value ? RowsOf<M>::value : kMaxRows][XWidth<M>::value];   // the rows' activation vectors (no more of them than the ops are compiled for where LDS is short)
  float res[kMaxRows][kRowRes];
  // the routing decision this workgroup last took (layer, -1: none yet), per row and slot, and the distinct experts
  int32_t route_layer;
  int32_t n_list;
  int32_t no_order;                     // ranking: a row's logits have no order (NaN or infinite)
  alignas(16) int32_t route_expert[kMaxRows][moe::kMaxTopK];
  float route_weight[kMaxRows][moe::kMaxTopK];
  int32_t list_expert[kMaxList];
  int32_t list_slot[kMaxList][kMaxRows];   // the slot in which row r picked list entry u, or -1
  alignas(16) float picked_p[kMaxRows][moe::kMaxTopK];
  int32_t picked_e[kMaxRows][moe::kMaxTopK];
  int32_t wave_count[kWaves];
  alignas(16) std::conditional_t<IsDense<M>::value, NoRoutingScratch, RoutingScratch> moe;
  alignas(16) ParkedRows<IsDense<M>::value ? M::PARK_ROWS : 0> park;   // up/gate rows an O-projection leaves for the instruction behind it
};

#define QMK_ROWS_STAMP(k)                                                     \
  do {                                                                        \
    if (p.timeline != nullptr && c.tid == 0) s.b.stamps[k] = wall_clock64(); \
  } while (0)

template <class M>
__device__ __forceinline__ bool bad_operand(const Params& p, Smem<M>& s, const Ctx& c, int operand) {
  return qmk::bad_operand(p, s.b, c, operand);
}

// Row r's tagged-unit workspace.
__device__ __forceinline__ uint64_t* ws_of(const Params& p, int r) { return p.ws + static_cast<size_t>(r) * p.ws_row_units; }

// The launch parameters as row r's batch-1 launch would have them: every per-request pointer moved to the row's
// slice, the position the row's own.
template <class M>
__device__ __forceinline__ Params row_view(const Params& p, int r, int pos) {
  Params q = p;
  const size_t R = static_cast<size_t>(r);
  const size_t cache = static_cast<size_t>(p.kv_row_tokens) * M::NKV * M::D;
  q.pos_id = pos;
  q.max_seq_len = p.kv_layer_tokens;   // (the batch-1 ops use it for nothing but the distance between two layers' rows)
  q.hidden = p.hidden + R * M::H;
  q.q_post_rope = p.q_post_rope + R * M::AW;
  q.attn_out = p.attn_out + R * M::AW;
  q.k_cache = p.k_cache + R * cache;
  q.v_cache = p.v_cache + R * cache;
  q.attn_lse = p.attn_lse + R * M::NQ * p.max_splits;
  q.attn_partial = p.attn_partial + R * M::NQ * p.max_splits * M::D;
  q.silu_out = p.silu_out + R * (p.moe_ffn > 0 ? p.moe_ffn : M::F);
  q.logits = p.logits + R * p.vocab_size;
  q.qkv_raw = p.qkv_raw != nullptr ? p.qkv_raw + R * M::QKV : nullptr;
  q.router_logits = p.router_logits + R * p.num_experts;
  q.expert_indices = p.expert_indices + R * p.top_k;
  q.expert_weights = p.expert_weights + R * p.top_k;
  q.normed_hidden = p.normed_hidden + R * M::H;
  q.routed_silu = p.routed_silu + R * p.top_k * p.moe_ffn;
  q.routed_out_f32 = p.routed_out_f32 + R * M::H;
  q.routed_out = p.routed_out + R * M::H;
  q.ws = ws_of(p, r);
  // the per-head counters of a row's split-KV instructions (and the row's word on the reduction row) behind those of
  // the rows before it: NQ slots per row (the launcher checks that a counter row has room for all rows)
  q.barriers = p.barriers + r * M::NQ;
  return q;
}

// RMSNorm of every row's residual stream into s.x[row] (the batch-1 kernel's rms_to_lds per row: the same sums in
// the same order).  `region` >= 0: the rows' tagged units at that offset of their workspaces, each thread polling
// its own two per row, all rows in one trip; < 0: the caller's buffers (layer 0).  `pace(k)` issues the op's k-th
// group of weight-row requests, one group per look at the units.
template <class M, int NP, class Pace>
__device__ __forceinline__ bool rms_rows(const Params& p, Smem<M>& s, const Ctx& c, int region, uint32_t tag, const u16* weight, Pace pace) {
  constexpr int NR = RowsOf<M>::value;
  static_assert(M::H == kThreads * 4, "one thread normalises four elements of every row");
  const int t = c.tid, B = p.batch;
  const uint2 wv = *reinterpret_cast<const uint2*>(weight + t * 4);
  uint32_t lo[NR], hi[NR];
  static_for<0, NR>([&](auto b) { lo[b] = hi[b] = 0u; });
  bool done = region < 0;
  auto look = [&] {
    uint64_t xx[NR], yy[NR];
    static_for<0, NR>([&](auto b) {
      xx[b] = yy[b] = static_cast<uint64_t>(tag) << 32;
      if (s.live[b]) {
        const uint64_t* mine = ws_of(p, b) + region + 2 * t;
        xx[b] = ld_shared64(mine);
        yy[b] = ld_shared64(mine + 1);
      }
    });
    bool ok = true;
    static_for<0, NR>([&](auto b) {
      lo[b] = static_cast<uint32_t>(xx[b]);
      hi[b] = static_cast<uint32_t>(yy[b]);
      ok = ok && static_cast<uint32_t>(xx[b] >> 32) == tag && static_cast<uint32_t>(yy[b] >> 32) == tag;
    });
    done = __builtin_amdgcn_ballot_w64(ok) == ~0ull;   // the wave moves on together: row requests are wave-wide
  };
  static_for<0, NP>([&](auto kk) {
    pace(kk);
    if (!done) look();
  });
  if (region < 0) {
    static_for<0, NR>([&](auto b) {
      if (s.live[b]) {
        const uint64_t hw = ld_shared64(p.hidden + static_cast<size_t>(b) * M::H + t * 4);
        lo[b] = static_cast<uint32_t>(hw);
        hi[b] = static_cast<uint32_t>(hw >> 32);
      }
    });
  } else {
    for (uint32_t polls = 0; !done; ++polls) {
      if (polls > p.spin_limit) {
        s.b.ctl[0] = 1;
        report_error(p, QMK_DEV_WAIT_TIMEOUT, c.inst_idx, c.opcode, t);
        break;
      }
      if (polls) __builtin_amdgcn_s_sleep(1);
      look();
    }
    if (p.timeline != nullptr && t == 0) {
      s.b.t_wait = wall_clock64();
      s.b.ctl[2] = 1;
    }
  }
  float ss[NR];
  static_for<0, NR>([&](auto b) {
    const float x0 = bf_lo(lo[b]), x1 = bf_hi(lo[b]), x2 = bf_lo(hi[b]), x3 = bf_hi(hi[b]);
    ss[b] = wave_sum(__builtin_fmaf(x3, x3, __builtin_fmaf(x2, x2, __builtin_fmaf(x1, x1, x0 * x0))));
  });
  const int lane = t & 63, wave = t >> 6;
  __syncthreads();
  if (lane == 0) static_for<0, NR>([&](auto b) { s.red[0][b][wave] = ss[b]; });
  __syncthreads();
  // A row's scale by one thread (the wave sums added in the batch-1 kernel's order): every thread adding up every row's
  // sums and taking its root is thirty instructions per row and thread in front of every GEMV.
  if (t < NR) {
    float total = 0.f;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) total += s.red[0][t][w];
    const float mean = total / static_cast<float>(M::H);
    s.red[1][t][0] = 1.0f / sqrtf(mean + p.rms_norm_eps);
  }
  __syncthreads();
  static_for<0, NR>([&](auto b) {
    if (b < B) {
      const float rstd = s.red[1][b][0];
      const float x0 = bf_lo(lo[b]), x1 = bf_hi(lo[b]), x2 = bf_lo(hi[b]), x3 = bf_hi(hi[b]);
      const uint32_t n01 = f2bf2(x0 * rstd, x1 * rstd), n23 = f2bf2(x2 * rstd, x3 * rstd);
      uint2 out;
      out.x = f2bf2(bf_lo(wv.x) * bf_lo(n01), bf_hi(wv.x) * bf_hi(n01));
      out.y = f2bf2(bf_lo(wv.y) * bf_lo(n23), bf_hi(wv.y) * bf_hi(n23));
      *reinterpret_cast<uint2*>(&s.x[b][t * 4]) = out;
    }
  });
  __syncthreads();
  return s.b.ctl[0] == 0;
}

// The rows' activation vectors of H elements from s.x into registers (lane l: columns (j*64 + l)*8 .. +7 of chunk j).
template <class M, int CH, int NR>
__device__ __forceinline__ void load_x_rows(const Smem<M>& s, v4u (&x)[NR][CH], int lane) {
  static_for<0, NR>([&](auto b) { load_x_from_lds(x[b], &s.x[b][0], lane); });
}

// ===================================================================== 1 ==
// [1, layer, tile_M, n_start, n_end, tile_M_g, tile_N_g]   the QKV rows of the instruction for every row of the batch
template <class M>
__device__ bool op_qkv(const Params& p, Smem<M>& s, const Ctx& c) {
  constexpr int NR = RowsOf<M>::value;
  constexpr int CH = M::H / 512;
  const int layer = s.b.inst[1], nstart = s.b.inst[3], nend = s.b.inst[4], tile = s.b.inst[6];
  const int bph = p.qkv_blocks_per_head, B = p.batch;
  if (layer < 0 || layer >= p.num_layers) return bad_operand(p, s, c, 1);
  if (tile <= 0 || (tile & 1) || tile * bph != M::D) return bad_operand(p, s, c, 6);
  if (nstart < 0 || nend < nstart || static_cast<long>(nend) * tile > M::QKV) return bad_operand(p, s, c, 4);
  if ((nend - nstart) * tile > kRowRes) return bad_operand(p, s, c, 3);
  const int lane = c.tid & 63;
  const int rs = nstart * tile, nrows = (nend - nstart) * tile;
  const u16* W = p.qkv_w + (static_cast<size_t>(layer) * M::QKV + rs) * M::H;
  auto src = [&](int r) { return W + static_cast<size_t>(r) * M::H; };
  RowRegs<CH> buf[kDepth];
  const uint32_t tag = tag_of(s.b.generation, layer);
  if (!rms_rows<M, kDepth>(p, s, c, layer > 0 ? kWsHiddenOut : -1, tag - 1, p.attn_norm + static_cast<size_t>(layer) * M::H,
                           [&](auto k) { preload_range<decltype(k)::value, decltype(k)::value + 1>(nrows, src, buf); }))
    return false;
  QMK_ROWS_STAMP(0);
  v4u x[NR][CH];
  load_x_rows<M, CH>(s, x, lane);
  stream<CH>(nrows, src, buf, [&](int r, const RowRegs<CH>& w) {
    float sum[NR];
    static_for<0, NR>([&](auto b) { sum[b] = wave_sum(dot_row(w, x[b])); });
    if (lane == 0) static_for<0, NR>([&](auto b) { s.res[b][r] = sum[b]; });
  });
  QMK_ROWS_STAMP(1);
  __syncthreads();
  // Epilogue per (row, output pair): the GEMV result is bf16 before anything else happens to it.
  const int pairs = nrows / 2;
  for (int item = c.tid; item < B * pairs; item += kThreads) {
    const int b = item / pairs, pair = item % pairs;
    if (!s.live[b]) continue;
    const int r = rs + 2 * pair;
    float a0 = s.res[b][2 * pair], a1 = s.res[b][2 * pair + 1];
    if constexpr (M::QKV_BIAS) {
      const uint32_t bw = *reinterpret_cast<const uint32_t*>(p.qkv_bias + static_cast<size_t>(layer) * M::QKV + r);
      a0 += bf_lo(bw), a1 += bf_hi(bw);
    }
    const float v0 = round_bf16(a0), v1 = round_bf16(a1);
    uint64_t* ws = ws_of(p, b);
    constexpr int kq = M::NQ * M::D, kk = (M::NQ + M::NKV) * M::D;
    if constexpr (M::QK_NORM) {
      const uint32_t w = f2bf2(v0, v1);
      st_shared32(p.qkv_raw + static_cast<size_t>(b) * M::QKV + r, w);
      st_tagged(ws + (r < kq ? kWsQ + r / 2 : (r < kk ? kWsK + (r - kq) / 2 : kWsV + (r - kk) / 2)), w, tag);
    } else {
      const int pos = s.pos[b];
      const float* cosr = p.rope_cos + static_cast<size_t>(pos) * M::D;
      const float* sinr = p.rope_sin + static_cast<size_t>(pos) * M::D;
      const size_t kv_row = (static_cast<size_t>(b) * p.kv_row_tokens + static_cast<size_t>(layer) * p.kv_layer_tokens + pos) * (M::NKV * M::D);
      if (r < kq) {
        const uint32_t w = rope_pair(v0, v1, cosr, sinr, r % M::D);
        st_shared32(p.q_post_rope + static_cast<size_t>(b) * M::AW + r, w);
        st_tagged(ws + kWsQ + r / 2, w, tag);
      } else if (r < kk) {
        const int i = r - kq;
        const uint32_t w = rope_pair(v0, v1, cosr, sinr, i % M::D);
        st_shared32(p.k_cache + kv_row + i, w);
        st_tagged(ws + kWsK + i / 2, w, tag);
      } else {
        const int i = r - kk;
        const uint32_t w = f2bf2(v0, v1);
        st_shared32(p.v_cache + kv_row + i, w);
        st_tagged(ws + kWsV + i / 2, w, tag);
      }
    }
  }
  return true;   // the units announce themselves
}

// Every live row's word on the reduction row has reached `expected` (lane r polls row r's).  False (uniformly) on a timeout.
// `merged`: the count of the rows' merged head groups, which lives on the lines of the rows' workspaces when the
// launch has them (this XCD's line; the lines count through the layers).
template <class M>
__device__ __forceinline__ bool wait_rows(const Params& p, Smem<M>& s, const Ctx& c, int layer, int expected, bool merged = false) {
  const bool lines = merged && (p.flags & kFlagRowAttentionLines);
  if (c.tid < p.batch && s.live[c.tid] &&
      !(lines ? poll_counter(row_attention_line(ws_of(p, c.tid), p.ws_row_units, blockIdx.x & (kXcds - 1)), (layer + 1) * expected, p.spin_limit)
              : poll_counter(counter_ptr(p, layer, ROW_REDUCE, c.tid * M::NQ), expected, p.spin_limit))) {
    s.b.ctl[0] = 1;
    report_error(p, QMK_DEV_WAIT_TIMEOUT, c.inst_idx, c.opcode, c.tid);
  }
  if (p.timeline != nullptr && c.tid == 0) {
    s.b.t_wait = wall_clock64();
    s.b.ctl[2] = 1;
  }
  __syncthreads();
  return s.b.ctl[0] == 0;
}

// ===================================================================== 4 ==
// [4, layer, tile_M, n_start, n_end, P, tile_M_g, tile_N_g]
// Every row's split-KV partials merged by this workgroup itself (P per KV head: the batch-1 op's self-merge, row by
// row), then hidden[b][r] = bf16(hidden[b][r] + bf16(W_o[r] . attn_out[b])) for the instruction's rows r.
// `carry` / `carried` / `parked` (dense kernels): as in the batch-1 op, the first rows of the up/gate instruction behind
// this one are asked for in front of the wait for the attention phase — CARRY_ROWS per wave handed over in registers,
// PARK_ROWS more left in LDS.
template <class M, bool kCarry>
__device__ bool op_oproj(const Params& p, Smem<M>& s, const Ctx& c, Carried& carry, bool& carried, bool& parked) {
  constexpr int NR = RowsOf<M>::value;
  constexpr int AW = M::AW, CH = AW / 512;
  static_assert(AW % (kThreads * 4) == 0, "whole 8-byte pieces per thread");
  const int layer = s.b.inst[1], nstart = s.b.inst[3], nend = s.b.inst[4], P = s.b.inst[5], tile = s.b.inst[7];
  const int B = p.batch;
  if (layer < 0 || layer >= p.num_layers) return bad_operand(p, s, c, 1);
  if (tile <= 0 || (tile & 1)) return bad_operand(p, s, c, 7);
  if (nstart < 0 || nend < nstart || static_cast<long>(nend) * tile > M::H) return bad_operand(p, s, c, 4);
  if ((nend - nstart) * tile > kRowRes || B * (nend - nstart) * tile / 2 > kThreads) return bad_operand(p, s, c, 3);
  if (P < 0 || P > kMaxSelfMerge || P > p.max_splits) return bad_operand(p, s, c, 5);
  const int lane = c.tid & 63;
  const int rs = nstart * tile, nrows = (nend - nstart) * tile, pairs = nrows / 2;
  const u16* W = p.o_w + (static_cast<size_t>(layer) * M::H + rs) * AW;
  auto src = [&](int r) { return W + static_cast<size_t>(r) * AW; };
  RowRegs<CH> buf[kOprojBuffers];
  preload<CH>(nrows, src, buf);
  const uint32_t tag = tag_of(s.b.generation, layer);
  // the residual values this thread adds to: those the previous layer's commit announced (layer 0: the caller's buffer)
  const int my_b = c.tid / max(pairs, 1), my_pair = c.tid % max(pairs, 1);
  const bool adds = c.tid < B * pairs && s.live[my_b];
  uint32_t res_old = 0;
  if (adds) {
    if (layer == 0) {
      res_old = ld_shared32(p.hidden + static_cast<size_t>(my_b) * M::H + rs + 2 * my_pair);
    } else if (!poll_tagged1(ws_of(p, my_b) + kWsHiddenOut + (rs + 2 * my_pair) / 2, tag - 1, p.spin_limit, res_old)) {
      s.b.ctl[0] = 1;   // seen by everybody after the barrier inside the wait below
      report_error(p, QMK_DEV_WAIT_TIMEOUT, c.inst_idx, c.opcode, c.tid);
    }
  }
  if (P == 0) {
    if constexpr (kCarry) {
      carried = carried && s.b.next[0] == OP_RMS_UPGATE_SILU && s.b.next[1] == layer && upgate_check<M>(p, s.b.next) < 0;
      if (carried) {
        const int un = s.b.next[3], utile = s.b.next[5 + un];
        const int wave = c.tid >> 6;
        static_assert(M::CARRY_ROWS <= kCarried, "the carried rows fit the up/gate ring");
#pragma unroll
        for (int k = 0; k < M::CARRY_ROWS; ++k) {
          const int e = wave + (k + 1) * kWaves;
          if (e < 2 * un * utile) load_row(carry.row[k], upgate_row<M>(p, s.b.next, layer, utile, e), lane);
        }
      } else {
        forget(carry);
      }
      parked = parked && carried && M::PARK_ROWS > 0;
      if constexpr (M::PARK_ROWS > 0) {
        if (parked) {   // (the batch-1 kernel's park_upgate_rows on this kernel's LDS)
          const int un = s.b.next[3], utile = s.b.next[5 + un], wave = c.tid >> 6;
#pragma unroll 1
          for (int k = 0; k < M::PARK_ROWS; ++k) {
            const int e = wave + (kUpGateBuffers + k) * kWaves;
            if (e < 2 * un * utile) {
              RowRegs<4> r;
              load_row(r, upgate_row<M>(p, s.b.next, layer, utile, e), lane);
#pragma unroll
              for (int j = 0; j < 4; ++j) s.park.v[k][wave][j][lane] = r.v[j];
            }
          }
        }
      }
    }
    // The rows' attention outputs are complete in memory: the last split-KV arrival of every (row, KV head) merged its
    // group's partials and counted the group's heads on the row's word of the reduction row.  All rows in one trip.
    if (!wait_rows(p, s, c, layer, M::NQ, /*merged=*/true)) return false;
    constexpr int kPieces = (NR * AW + kThreads * 8 - 1) / (kThreads * 8);   // 16-byte pieces per thread
    v4u piece[kPieces];
#pragma unroll
    for (int k = 0; k < kPieces; ++k) {
      const int at = (c.tid + k * kThreads) * 8;            // element index in [B, AW]
      piece[k] = v4u{0, 0, 0, 0};
      if (at < B * AW) piece[k] = ld_shared128(p.attn_out + at);
    }
#pragma unroll
    for (int k = 0; k < kPieces; ++k) {
      const int at = (c.tid + k * kThreads) * 8;
      if (at < B * AW) *reinterpret_cast<v4u*>(&s.x[at / AW][at % AW]) = piece[k];
    }
  } else {
  if constexpr (kCarry) carried = parked = false;   // (this mode's merge needs the registers)
  // one arrival per split-KV instruction, on its row's word of the reduction row
  if (!wait_rows(p, s, c, layer, M::NKV * P)) return false;
  // Item t (one or two per thread) is dims 4*(t % (D/4)).. of head t / (D/4); four partials of every item per round,
  // all loads first — the batch-1 op's arithmetic, one row of the batch after the other.
  constexpr int kItems = AW / (kThreads * 4);
  for (int b = 0; b < B; ++b) {
    const float* lse_b = p.attn_lse + static_cast<size_t>(b) * M::NQ * p.max_splits;
    const float* part_b = p.attn_partial + static_cast<size_t>(b) * M::NQ * p.max_splits * M::D;
    const float* lse[kItems];
    const float* part[kItems];
    float mx[kItems], den[kItems], n0[kItems], n1[kItems], n2[kItems], n3[kItems];
#pragma unroll
    for (int k = 0; k < kItems; ++k) {
      const int item = c.tid + k * kThreads;
      const int h = item / (M::D / 4), d0 = 4 * (item % (M::D / 4));
      lse[k] = lse_b + static_cast<size_t>(h) * p.max_splits;
      part[k] = part_b + static_cast<size_t>(h) * p.max_splits * M::D + d0;
      mx[k] = -INFINITY;
      den[k] = n0[k] = n1[k] = n2[k] = n3[k] = 0.f;
    }
    for (int j0 = 0; j0 < P; j0 += 4) {
      float e[kItems][4];
      v4u o[kItems][4];
#pragma unroll
      for (int k = 0; k < kItems; ++k)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int j = min(j0 + q, P - 1);
          e[k][q] = (j0 + q < P) ? ld_shared_f32(lse[k] + j) : -INFINITY;
          o[k][q] = ld_shared128(part[k] + static_cast<size_t>(j) * M::D);
        }
#pragma unroll
      for (int k = 0; k < kItems; ++k) {
        float mn = mx[k];
#pragma unroll
        for (int q = 0; q < 4; ++q) mn = fmaxf(mn, e[k][q]);
        const float rescale = (mx[k] == -INFINITY) ? 0.f : exp2_fast(mx[k] - mn);
        den[k] *= rescale; n0[k] *= rescale; n1[k] *= rescale; n2[k] *= rescale; n3[k] *= rescale;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const float f = (e[k][q] == -INFINITY) ? 0.f : exp2_fast(e[k][q] - mn);
          den[k] += f;
          n0[k] = __builtin_fmaf(__uint_as_float(o[k][q].x), f, n0[k]);
          n1[k] = __builtin_fmaf(__uint_as_float(o[k][q].y), f, n1[k]);
          n2[k] = __builtin_fmaf(__uint_as_float(o[k][q].z), f, n2[k]);
          n3[k] = __builtin_fmaf(__uint_as_float(o[k][q].w), f, n3[k]);
        }
        mx[k] = mn;
      }
    }
#pragma unroll
    for (int k = 0; k < kItems; ++k) {
      const int item = c.tid + k * kThreads;
      const float inv = den[k] > 0.f ? 1.0f / den[k] : 0.f;
      const uint32_t lo = f2bf2(n0[k] * inv, n1[k] * inv);
      const uint32_t hi = f2bf2(n2[k] * inv, n3[k] * inv);
      *reinterpret_cast<uint2*>(&s.x[b][item * 4]) = make_uint2(lo, hi);
      if (nstart == 0) {  // one workgroup also leaves attn_out in memory, as the reference does
        u16* out = p.attn_out + static_cast<size_t>(b) * AW + item * 4;
        st_shared32(out, lo);
        st_shared32(out + 2, hi);
      }
    }
  }
  if constexpr (kCarry) forget(carry);
  }
  __syncthreads();
  QMK_ROWS_STAMP(0);
  if constexpr (CH <= 4) {
    // (an attention output as wide as the hidden state: the rows' vectors fit the registers beside this op's two row buffers)
    v4u x[NR][CH];
    load_x_rows<M, CH>(s, x, lane);
    stream<CH>(nrows, src, buf, [&](int r, const RowRegs<CH>& w) {
      float sum[NR];
      static_for<0, NR>([&](auto b) { sum[b] = wave_sum(dot_row(w, x[b])); });
      if (lane == 0) static_for<0, NR>([&](auto b) { s.res[b][r] = sum[b]; });
    });
  } else {
    // The activation pieces come from LDS as they are used (CH * rows of them do not fit the registers beside the rows).
    stream<CH>(nrows, src, buf, [&](int r, const RowRegs<CH>& w) {
      static_for<0, NR>([&](auto b) {
        float a = 0.f;
#pragma unroll
        for (int j = 0; j < CH; ++j) a = dot8(w.v[j], *reinterpret_cast<const v4u*>(&s.x[b][(j * kWaveSize + lane) * 8]), a);
        const float sum = wave_sum(a);
        if (lane == 0) s.res[b][r] = sum;
      });
    });
  }
  QMK_ROWS_STAMP(1);
  __syncthreads();
  if (adds) {
    const uint32_t w = residual_word(res_old, s.res[my_b][2 * my_pair], s.res[my_b][2 * my_pair + 1]);
    st_tagged(ws_of(p, my_b) + kWsHiddenMid + (rs + 2 * my_pair) / 2, w, tag);
    st_shared32(p.hidden + static_cast<size_t>(my_b) * M::H + rs + 2 * my_pair, w);
  }
  return true;
}

template <class M>
__device__ __forceinline__ bool op_oproj(const Params& p, Smem<M>& s, const Ctx& c) {
  Carried none;
  bool no = false, neither = false;
  return op_oproj<M, false>(p, s, c, none, no, neither);
}

// ===================================================================== 8 ==
// [8, layer, e_start, e_end, write_normed_hidden, tile_N_g]   router logits of the instruction's experts for every row
template <class M>
__device__ bool op_router(const Params& p, Smem<M>& s, const Ctx& c) {
  constexpr int CH = M::H / 512;
  const int layer = s.b.inst[1], g = s.b.inst[5], e0 = s.b.inst[2] * g, e1 = min(s.b.inst[3] * g, p.num_experts);
  const int B = p.batch;
  if (layer < 0 || layer >= p.num_layers) return bad_operand(p, s, c, 1);
  if (g < 1 || e0 < 0 || e1 < e0) return bad_operand(p, s, c, 2);
  const int lane = c.tid & 63, wave = c.tid >> 6;
  const u16* w = p.router_w + static_cast<size_t>(layer) * p.num_experts * M::H;
  const uint32_t tag = tag_of(s.b.generation, layer);
  RowRegs<CH> first;   // the wave's first expert row lands during the wait for the residual stream
#pragma unroll
  for (int j = 0; j < CH; ++j) first.v[j] = v4u{0, 0, 0, 0};
  if (e0 + wave < e1) load_row(first, w + static_cast<size_t>(e0 + wave) * M::H, lane);
  if (!rms_rows<M, 0>(p, s, c, kWsHiddenMid, tag, p.mlp_norm + static_cast<size_t>(layer) * M::H, [](auto) {})) return false;
  v4u x[kMaxRows][CH];
  load_x_rows<M, CH>(s, x, lane);
  for (int e = e0 + wave; e < e1; e += kWaves) {
    RowRegs<CH> row = first;
    if (e != e0 + wave) load_row(row, w + static_cast<size_t>(e) * M::H, lane);
    float v[kMaxRows];
    static_for<0, kMaxRows>([&](auto b) { v[b] = wave_sum(dot_row(row, x[b])); });
    static_for<0, kMaxRows>([&](auto b) {
      if (lane == b && b < B) {
        st_shared_f32(p.router_logits + static_cast<size_t>(b) * p.num_experts + e, v[b]);
        st_tagged(ws_of(p, b) + kWsLogits + e * kLogitStride, __float_as_uint(v[b]), tag);
      }
    });
  }
  if (s.b.inst[4] != 0)   // one instruction of a layer also leaves the normalised rows, as opcode 8 of the batch-1 route does
    for (int i = c.tid * 2; i < B * M::H; i += kThreads * 2)
      st_shared32(p.normed_hidden + i, *reinterpret_cast<const uint32_t*>(&s.x[i / M::H][i % M::H]));
  return true;
}

// The routing decision of every row, taken by the consumer itself from the router's logits as they announce
// themselves (the batch-1 kernel's rank_experts and renormalisation per row: the same function of the same 32-bit
// values, the sums added in the same order), then the rows' picks merged into the list of distinct experts in
// ascending order — the same list in every workgroup.  Thread t works for row t / per, expert t % per, where per is
// the expert count rounded up to whole waves (the launcher checks rows * per <= threads), so that a row's softmax sums
// are added up wave by wave exactly as the batch-1 kernel adds them.  Taken once per layer and workgroup.
template <class M>
__device__ __forceinline__ bool route_rows(const Params& p, Smem<M>& s, const Ctx& c, int layer) {
  if (s.route_layer == layer) {
    if (p.timeline != nullptr && c.tid == 0) {
      s.b.t_wait = wall_clock64();
      s.b.ctl[2] = 1;
    }
    return true;
  }
  const int E = p.num_experts, B = p.batch, K = p.top_k;
  const int per = ((E + kWaveSize - 1) / kWaveSize) * kWaveSize, waves_per_row = per / kWaveSize;
  const int t = c.tid, lane = t & 63, wave = t >> 6;
  const int r = t / per, e = t % per;
  const bool live = r < B && e < E;
  const uint32_t tag = tag_of(s.b.generation, layer);
  uint32_t bits = 0;
  if (live && !poll_tagged1(ws_of(p, r) + kWsLogits + e * kLogitStride, tag, p.spin_limit, bits)) {
    s.b.ctl[0] = 1;
    report_error(p, QMK_DEV_WAIT_TIMEOUT, c.inst_idx, c.opcode, t);
  }
  if (p.timeline != nullptr && t == 0) {
    s.b.t_wait = wall_clock64();
    s.b.ctl[2] = 1;
  }
  const float logit = __uint_as_float(bits);
  const float wmax = wave_max(live ? logit : -INFINITY);
  __syncthreads();
  QMK_ROWS_STAMP(2);   // every thread has its logit
  if (lane == 0) s.red[0][0][wave] = wmax;
  if (t == 0) s.no_order = 0;
  if (t < kMaxRows * moe::kMaxTopK) {
    s.picked_p[t / moe::kMaxTopK][t % moe::kMaxTopK] = 0.f;
    s.picked_e[t / moe::kMaxTopK][t % moe::kMaxTopK] = -1;
  }
  __syncthreads();
  if (s.b.ctl[0]) return false;
  float mx = -INFINITY;
  if (r < B)
    for (int w = 0; w < waves_per_row; ++w) mx = fmaxf(mx, s.red[0][0][r * waves_per_row + w]);
  const float x = live ? expf(logit - mx) : 0.f;
  // An expert goes before another when its probability is larger, or equal with the lower index: one unsigned compare
  // of {numerator bits (not negative: ordered like the floats), ~index}.  Padded to pairs with keys nobody goes behind.
  const int padded = (E + 1) & ~1;
  const uint64_t my_key = (static_cast<uint64_t>(__float_as_uint(x)) << 32) | (0xffffffffu - static_cast<uint32_t>(e));
  if (r < B && e < padded) s.moe.key[r][e] = live ? my_key : 0ull;
  const float wsum = wave_sum(x);
  if (lane == 0) s.red[1][0][wave] = wsum;
  __syncthreads();
  float sum = 0.f;
  if (r < B)
    for (int w = 0; w < waves_per_row; ++w) sum += s.red[1][0][r * waves_per_row + w];
  const bool ok = !(r < B) || (sum > 0.f && sum < INFINITY);
  if (!ok) s.no_order = 1;   // a logit is NaN or infinite: no order to pick by
  if (live && ok) {
    typedef uint64_t u64x2 __attribute__((ext_vector_type(2)));
    const u64x2* all = reinterpret_cast<const u64x2*>(&s.moe.key[r][0]);
    int before = 0;
#pragma unroll 8
    for (int k = 0; k < padded; k += 2) {
      const u64x2 v = all[k >> 1];
      before += v.x > my_key ? 1 : 0;
      before += v.y > my_key ? 1 : 0;
    }
    if (before < K) {
      s.picked_p[r][before] = x / sum;
      s.picked_e[r][before] = e;
    }
  }
  __syncthreads();
  if (s.no_order) return bad_operand(p, s, c, 2);
  if (t < B * K) {   // norm_topk_prob: the picks' probabilities divided by their sum, added up in slot order (fp32)
    const int rr = t / K, j = t % K;
    float pk[moe::kMaxTopK];
    *reinterpret_cast<float4*>(&pk[0]) = *reinterpret_cast<const float4*>(&s.picked_p[rr][0]);
    *reinterpret_cast<float4*>(&pk[4]) = *reinterpret_cast<const float4*>(&s.picked_p[rr][4]);
    float total = 0.f;
#pragma unroll
    for (int q = 0; q < moe::kMaxTopK; ++q) total += q < K ? pk[q] : 0.f;
    s.route_expert[rr][j] = s.picked_e[rr][j];
    s.route_weight[rr][j] = p.norm_topk ? s.picked_p[rr][j] / total : s.picked_p[rr][j];
  }
  __syncthreads();
  // distinct experts in ascending order: thread e (< E) knows whether anybody picked expert e and in which slots
  int slot_of[kMaxRows];
  bool present = false;
  static_for<0, kMaxRows>([&](auto b) {
    slot_of[b] = -1;
    if (t < E && b < B) {
      int picks[moe::kMaxTopK];
      *reinterpret_cast<int4*>(&picks[0]) = *reinterpret_cast<const int4*>(&s.route_expert[b][0]);
      *reinterpret_cast<int4*>(&picks[4]) = *reinterpret_cast<const int4*>(&s.route_expert[b][4]);
#pragma unroll
      for (int j = 0; j < moe::kMaxTopK; ++j)
        if (j < K && picks[j] == t) slot_of[b] = j;
    }
    present = present || slot_of[b] >= 0;
  });
  const uint64_t mask = __builtin_amdgcn_ballot_w64(present);
  if (lane == 0) s.wave_count[wave] = __builtin_popcountll(mask);
  __syncthreads();
  int offset = 0, total = 0;
  for (int w = 0; w < kWaves; ++w) {
    offset += w < wave ? s.wave_count[w] : 0;
    total += s.wave_count[w];
  }
  if (present) {
    const int u = offset + __builtin_popcountll(mask & ((1ull << lane) - 1ull));
    if (u < kMaxList) {
      s.list_expert[u] = t;
      static_for<0, kMaxRows>([&](auto b) { s.list_slot[u][b] = slot_of[b]; });
    }
  }
  if (t == 0) {
    s.n_list = min(total, kMaxList);
    s.route_layer = layer;
  }
  __syncthreads();
  QMK_ROWS_STAMP(3);   // the list of distinct experts is complete
  return true;
}

// ==================================================================== 15 ==
// [15, layer, part, nparts, tile_N_g]
// The gate and up rows of every DISTINCT expert the rows of the batch picked in this layer, streamed once against the
// normalised residual streams of all rows: item g = (list entry g / (F/2), output pair g % (F/2)); wave w of the
// instruction takes the items part*8 + w, + nparts*8, ... (dealt at run time: the length of the list is not known
// to the scheduler).  silu = bf16(silu(bf16(gate . x)) * bf16(up . x)) as in opcode 12 (python_vm.py:421-464), for every
// row that picked the expert, into that row's slot: routed_silu[row][slot] and the slot's tagged units.  A wave owns
// both outputs of a pair (four weight rows, 16 KiB in flight), so nothing is exchanged between waves.
template <class M>
__device__ bool op_routed_upgate(const Params& p, Smem<M>& s, const Ctx& c) {
  constexpr int CH = M::H / 512;
  const int layer = s.b.inst[1], part = s.b.inst[2], nparts = s.b.inst[3];
  const int B = p.batch, F = p.moe_ffn, K = p.top_k;
  if (layer < 0 || layer >= p.num_layers) return bad_operand(p, s, c, 1);
  if (nparts < 1 || part < 0 || part >= nparts) return bad_operand(p, s, c, 2);
  const int lane = c.tid & 63, wave = c.tid >> 6;
  const uint32_t tag = tag_of(s.b.generation, layer);
  // the normalised rows long before the experts are known
  if (!rms_rows<M, 0>(p, s, c, kWsHiddenMid, tag, p.mlp_norm + static_cast<size_t>(layer) * M::H, [](auto) {})) return false;
  QMK_ROWS_STAMP(0);
  if (!route_rows<M>(p, s, c, layer)) return false;
  QMK_ROWS_STAMP(1);
  const int ppe = F / 2, total = s.n_list * ppe, stride = nparts * kWaves;
  const u16* base = p.expert_gate_up_w + static_cast<size_t>(layer) * p.num_experts * 2 * F * M::H;
  RowRegs<CH> w[4];   // gate o, gate o+1, up o, up o+1
  auto request = [&](int g) {
    if (g >= total) return;
    const int u = g / ppe, o = 2 * (g % ppe);
    const u16* ex = base + static_cast<size_t>(s.list_expert[u]) * 2 * F * M::H;
    load_row(w[0], ex + static_cast<size_t>(o) * M::H, lane);
    load_row(w[1], ex + static_cast<size_t>(o + 1) * M::H, lane);
    load_row(w[2], ex + static_cast<size_t>(F + o) * M::H, lane);
    load_row(w[3], ex + static_cast<size_t>(F + o + 1) * M::H, lane);
  };
  int g = part * kWaves + wave;
  request(g);
  v4u x[kMaxRows][CH];
  load_x_rows<M, CH>(s, x, lane);
  for (; g < total; g += stride) {
    float v[4][kMaxRows];
    static_for<0, 4>([&](auto k) { static_for<0, kMaxRows>([&](auto b) { v[k][b] = wave_sum(dot_row(w[k], x[b])); }); });
    const int u = g / ppe, o = 2 * (g % ppe);
    request(g + stride);
    static_for<0, kMaxRows>([&](auto b) {
      if (lane == b && b < B) {
        const int j = s.list_slot[u][b];
        if (j >= 0) {
          const float g0 = round_bf16(v[0][b]), g1 = round_bf16(v[1][b]);
          const float a0 = (g0 / (1.0f + expf(-g0))) * round_bf16(v[2][b]);
          const float a1 = (g1 / (1.0f + expf(-g1))) * round_bf16(v[3][b]);
          const uint32_t word = f2bf2(a0, a1);
          st_shared32(p.routed_silu + (static_cast<size_t>(b) * K + j) * F + o, word);
          if (j == K - 1) st_shared32(p.silu_out + static_cast<size_t>(b) * F + o, word);   // what the last slot leaves, as after the VM's run
          st_tagged(ws_of(p, b) + kWsRoutedSilu + j * 1024 + o / 2, word, tag);
        }
      }
    });
  }
  return true;
}

// ==================================================================== 16 ==
// [16, layer, n_start, n_end, tile_N_g]
// ALL distinct experts of the rows [r0, r0 + n) of the residual stream and the commit, for every row of the batch:
// wave w takes the list entries w, w + 8, ...; for each it streams the expert's n down-projection rows once (in halves
// of four rows through a ring of two buffers) and multiplies them with the silu vector of every row that picked the
// expert (looked at as tagged units, straight into registers: exactly the units its pieces multiply), leaving
// bf16(W_down[e][r] . silu) * weight in the (row, slot) the expert has there.  Then, per row, the slots' terms are
// added in slot order in fp32 and committed, hidden[b][r] = bf16(hidden[b][r] + routed[b][r])  (python_vm.py:467-530
// without a shared expert): the batch-1 route's committing instruction for every row.
template <class M>
__device__ bool op_routed_down_commit(const Params& p, Smem<M>& s, const Ctx& c) {
  constexpr int kChunks = 2, kHalf = 4;   // an expert's width is at most 1024: two 512-column chunks per row
  const int layer = s.b.inst[1], n0 = s.b.inst[2], n1 = s.b.inst[3], tile = s.b.inst[4];
  const int B = p.batch, K = p.moe_ffn, TK = p.top_k;
  if (layer < 0 || layer >= p.num_layers) return bad_operand(p, s, c, 1);
  if ((tile != 8 && tile != 16) || n0 < 0 || n1 <= n0 || n1 * tile > M::H || (n1 - n0) * tile > kCommitRows) return bad_operand(p, s, c, 3);
  const int lane = c.tid & 63, wave = c.tid >> 6;
  const int r0 = n0 * tile, n = (n1 - n0) * tile, pairs = n / 2;
  const uint32_t tag = tag_of(s.b.generation, layer);
  if (!route_rows<M>(p, s, c, layer)) return false;
  const int halves = n / kHalf;                       // 2 or 4
  const int mine = s.n_list > wave ? (s.n_list - wave + kWaves - 1) / kWaves : 0;   // list entries of this wave
  const int nsteps = mine * halves;
  const u16* base = p.expert_down_w + static_cast<size_t>(layer) * p.num_experts * M::H * K;
  constexpr int kRing = 3;   // half tiles of a wave in flight (6 KiB each for an expert width of 768)
  v4u ring[kRing][kHalf][kChunks];
  auto request = [&](auto slot, int step) {
    static_for<0, kHalf>([&](auto i) { static_for<0, kChunks>([&](auto q) { ring[slot][i][q] = v4u{0, 0, 0, 0}; }); });
    if (step >= nsteps) return;
    const int u = wave + kWaves * (step / halves), h = step % halves;
    const u16* rows = base + (static_cast<size_t>(s.list_expert[u]) * M::H + r0 + h * kHalf) * K + lane * 8;
    static_for<0, kHalf>([&](auto i) {
      static_for<0, kChunks>([&](auto q) {
        if (lane * 8 + q * 512 < K) ring[slot][i][q] = __builtin_nontemporal_load(reinterpret_cast<const v4u*>(rows + static_cast<size_t>(i) * K + q * 512));
      });
    });
  };
  static_for<0, kRing>([&](auto k) { request(k, k); });
  // the residual pair this thread commits, from the unit the O-projection announced it in
  const int my_b = c.tid / pairs, my_pair = c.tid % pairs;
  const bool commits = c.tid < B * pairs;
  uint32_t old = 0;
  if (commits && !poll_tagged1(ws_of(p, my_b) + kWsHiddenMid + (r0 + 2 * my_pair) / 2, tag, p.spin_limit, old)) {
    s.b.ctl[0] = 1;   // seen by everybody after the barrier in front of the commit
    report_error(p, QMK_DEV_WAIT_TIMEOUT, c.inst_idx, c.opcode, c.tid);
  }
  v4u x[kMaxRows][kChunks];   // columns lane*8 + q*512 .. +7 of the silu vector of (row, its slot for the entry)
  auto step_of = [&](auto slot, int step) {
    if (step >= nsteps) return;
    const int u = wave + kWaves * (step / halves), h = step % halves;
    if (h == 0) {   // a new list entry: the silu vectors of the rows that picked it
      static_for<0, kMaxRows>([&](auto b) { static_for<0, kChunks>([&](auto q) { x[b][q] = v4u{0, 0, 0, 0}; }); });
      uint32_t polls = 0;
      while (true) {
        bool all = true;
        static_for<0, kMaxRows>([&](auto b) {
          const int j = b < B ? s.list_slot[u][b] : -1;
          if (j >= 0) {   // uniform over the wave
            const uint64_t* units = ws_of(p, b) + kWsRoutedSilu + j * 1024 + lane * 4;
            uint64_t un[kChunks][4];
            static_for<0, kChunks>([&](auto q) {
              static_for<0, 4>([&](auto k) {
                un[q][k] = static_cast<uint64_t>(tag) << 32;
                if (lane * 8 + q * 512 < K) un[q][k] = ld_shared64(units + q * 256 + k);
              });
            });
            static_for<0, kChunks>([&](auto q) {
              static_for<0, 4>([&](auto k) { all = all && static_cast<uint32_t>(un[q][k] >> 32) == tag; });
              x[b][q] = v4u{static_cast<uint32_t>(un[q][0]), static_cast<uint32_t>(un[q][1]), static_cast<uint32_t>(un[q][2]), static_cast<uint32_t>(un[q][3])};
            });
          }
        });
        if (__builtin_amdgcn_ballot_w64(all) == ~0ull) break;
        if (++polls > p.spin_limit) {
          s.b.ctl[0] = 1;
          report_error(p, QMK_DEV_WAIT_TIMEOUT, c.inst_idx, c.opcode, u);
          break;
        }
        __builtin_amdgcn_s_sleep(1);
      }
    }
    static_for<0, kMaxRows>([&](auto b) {
      const int j = b < B ? s.list_slot[u][b] : -1;
      if (j >= 0) {
        float v[kHalf];
        static_for<0, kHalf>([&](auto i) {
          float a = 0.f;
          static_for<0, kChunks>([&](auto q) { a = dot8(ring[slot][i][q], x[b][q], a); });
          v[i] = wave_sum(a);
        });
        if (lane == 0) {
          const float weight = s.route_weight[b][j];
          static_for<0, kHalf>([&](auto i) { s.moe.terms[b][j][h * kHalf + i] = round_bf16(v[i]) * weight; });
        }
      }
    });
    request(slot, step + kRing);
  };
  if (p.timeline != nullptr && c.tid == 0) {
    s.b.t_wait = wall_clock64();
    s.b.ctl[2] = 1;
  }
  for (int step = 0; step < nsteps; step += kRing) static_for<0, kRing>([&](auto k) { step_of(k, step + k); });
  QMK_ROWS_STAMP(1);
  __syncthreads();
  if (s.b.ctl[0]) return false;
  if (commits) {
    const int r = r0 + 2 * my_pair;
    float ro0 = 0.f, ro1 = 0.f;
    for (int j = 0; j < TK; ++j) {
      ro0 += s.moe.terms[my_b][j][2 * my_pair];
      ro1 += s.moe.terms[my_b][j][2 * my_pair + 1];
    }
    const float h0 = (bf_lo(old) + ro0) + 0.f, h1 = (bf_hi(old) + ro1) + 0.f;   // opcode 14's expression without a shared term
    const uint32_t word = f2bf2(h0, h1);
    st_shared32(p.hidden + static_cast<size_t>(my_b) * M::H + r, word);
    st_tagged(ws_of(p, my_b) + kWsHiddenOut + r / 2, word, tag);
    st_shared_f32(p.routed_out_f32 + static_cast<size_t>(my_b) * M::H + r, 0.f);
    st_shared_f32(p.routed_out_f32 + static_cast<size_t>(my_b) * M::H + r + 1, 0.f);
  }
  // how many distinct experts the layer streamed: what the step's algorithmic bytes are counted from
  if (n0 == 0 && c.tid == 0 && p.distinct_out != nullptr) p.distinct_out[layer] = s.n_list;
  __syncthreads();   // s.moe.terms is read: the next instruction may write it
  return true;
}

// ===================================================================== 5 ==
// [5, layer, tile_M, n, block_0..block_{n-1}, tile_M_g, tile_N_g]   dense MLP, every row of the batch:
// silu_out[b] = bf16(bf16(silu(bf16(W_g y_b))) * bf16(W_u y_b))  (operations.py:265-282; the batch-1 op's arithmetic per row)
template <class M>
__device__ bool op_upgate(const Params& p, Smem<M>& s, const Ctx& c, const Carried& carry, bool carried, bool parked) {
  constexpr int NR = RowsOf<M>::value;
  constexpr int CH = M::H / 512;
  static_assert(CH == 4, "the carried rows are 4 KiB");
  const int bad = upgate_check<M>(p, s.b.inst);
  if (bad >= 0) return bad_operand(p, s, c, bad);
  const int layer = s.b.inst[1], n = s.b.inst[3], B = p.batch;
  const int tile = s.b.inst[5 + n];
  const int lane = c.tid & 63, wave = c.tid >> 6;
  const int nout = n * tile, nrows = 2 * nout;     // streamed rows: element 2i = up row i, 2i+1 = gate row i
  if (nrows > kRowRes) return bad_operand(p, s, c, 3);
  auto row_of = [&](int i) { return s.b.inst[4 + i / tile] * tile + i % tile; };
  auto src = [&](int e) { return upgate_row<M>(p, s.b.inst, layer, tile, e); };
  bool in_lds = false;   // the O-projection before this instruction has left rows kUpGateBuffers.. of every wave in LDS
  if constexpr (M::PARK_ROWS > 0) in_lds = parked && carried;
  RowRegs<CH> buf[kUpGateBuffers];
  if (carried) {  // ... and has asked for the elements of buffers 1..
#pragma unroll
    for (int k = 0; k < M::CARRY_ROWS; ++k) buf[k + 1] = carry.row[k];
  }
  const uint32_t tag = tag_of(s.b.generation, layer);
  if (!rms_rows<M, kUpGateBuffers>(p, s, c, kWsHiddenMid, tag, p.mlp_norm + static_cast<size_t>(layer) * M::H, [&](auto k) {
        constexpr int kk = decltype(k)::value;
        if (kk == 0 || kk > M::CARRY_ROWS || !carried) preload_range<kk, kk + 1>(nrows, src, buf);
      }))
    return false;
  QMK_ROWS_STAMP(0);
  v4u x[NR][CH];
  load_x_rows<M, CH>(s, x, lane);
  auto use = [&](int e, const RowRegs<CH>& w) {
    float sum[NR];
    static_for<0, NR>([&](auto b) { sum[b] = wave_sum(dot_row(w, x[b])); });
    if (lane == 0) static_for<0, NR>([&](auto b) { s.res[b][e] = sum[b]; });
  };
  // The ring holds the wave's first kUpGateBuffers rows and, when they were parked, LDS the PARK_ROWS behind them: a ring
  // buffer is refilled with the row behind those, and the parked rows are used while the refills are on their way.
  int pk = 0;
  if constexpr (M::PARK_ROWS > 0) pk = in_lds ? M::PARK_ROWS : 0;
  const int shift = (kUpGateBuffers + pk) * kWaves;
#pragma unroll
  for (int k = 0; k < kUpGateBuffers; ++k) {
    const int e = wave + k * kWaves;
    if (e < nrows) {
      use(e, buf[k]);
      if (e + shift < nrows) load_row(buf[k], src(e + shift), lane);
    }
  }
  if constexpr (M::PARK_ROWS > 0) {
#pragma unroll 1
    for (int k = 0; k < pk; ++k) {
      const int e = wave + (kUpGateBuffers + k) * kWaves;
      if (e < nrows) {
        RowRegs<CH> r;
#pragma unroll
        for (int q = 0; q < CH; ++q) r.v[q] = s.park.v[k][wave][q][lane];
        use(e, r);
      }
    }
  }
  stream<CH>(nrows - shift, [&](int e) { return src(e + shift); }, buf, [&](int e, const RowRegs<CH>& w) { use(e + shift, w); });
  QMK_ROWS_STAMP(1);
  __syncthreads();
  const int pairs = nout / 2;
  for (int item = c.tid; item < B * pairs; item += kThreads) {
    const int b = item / pairs, pair = item % pairs;
    uint32_t word = 0;
    if (s.live[b]) {
      const uint32_t ug0 = f2bf2(s.res[b][4 * pair], s.res[b][4 * pair + 1]), ug1 = f2bf2(s.res[b][4 * pair + 2], s.res[b][4 * pair + 3]);
      const float g0 = bf_hi(ug0), g1 = bf_hi(ug1);
      const uint32_t act = f2bf2(g0 / (1.0f + expf(-g0)), g1 / (1.0f + expf(-g1)));
      word = f2bf2(bf_lo(act) * bf_lo(ug0), bf_hi(act) * bf_lo(ug1));
      st_tagged(ws_of(p, b) + kWsSilu + row_of(2 * pair) / 2, word, tag);
    }
    st_shared32(p.silu_out + static_cast<size_t>(b) * M::F + row_of(2 * pair), word);   // zeros for a row that is not decoded
  }
  return true;
}

// ===================================================================== 6 ==
// [6, layer, tile_M, n_start, n_end, split_K_idx, tile_M_g, tile_N_g, split_K_g]   one K slice over the whole F only:
// hidden[b][r] = bf16(hidden[b][r] + bf16(W_d[r] . silu_out[b])) for every row of the batch  (operations.py:285-295)
template <class M>
__device__ bool op_down(const Params& p, Smem<M>& s, const Ctx& c) {
  constexpr int NR = RowsOf<M>::value;
  constexpr int CH = 4;
  static_assert(M::F % (4 * kThreads) == 0 && M::F <= XWidth<M>::value, "whole unit pairs per thread; the vectors fit");
  const int layer = s.b.inst[1], nstart = s.b.inst[3], nend = s.b.inst[4], split = s.b.inst[5];
  const int tile = s.b.inst[7], kg = s.b.inst[8], B = p.batch;
  if (layer < 0 || layer >= p.num_layers) return bad_operand(p, s, c, 1);
  if (tile <= 0 || (tile & 1)) return bad_operand(p, s, c, 7);
  if (nstart < 0 || nend < nstart || static_cast<long>(nend) * tile > M::H) return bad_operand(p, s, c, 4);
  if ((nend - nstart) * tile > kRowRes || B * (nend - nstart) * tile / 2 > kThreads) return bad_operand(p, s, c, 3);
  if (split != 0 || kg != M::F) return bad_operand(p, s, c, 8);
  const int lane = c.tid & 63, wave = c.tid >> 6;
  const int rs = nstart * tile, nrows = (nend - nstart) * tile, pairs = nrows / 2;
  constexpr int segs = M::F / (512 * CH);
  auto row_of = [&](int e) { return (e & (kWaves - 1)) + kWaves * ((e >> 3) / segs); };
  auto seg_of = [&](int e) { return (e >> 3) % segs; };
  const u16* W = p.down_w + (static_cast<size_t>(layer) * M::H + rs) * M::F;
  auto src = [&](int e) { return W + static_cast<size_t>(row_of(e)) * M::F + seg_of(e) * (512 * CH); };
  const int rows_w = (nrows - wave + kWaves - 1) / kWaves;
  const int n_elems = rows_w > 0 ? wave + kWaves * (rows_w * segs - 1) + 1 : 0;
  RowRegs<CH> buf[kDepth];
  preload_range<0, kEarly>(n_elems, src, buf);
  const uint32_t tag = tag_of(s.b.generation, layer);
  const int my_b = c.tid / max(pairs, 1), my_pair = c.tid % max(pairs, 1);
  const bool adds = c.tid < B * pairs && s.live[my_b];
  uint32_t res_old = 0;
  if (adds && !poll_tagged1(ws_of(p, my_b) + kWsHiddenMid + (rs + 2 * my_pair) / 2, tag, p.spin_limit, res_old)) {
    s.b.ctl[0] = 1;
    report_error(p, QMK_DEV_WAIT_TIMEOUT, c.inst_idx, c.opcode, c.tid);
  }
  // silu_out of every live row from its tagged units: thread t looks at the unit pairs 2t + 1024k of every row until
  // they carry this layer's tag; what has been staged is not fetched again.
  {
    constexpr int kPairs = M::F / (4 * kThreads);
    bool have[NR][kPairs];
    static_for<0, NR>([&](auto b) {
#pragma unroll
      for (int k = 0; k < kPairs; ++k) have[b][k] = !s.live[b];
    });
    for (uint32_t polls = 0;; ++polls) {
      bool all = true;
      static_for<0, NR>([&](auto b) {
        if (s.live[b]) {
          const uint64_t* mine = ws_of(p, b) + kWsSilu + 2 * c.tid;
          uint32_t* words = reinterpret_cast<uint32_t*>(&s.x[b][0]);
          uint64_t u[2 * kPairs];
#pragma unroll
          for (int k = 0; k < kPairs; ++k)
            if (!have[b][k]) {
              u[2 * k] = ld_shared64(mine + 1024 * k);
              u[2 * k + 1] = ld_shared64(mine + 1024 * k + 1);
            }
#pragma unroll
          for (int k = 0; k < kPairs; ++k) {
            if (!have[b][k] && static_cast<uint32_t>(u[2 * k] >> 32) == tag && static_cast<uint32_t>(u[2 * k + 1] >> 32) == tag) {
              words[2 * c.tid + 1024 * k] = static_cast<uint32_t>(u[2 * k]);
              words[2 * c.tid + 1024 * k + 1] = static_cast<uint32_t>(u[2 * k + 1]);
              have[b][k] = true;
            }
            all = all && have[b][k];
          }
        }
      });
      if (all) break;
      if (polls > p.spin_limit) {
        s.b.ctl[0] = 1;
        report_error(p, QMK_DEV_WAIT_TIMEOUT, c.inst_idx, c.opcode, c.tid);
        break;
      }
      __builtin_amdgcn_s_sleep(8);
    }
  }
  preload_range<kEarly, kDepth>(n_elems, src, buf);
  if (p.timeline != nullptr && c.tid == 0) {
    s.b.t_wait = wall_clock64();
    s.b.ctl[2] = 1;
  }
  __syncthreads();
  if (s.b.ctl[0]) return false;
  float acc[NR];
  static_for<0, NR>([&](auto b) { acc[b] = 0.f; });
  stream<CH>(n_elems, src, buf, [&](int e, const RowRegs<CH>& w) {
    const int seg = seg_of(e);
    static_for<0, NR>([&](auto b) {
#pragma unroll
      for (int j = 0; j < CH; ++j) acc[b] = dot8(w.v[j], *reinterpret_cast<const v4u*>(&s.x[b][seg * (512 * CH) + (j * kWaveSize + lane) * 8]), acc[b]);
    });
    if (seg == segs - 1) {
      static_for<0, NR>([&](auto b) {
        const float sum = wave_sum(acc[b]);
        acc[b] = 0.f;
        if (lane == 0) s.res[b][row_of(e)] = sum;
      });
    }
  });
  QMK_ROWS_STAMP(1);
  __syncthreads();
  if (adds) {
    const uint32_t w = residual_word(res_old, s.res[my_b][2 * my_pair], s.res[my_b][2 * my_pair + 1]);
    st_tagged(ws_of(p, my_b) + kWsHiddenOut + (rs + 2 * my_pair) / 2, w, tag);
    st_shared32(p.hidden + static_cast<size_t>(my_b) * M::H + rs + 2 * my_pair, w);
  }
  return true;
}

// ===================================================================== 7 ==
// [7, start_block, end_block, tile_M_g, tile_N_g]     logits[b] = bf16(W_lm . rms(hidden[b])) for every row
template <class M>
__device__ bool op_lmhead(const Params& p, Smem<M>& s, const Ctx& c) {
  constexpr int NR = RowsOf<M>::value;
  constexpr int CH = M::H / 512;
  const int bstart = s.b.inst[1], bend = s.b.inst[2], tile = s.b.inst[4];
  const int B = p.batch;
  if (tile <= 0) return bad_operand(p, s, c, 4);
  if (bstart < 0 || bend < bstart || static_cast<long>(bend) * tile > p.vocab_size) return bad_operand(p, s, c, 2);
  if (p.num_layers < 1) return bad_operand(p, s, c, 0);
  const int lane = c.tid & 63;
  const int rs = bstart * tile, nrows = (bend - bstart) * tile;
  const u16* W = p.lm_w + static_cast<size_t>(rs) * M::H;
  auto src = [&](int r) { return W + static_cast<size_t>(r) * M::H; };
  RowRegs<CH> buf[kDepth];
  preload<CH>(nrows, src, buf);
  if (!rms_rows<M, 0>(p, s, c, kWsHiddenOut, tag_of(s.b.generation, p.num_layers - 1), p.lm_norm, [](auto) {})) return false;
  v4u x[NR][CH];
  load_x_rows<M, CH>(s, x, lane);
  // Terminal op: nothing inside the launch reads the logits, so ordinary stores do.
  stream<CH>(nrows, src, buf, [&](int r, const RowRegs<CH>& w) {
    float sum[NR];
    static_for<0, NR>([&](auto b) { sum[b] = wave_sum(dot_row(w, x[b])); });
    static_for<0, NR>([&](auto b) {
      if (lane == b && b < B) p.logits[static_cast<size_t>(b) * p.vocab_size + rs + r] = f2bf(s.live[b] ? sum[b] : -1e9f);   // (a row that is not decoded: as the batch route leaves it)
    });
  });
  return true;
}

}  // namespace rows
}  // namespace qmk
