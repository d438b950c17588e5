// The seven decode opcodes as workgroup-wide device functions.
//
// Semantics follow the reference's fused PyTorch route, including where it
// rounds to bf16 (qimeng_megakernel/models/LLM/llama/llama3_2__1b/A100/
// single_batch/decode_schedule/fused/operations.py:126-321); operand layout
// and the counter protocol follow its instruction VM
// (…/decode_schedule/instructions/python_vm.py:109-488).  The file is compiled
// with -ffp-contract=off: where the fused route rounds between a multiply and
// an add, so does this code; fused multiply-adds are written explicitly.
#pragma once

#include "qmk_device.h"

namespace qmk {

// Ops of a dense kernel that read the launch parameters from the kernel-argument segment (per instruction) instead of
// the kernel's by-value parameter: bits of M::PARAMS_FROM_SEGMENT.
enum : int { kSegmentQkv = 1, kSegmentAttention = 2, kSegmentOproj = 4, kSegmentUpGate = 8, kSegmentDown = 16, kSegmentLmHead = 32 };

struct Llama1B {
  static constexpr int H = 2048;    // hidden size
  static constexpr int F = 8192;    // MLP intermediate size
  static constexpr int D = 64;      // head dim
  static constexpr int NQ = 32;     // query heads
  static constexpr int NKV = 8;     // key/value heads
  static constexpr int GQA = NQ / NKV;
  static constexpr int QKV = (NQ + 2 * NKV) * D;
  static constexpr int AW = NQ * D;    // width of the attention output = columns of the O-projection
  static constexpr int KV_BLOCK = 16;  // split-KV partition granularity in tokens
  static constexpr int CARRY_ROWS = 2;  // up/gate rows per wave requested by the O-proj before it
  static constexpr int PARK_ROWS = 2;   // ... and further ones that it leaves in LDS (measured: 1 860 tok/s; 3 rows 1 836, none 1 791)
  static constexpr bool CARRY_AFTER_ATTENTION = false;  // ... also by a workgroup that has just run attention
  static constexpr bool QK_NORM = false;
  static constexpr bool QKV_BIAS = false;
  static constexpr int REDUCE_HEADS = GQA;  // query heads one reduction instruction merges
  static constexpr int PREV_ROW = 5;        // counter row that completes a layer: the down projection's
  static constexpr int PARAMS_FROM_SEGMENT = kSegmentOproj;  // measured op by op: +0.7 %; with the up/gate op -2 %
};

// Qwen3-1.7B shape with the Qwen3 op set: opcode 1 leaves the raw QKV vector, the attention
// prologue applies the per-head RMSNorm of q and k and RoPE
// (qimeng_megakernel/models/LLM/qwen/qwen3__0_6b/A100/single_batch/decode_schedule/fused/operations.py:52-120).
struct Qwen3_1p7B {
  static constexpr int H = 2048;
  static constexpr int F = 6144;
  static constexpr int D = 128;
  static constexpr int NQ = 16;
  static constexpr int NKV = 8;
  static constexpr int GQA = NQ / NKV;
  static constexpr int QKV = (NQ + 2 * NKV) * D;
  static constexpr int AW = NQ * D;
  static constexpr int KV_BLOCK = 16;
  static constexpr int CARRY_ROWS = 3;
  static constexpr int PARK_ROWS = 2;   // (1 152 tok/s; 1 row 1 132, none 1 097)
  static constexpr bool CARRY_AFTER_ATTENTION = true;
  static constexpr bool QK_NORM = true;
  static constexpr bool QKV_BIAS = false;
  static constexpr int REDUCE_HEADS = GQA;
  static constexpr int PREV_ROW = 5;
  static constexpr int PARAMS_FROM_SEGMENT = kSegmentQkv | kSegmentAttention | kSegmentOproj | kSegmentLmHead;  // +2.7 %; all six: +1.8 %
};

constexpr int kResSlots = 4096;
// A geometry whose kernel parks no GEMV results in Smem::res says how few slots it needs (M::RES_SLOTS).
template <class M, class = void>
struct ResSlotsOf {
  static constexpr int value = kResSlots;
};
template <class M>
struct ResSlotsOf<M, std::void_t<decltype(M::RES_SLOTS)>> {
  static constexpr int value = M::RES_SLOTS;
};

// Up/gate rows that the O-proj before them leaves in LDS: [row][wave][chunk][lane], 4 KiB per row and wave.
template <int N>
struct ParkedRows {
  v4u v[N][kWaves][4][kWaveSize];
};
template <>
struct ParkedRows<0> {};

template <class M>
struct Smem {
  int32_t inst[kInstWords];
  int32_t next[kInstWords];             // the instruction after this one (zeros behind the last)
  int32_t ctl[8];                       // [0] abort, [1] last workgroup to retire
  uint32_t generation;                  // launch count of the tagged-activation workspace
  float best_val;                       // greedy candidate of this workgroup: largest bf16 logit so far ...
  int32_t best_idx;                     // ... and the first row that has it
  int32_t wave_idx[kWaves];             // per-wave candidates on their way to best_val/best_idx
  float red[kWaves];
  alignas(16) u16 x[M::F];              // activation vector handed to the GEMV lanes
  alignas(16) float res[ResSlotsOf<M>::value];   // per-row GEMV results awaiting the epilogue pass
  float merge[kWaves][M::GQA][M::D + 4];  // attention state per wave and head: acc[D], m, l
  unsigned long long t_wait;            // timeline: when the last counter wait finished
  unsigned long long stamps[4];         // timeline: op-specific intermediate timestamps
  // MoE route, tagged launches: the routing decision this workgroup last took from a layer's logits (-1: none yet)
  int32_t route_layer;
  int32_t route_expert[8];
  float route_weight[8];
  alignas(16) ParkedRows<M::PARK_ROWS> park;
};

enum Opcode {
  OP_NOOP = 0,
  OP_RMS_QKV_ROPE = 1,
  OP_ATTN_SPLITKV = 2,
  OP_ATTN_REDUCE = 3,
  OP_OPROJ_RESIDUAL = 4,
  OP_RMS_UPGATE_SILU = 5,
  OP_DOWN_RESIDUAL = 6,
  OP_RMS_LMHEAD = 7,
};

// Counter rows: opcode - 1.
constexpr int ROW_QKV = 0, ROW_SPLITKV = 1, ROW_REDUCE = 2, ROW_OPROJ = 3, ROW_UPGATE = 4, ROW_DOWN = 5;

struct Ctx {
  int inst_idx;
  int opcode;
  int tid;  // c.tid through an opaque copy made per instruction: what an op derives from it
            // stays inside that op instead of being computed once for all ops and kept in registers
};

// Optional intermediate timestamp k (0..3) of the running instruction, thread 0 only.
#define QMK_STAMP(k)                                                        \
  do {                                                                      \
    if (p.timeline != nullptr && c.tid == 0) s.stamps[k] = wall_clock64(); \
  } while (0)

template <class M>
__device__ __forceinline__ bool bad_operand(const Params& p, Smem<M>& s, const Ctx& c, int operand) {
  if (c.tid == 0) report_error(p, QMK_DEV_BAD_OPERAND, c.inst_idx, c.opcode, operand);
  return false;
}

// Lanes 0..n-1 each poll the counter `ctr_of(i)` up to `expected`; afterwards
// every thread has acquired.  False (uniformly) when a poll ran out of budget.
template <class M, class CtrOf>
__device__ __forceinline__ bool wg_wait(const Params& p, Smem<M>& s, const Ctx& c, int n, CtrOf ctr_of, int expected) {
  if (c.tid < n) {
    if (!poll_counter(ctr_of(c.tid), expected, p.spin_limit)) {
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
  acquire_loads();
  return true;
}

// Wait on an all-to-all edge (counter row 2..5): slot 0 of the row, or the eight
// per-XCD sub-counters of the edge when the launch uses them.
template <class M>
__device__ __forceinline__ bool wg_wait_all(const Params& p, Smem<M>& s, const Ctx& c, int layer, int row, int slot, int expected) {
  if (!xcd_counters(p)) {
    if (row == ROW_REDUCE && (p.flags & kFlagAttentionRows2To5))   // this XCD's line holds the whole count
      return wg_wait(p, s, c, 1, [&](int) { return counter_ptr(p, layer, ROW_REDUCE, static_cast<int>(blockIdx.x & (kXcds - 1)) * kLineInts); }, expected);
    return wg_wait(p, s, c, 1, [&](int) { return counter_ptr(p, layer, row, slot); }, expected);
  }
  if (row == ROW_REDUCE) {
    // The attention edge: every split-KV instruction arrives on all eight lines, this XCD's line holds the whole count.
    if (c.tid == 0 && !poll_counter(sub_counter(p, layer, row, blockIdx.x & (kXcds - 1)), expected, p.spin_limit)) {
      s.ctl[0] = 1;
      report_error(p, QMK_DEV_WAIT_TIMEOUT, c.inst_idx, c.opcode, row);
    }
  } else if (c.tid < kXcds) {
    if (!wait_edge_xcd(p, layer, row, expected, p.spin_limit) && c.tid == 0) {
      s.ctl[0] = 1;
      report_error(p, QMK_DEV_WAIT_TIMEOUT, c.inst_idx, c.opcode, row);
    }
  }
  if (p.timeline != nullptr && c.tid == 0) {
    s.t_wait = wall_clock64();
    s.ctl[2] = 1;
  }
  __syncthreads();
  return s.ctl[0] == 0;
}

// RMSNorm of the residual stream into s.x as bf16:
//   n = bf16(x * rsqrt(mean(x^2) + eps));  y = bf16(w * n)
// (fused/operations.py:126-131 — two roundings, the product taken on bf16 values).
// The residual stream comes from the caller's buffer (units == nullptr: a counter wait has made
// it complete) or from its tagged copy, each thread polling its own two units.  False
// (uniformly) when a tagged poll ran out of budget.
// `pace(k)`, k = 0..NP-1, issues the op's k-th group of weight-row requests.  With a tagged
// residual stream they go out one group per look at the units: loads return in issue order, so a
// look that stands behind all NP groups learns of the hand-over only when the last of them has
// landed, while behind one group it costs one round trip and the rows still arrive in the
// meantime.  Whatever has not been asked for when the units are complete goes out then.
template <class M, int NP, class Pace, class Wait>
__device__ __forceinline__ bool rms_to_lds(const Params& p, Smem<M>& s, const Ctx& c, const uint64_t* units, uint32_t tag,
                                           const u16* weight, Pace pace, Wait wait) {
  static_assert(M::H == kThreads * 4, "one thread normalises four elements");
  const int t = c.tid;
  uint32_t hlo = 0, hhi = 0;
  // Asked for first: the norm weights are then in registers when the residual stream arrives,
  // instead of costing a round trip of their own behind it.
  const uint2 wv = *reinterpret_cast<const uint2*>(weight + t * 4);
  const uint64_t* mine = units + 2 * t;
  bool done = units == nullptr;
  auto look = [&] {
    const uint64_t x = ld_shared64(mine), y = ld_shared64(mine + 1);
    hlo = static_cast<uint32_t>(x);
    hhi = static_cast<uint32_t>(y);
    const bool ok = static_cast<uint32_t>(x >> 32) == tag && static_cast<uint32_t>(y >> 32) == tag;
    done = __builtin_amdgcn_ballot_w64(ok) == ~0ull;  // the wave moves on together: row requests are wave-wide
  };
  static_for<0, NP>([&](auto kk) {
    pace(kk);
    if (!done) look();
  });
  if (units == nullptr) {
    if (!wait()) return false;  // counters: the caller's wait, behind all row requests
    const uint64_t hw = ld_shared64(p.hidden + t * 4);
    hlo = static_cast<uint32_t>(hw);
    hhi = static_cast<uint32_t>(hw >> 32);
  } else {
    for (uint32_t polls = 0; !done; ++polls) {
      if (polls > p.spin_limit) {
        s.ctl[0] = 1;
        report_error(p, QMK_DEV_WAIT_TIMEOUT, c.inst_idx, c.opcode, t);
        break;
      }
      if (polls) __builtin_amdgcn_s_sleep(1);
      look();
    }
    if (p.timeline != nullptr && t == 0) {
      s.t_wait = wall_clock64();
      s.ctl[2] = 1;
    }
  }
  const float x0 = bf_lo(hlo), x1 = bf_hi(hlo), x2 = bf_lo(hhi), x3 = bf_hi(hhi);
  float ss = __builtin_fmaf(x3, x3, __builtin_fmaf(x2, x2, __builtin_fmaf(x1, x1, x0 * x0)));
  ss = block_sum(ss, s.red);
  const float mean = ss / static_cast<float>(M::H);
  const float rstd = 1.0f / sqrtf(mean + p.rms_norm_eps);
  const uint32_t n01 = f2bf2(x0 * rstd, x1 * rstd), n23 = f2bf2(x2 * rstd, x3 * rstd);   // bf16(x * rstd) ...
  uint2 out;
  out.x = f2bf2(bf_lo(wv.x) * bf_lo(n01), bf_hi(wv.x) * bf_hi(n01));                     // ... times the weight, rounded again
  out.y = f2bf2(bf_lo(wv.y) * bf_lo(n23), bf_hi(wv.y) * bf_hi(n23));
  *reinterpret_cast<uint2*>(s.x + t * 4) = out;
  __syncthreads();
  return s.ctl[0] == 0;
}
template <class M>
__device__ __forceinline__ bool rms_to_lds(const Params& p, Smem<M>& s, const Ctx& c, const uint64_t* units, uint32_t tag,
                                           const u16* weight) {
  return rms_to_lds<M, 0>(p, s, c, units, tag, weight, [](auto) {}, [] { return true; });
}

// Interleaved-pair RoPE on bf16-rounded inputs, evaluated in fp32 with a
// rounding after every multiply and the add, then rounded to bf16
// (fused/operations.py:134-148, 173-181).
__device__ __forceinline__ uint32_t rope_pair(float v0, float v1, float2 cs, float2 sn) {
  const float o0 = v0 * cs.x + (-v1) * sn.x;
  const float o1 = v1 * cs.y + v0 * sn.y;
  return f2bf2(o0, o1);
}
__device__ __forceinline__ uint32_t rope_pair(float v0, float v1, const float* cosr, const float* sinr, int d) {
  return rope_pair(v0, v1, *reinterpret_cast<const float2*>(cosr + d), *reinterpret_cast<const float2*>(sinr + d));
}

// ------------------------------------------------------------ streaming ----
constexpr int kDepth = 4;  // row buffers per wave: 4 x CH x 16 B per lane in flight

// Wave w consumes elements w, w+8, w+16, ... of a sequence of weight-row segments
// (`src(e)` = address of CH*512 bf16) through NB register buffers.  `buf[k]` must already hold
// element w + 8k (issued by `preload` / `preload_range`); each buffer is refilled with the
// element 8*NB further on as soon as it has been consumed.  `use(e, buf)` gets the raw
// registers of element e.
//
// How much to ask for before the wait is a trade: what is in flight then lands while the
// workgroup waits, but it also stands in the memory queues in front of the last producers'
// stores, and in front of this wave's own looks at the hand-over (loads return in issue order).
// The ops that normalise the residual stream ask for one buffer per look; the down projection
// asks for kEarly buffers up front and for the rest once silu_out is complete.
template <int K0, int K1, int CH, int NB, class Src>
__device__ __forceinline__ void preload_range(int n, Src src, RowRegs<CH> (&buf)[NB]) {
  static_assert(K0 >= 0 && K1 <= NB, "buffer range");
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
  for (int k = K0; k < K1; ++k)
    if (wave + k * kWaves < n) load_row(buf[k], src(wave + k * kWaves), lane);
}

template <int CH, int NB, class Src>
__device__ __forceinline__ void preload(int n, Src src, RowRegs<CH> (&buf)[NB]) {
  preload_range<0, NB>(n, src, buf);
}

template <int CH, int NB, class Src, class Use>
__device__ __forceinline__ void stream(int n, Src src, RowRegs<CH> (&buf)[NB], Use use) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (int e = wave; e < n; e += NB * kWaves) {
#pragma unroll
    for (int k = 0; k < NB; ++k) {
      const int ek = e + k * kWaves;
      if (ek < n) {
        use(ek, buf[k]);
        const int nx = ek + NB * kWaves;
        if (nx < n) load_row(buf[k], src(nx), lane);
      }
    }
  }
}

constexpr int kEarly = 2;           // buffers of the down projection requested before its wait
constexpr int kUpGateBuffers = 4;   // row buffers of the up/gate GEMV

// Rows that one instruction requests for the next one of its queue: the O-proj has three of its
// four row buffers to spare and waits for the whole attention phase, in which the memory system
// has little to do; it asks for the up/gate rows that would otherwise be requested behind that wait.
// (Only there: anywhere else such requests would stand in front of the stores that hand the
// instruction's own results over.)
constexpr int kOprojBuffers = 2;  // row buffers of the O-proj (8 rows per workgroup: one per wave)
constexpr int kCarried = kUpGateBuffers - 1;  // at most; a model asks for M::CARRY_ROWS of them (measured)
struct Carried {
  RowRegs<4> row[kCarried];  // element wave + 8 * (k + 1) of the up/gate instruction
};
// The registers hold nothing of interest from here on (no instruction is generated: this only
// ends their live range, so that they are not kept across the ops that do not use them).
__device__ __forceinline__ void forget(Carried& c) {
#pragma unroll
  for (int k = 0; k < kCarried; ++k)
#pragma unroll
    for (int j = 0; j < 4; ++j) asm volatile("" : "=v"(c.row[k].v[j]));
}

// Row of element e of an up/gate instruction (words w): element 2i is the up row of the
// instruction's i-th output, 2i + 1 its gate row.
template <class M>
__device__ __forceinline__ const u16* upgate_row(const Params& p, const int32_t* w, int layer, int tile, int e) {
  const int i = e >> 1;
  const int sh = __builtin_ctz(static_cast<unsigned>(tile));   // tiles are powers of two (upgate_check): no integer division per row request
  const int row = w[4 + (i >> sh)] * tile + (i & (tile - 1));
  const u16* base = (e & 1) ? p.gate_w : p.up_w;
  return base + (static_cast<size_t>(layer) * M::F + row) * M::H;
}
// Operand checks of an up/gate instruction; the index of the offending word, or -1.
template <class M>
__device__ __forceinline__ int upgate_check(const Params& p, const int32_t* w) {
  const int layer = w[1], n = w[3];
  if (layer < 0 || layer >= p.num_layers) return 1;
  if (n < 0 || n > kInstWords - 6) return 3;
  const int tile = w[5 + n];
  if (tile < 2 || (tile & (tile - 1)) || M::F % tile != 0) return 5 + n;   // an even power of two
  if (n * tile * 2 > kResSlots) return 3;
  for (int i = 0; i < n; ++i)
    if (w[4 + i] < 0 || static_cast<long>(w[4 + i] + 1) * tile > M::F) return 4 + i;
  return -1;
}

// ===================================================================== 1 ==
// [1, layer, tile_M, n_start, n_end, tile_M_g, tile_N_g]
template <class M>
__device__ bool op_rms_qkv_rope(const Params& p, Smem<M>& s, const Ctx& c) {
  constexpr int CH = M::H / 512;
  const int layer = s.inst[1], nstart = s.inst[3], nend = s.inst[4], tile = s.inst[6];
  const int bph = p.qkv_blocks_per_head;
  if (layer < 0 || layer >= p.num_layers) return bad_operand(p, s, c, 1);
  if (tile <= 0 || (tile & 1) || tile * bph != M::D) return bad_operand(p, s, c, 6);
  if (nstart < 0 || nend < nstart || static_cast<long>(nend) * tile > M::QKV) return bad_operand(p, s, c, 4);
  if ((nend - nstart) * tile > kResSlots) return bad_operand(p, s, c, 3);

  const int lane = c.tid & 63;
  const int rs = nstart * tile, nrows = (nend - nstart) * tile;
  const u16* W = p.qkv_w + (static_cast<size_t>(layer) * M::QKV + rs) * M::H;
  auto src = [&](int r) { return W + static_cast<size_t>(r) * M::H; };

  // The RoPE factors of this thread's first output pair are asked for before anything else.
  const float* cosr = p.rope_cos + static_cast<size_t>(p.pos_id) * M::D;
  const float* sinr = p.rope_sin + static_cast<size_t>(p.pos_id) * M::D;
  float2 cs0 = {0.0f, 0.0f}, sn0 = {0.0f, 0.0f};
  if constexpr (!M::QK_NORM) {
    const int r0 = rs + 2 * c.tid;
    if (c.tid < nrows / 2 && r0 < (M::NQ + M::NKV) * M::D) {
      cs0 = *reinterpret_cast<const float2*>(cosr + r0 % M::D);
      sn0 = *reinterpret_cast<const float2*>(sinr + r0 % M::D);
    }
  }
  RowRegs<CH> buf[kDepth];
  const bool tg = tagged(p);
  const uint32_t tag = tag_of(s.generation, layer);
  if (!rms_to_lds<M, kDepth>(
          p, s, c, (tg && layer > 0) ? p.ws + kWsHiddenOut : nullptr, tag - 1, p.attn_norm + static_cast<size_t>(layer) * M::H,
          [&](auto k) { preload_range<decltype(k)::value, decltype(k)::value + 1>(nrows, src, buf); },
          [&] { return layer == 0 || tg || wg_wait_all(p, s, c, layer - 1, M::PREV_ROW, 0, p.down_arrivals); }))
    return false;
  QMK_STAMP(0);
  v4u x[CH];
  load_x_from_lds(x, s.x, lane);
  stream<CH>(nrows, src, buf, [&](int r, const RowRegs<CH>& w) {
    const float sum = wave_sum(dot_row(w, x));
    if (lane == 0) s.res[r] = sum;
  });
  QMK_STAMP(1);
  __syncthreads();
  QMK_STAMP(2);

  // Epilogue: the GEMV result is bf16 before RoPE; q -> q_post_rope, k/v -> cache row of this position.
  const size_t kv_row = (static_cast<size_t>(layer) * p.max_seq_len + p.pos_id) * (M::NKV * M::D);
  for (int pair = c.tid; pair < nrows / 2; pair += kThreads) {
    const int r = rs + 2 * pair;
    const bool first = pair == c.tid;
    float a0 = s.res[2 * pair], a1 = s.res[2 * pair + 1];
    if constexpr (M::QKV_BIAS) {   // the bias belongs to the projection: added before its one rounding
      const uint32_t bw = *reinterpret_cast<const uint32_t*>(p.qkv_bias + static_cast<size_t>(layer) * M::QKV + r);
      a0 += bf_lo(bw), a1 += bf_hi(bw);
    }
    const float v0 = round_bf16(a0), v1 = round_bf16(a1);
    if constexpr (M::QK_NORM) {
      // Qwen3 op set: the rounded GEMV result leaves as it is; norm and RoPE belong to the attention prologue.
      const uint32_t w = f2bf2(v0, v1);
      st_shared32(p.qkv_raw + r, w);
      if (tg) {
        const int kq = M::NQ * M::D, kk = (M::NQ + M::NKV) * M::D;
        st_tagged(p.ws + (r < kq ? kWsQ + r / 2 : (r < kk ? kWsK + (r - kq) / 2 : kWsV + (r - kk) / 2)), w, tag);
      }
    } else if (r < M::NQ * M::D) {
      const uint32_t w = first ? rope_pair(v0, v1, cs0, sn0) : rope_pair(v0, v1, cosr, sinr, r % M::D);
      st_shared32(p.q_post_rope + r, w);
      if (tg) st_tagged(p.ws + kWsQ + r / 2, w, tag);
    } else if (r < (M::NQ + M::NKV) * M::D) {
      const int i = r - M::NQ * M::D;
      const uint32_t w = first ? rope_pair(v0, v1, cs0, sn0) : rope_pair(v0, v1, cosr, sinr, i % M::D);
      st_shared32(p.k_cache + kv_row + i, w);
      if (tg) st_tagged(p.ws + kWsK + i / 2, w, tag);
    } else {
      const int i = r - (M::NQ + M::NKV) * M::D;
      const uint32_t w = f2bf2(v0, v1);
      st_shared32(p.v_cache + kv_row + i, w);
      if (tg) st_tagged(p.ws + kWsV + i / 2, w, tag);
    }
  }
  QMK_STAMP(3);
  if (tg) return true;  // the units announce themselves: nothing to wait for, nothing to count

  release_stores();
  __syncthreads();
  // One arrival per tile, on the counter of the head the tile belongs to.
  if (nend > nstart) {
    const int slot0 = nstart / bph, slot1 = (nend - 1) / bph;
    const int slot = slot0 + c.tid;
    if (slot <= slot1) {
      const int lo = max(nstart, slot * bph), hi = min(nend, (slot + 1) * bph);
      publish(counter_ptr(p, layer, ROW_QKV, slot), hi - lo);
    }
  }
  return true;
}

// Log-sum-exp merge of `n` split-KV partials (slot indices `list[i]`, or 0..n-1 when
// list is null) for the GQA heads head0..head0+3 (python_vm.py:439-488).  Thread
// (h, d/2) of the first 128 produces two neighbouring output dims.  All partial
// reads are issued before the first use so that they overlap.
template <class M, int HEADS = M::GQA>
__device__ __forceinline__ void merge_partials(const Params& p, int head0, int n, const int32_t* list, bool terminal,
                                               int out_slot) {
  static_assert(HEADS * M::D / 2 <= kThreads, "one thread per output pair");
  if (threadIdx.x >= HEADS * M::D / 2) return;
  const int h = head0 + threadIdx.x / (M::D / 2), d = 2 * (threadIdx.x % (M::D / 2));
  const float* lse = p.attn_lse + static_cast<size_t>(h) * p.max_splits;
  const float* part = p.attn_partial + static_cast<size_t>(h) * p.max_splits * M::D + d;
  // Branch-free: slots beyond n re-read the last listed partial and get weight 0.
  float e[kMaxPartials];
  uint64_t two[kMaxPartials];
#pragma unroll
  for (int i = 0; i < kMaxPartials; ++i) {
    const int ii = min(i, n - 1);
    const int j = list ? list[ii] : ii;
    e[i] = ld_shared_f32(lse + j);
    two[i] = ld_shared64(part + static_cast<size_t>(j) * M::D);
  }
  float mx = -INFINITY;
#pragma unroll
  for (int i = 0; i < kMaxPartials; ++i) mx = fmaxf(mx, e[i]);
  float num0 = 0.f, num1 = 0.f, den = 0.f;
#pragma unroll
  for (int i = 0; i < kMaxPartials; ++i) {
    const float f = (i < n && e[i] != -INFINITY) ? exp2_fast(e[i] - mx) : 0.f;
    num0 = __builtin_fmaf(__uint_as_float(static_cast<uint32_t>(two[i])), f, num0);
    num1 = __builtin_fmaf(__uint_as_float(static_cast<uint32_t>(two[i] >> 32)), f, num1);
    den += f;
  }
  const float o0 = den > 0.f ? num0 / den : 0.f, o1 = den > 0.f ? num1 / den : 0.f;
  if (terminal) {
    st_shared32(p.attn_out + h * M::D + d, f2bf2(o0, o1));
  } else {
    float* dst = p.attn_partial + (static_cast<size_t>(h) * p.max_splits + out_slot) * M::D + d;
    st_shared_f32(dst, o0);
    st_shared_f32(dst + 1, o1);
    if (d == 0) st_shared_f32(p.attn_lse + static_cast<size_t>(h) * p.max_splits + out_slot, den > 0.f ? mx + log2f(den) : -INFINITY);
  }
}

// One role of the Qwen3 op set's attention prologue, run by one wave on the staged vectors (`words`: q heads
// from 0, then the new K row, then the new V row; lane l owns the rotation pair (2l, 2l+1)).  Roles 0..GQA-1:
// a query head; GQA: the K row — per-head RMSNorm, n = bf16(w * (x * rsqrt(mean(x^2) + eps))) in fp32 with one
// rounding, then RoPE, in place; GQA+1: the V row, which goes to the cache as it is.  The one partial of the KV
// head whose slice holds this position (`has_new`) also writes the caller's copies.
template <class M>
__device__ __forceinline__ void qk_norm_rope_role(const Params& p, uint32_t* words, int role, int lane, int layer, int kvh,
                                                  bool has_new, size_t new_row) {
  constexpr int D = M::D, GQA = M::GQA, kQ = 0, kK = GQA * D, kV = GQA * D + D;
  if (role <= GQA && (role < GQA || has_new)) {
    const bool is_k = role == GQA;
    const int at = is_k ? kK / 2 : (kQ + role * D) / 2;
    const uint32_t raw = words[at + lane];
    const float x0 = bf_lo(raw), x1 = bf_hi(raw);
    const float ss = wave_sum(__builtin_fmaf(x1, x1, x0 * x0));
    const float rstd = 1.0f / sqrtf(ss / static_cast<float>(D) + p.rms_norm_eps);
    const uint32_t wn = reinterpret_cast<const uint32_t*>((is_k ? p.k_norm : p.q_norm) + static_cast<size_t>(layer) * D)[lane];
    const float n0 = round_bf16(bf_lo(wn) * (x0 * rstd)), n1 = round_bf16(bf_hi(wn) * (x1 * rstd));
    const float* cosr = p.rope_cos + static_cast<size_t>(p.pos_id) * D;
    const float* sinr = p.rope_sin + static_cast<size_t>(p.pos_id) * D;
    const uint32_t out = rope_pair(n0, n1, cosr, sinr, 2 * lane);
    words[at + lane] = out;
    if (has_new) {
      if (is_k) st_shared32(p.k_cache + new_row + 2 * lane, out);
      else st_shared32(p.q_post_rope + (kvh * GQA + role) * D + 2 * lane, out);
    }
  } else if (role == GQA + 1 && has_new) {
    st_shared32(p.v_cache + new_row + 2 * lane, words[kV / 2 + lane]);
  }
}

// ===================================================================== 2 ==
// [2, layer, kv_head, num_partials, partial_idx, merge_in_last]
// Flash-decoding over one contiguous slice of the context for the GQA group of
// one KV head.  A wave takes 16 tokens at a time (tiles w, w+8, ... of the slice) and keeps one
// running (max, sum, acc) per query head; the eight wave states are merged once at the end.
// Scores live in the log2 domain.
//
// The query heads and the K/V row appended in this launch are first staged in LDS (bf16:
// [0, GQA*D) q, then k, then v) — from their tagged units, or after the per-head counters from
// the caller's buffers.  With the Qwen3 op set (M::QK_NORM) what is staged is the raw QKV
// vector; one wave per vector then applies the per-head RMSNorm and RoPE in place
// (qwen3__0_6b/…/fused/operations.py:52-120), and the workgroup whose slice holds this position
// also writes q_post_rope and the cache row.
//
// merge_in_last (an extension; 0 in streams built by the reference scheduler): the
// workgroup whose arrival completes the head group's counter merges all partials
// itself and publishes on the reduction row, so no separate reduction instruction
// (and no second wait) is needed.
template <class M>
__device__ bool op_attn_splitkv(const Params& p, Smem<M>& s, const Ctx& c) {
  constexpr int D = M::D, GQA = M::GQA;
  static_assert(D % 64 == 0 && GQA <= 8 && GQA * D <= 2 * kThreads, "a lane owns whole 16-byte vectors of K; heads 4g..4g+3 live in lane group g");
  static_assert(!M::QK_NORM || D == 2 * kWaveSize, "the per-head norm gives every lane one rotation pair");
  const int layer = s.inst[1], kvh = s.inst[2], P = s.inst[3], part = s.inst[4];
  const int merge_mode = s.inst[5];  // 0: per-head counters, 1: last arrival merges, 2: the O-proj merges
  const bool merge_in_last = merge_mode == 1;
  if (merge_mode < 0 || merge_mode > 2) return bad_operand(p, s, c, 5);
  if (layer < 0 || layer >= p.num_layers) return bad_operand(p, s, c, 1);
  if (kvh < 0 || kvh >= M::NKV) return bad_operand(p, s, c, 2);
  if (P < 1 || P > p.max_splits || part < 0 || part >= P) return bad_operand(p, s, c, 3);
  if (merge_in_last && P > kMaxPartials) return bad_operand(p, s, c, 3);

  const int lane = c.tid & 63, wave = c.tid >> 6;

  // Context slice of this partial (python_vm.py:391-401).
  const int seq_len = p.pos_id + 1;
  const int total_blocks = (seq_len + M::KV_BLOCK - 1) / M::KV_BLOCK;
  const int bpp = (total_blocks + P - 1) / P;
  const int t0 = min(part * bpp, total_blocks) * M::KV_BLOCK;
  const int t1 = min(min((part + 1) * bpp, total_blocks) * M::KV_BLOCK, seq_len);
  const bool has_new = p.pos_id >= t0 && p.pos_id < t1;

  // A wave scores 16 tokens at a time on the matrix cores: S^T[token][head] = K[token][:] . q[head][:]
  // (v_mfma_f32_16x16x16_bf16, K rows as the A operand, the GQA heads as GQA of the 16 B columns), then
  // O[head][:] += P[head][token] . V[token][:] with P split into two bf16 terms so that it keeps 16
  // mantissa bits.  Operand layout of the instruction: lane l holds A[l%16][4*(l/16)..+3],
  // B[4*(l/16)..+3][l%16] and C[4*(l/16)..+3][l%16].  Which of the D dims sits in which k slot is free
  // as long as q and K agree, and so is the order of the output columns: lane (c16, g4) reads K dims
  // g4*D/4 .. +D/4 of token c16 and V dims c16*D/16 .. +D/16 of tokens 4*g4 .. +3, in 16- or 8-byte pieces.
  // Rows of earlier positions do not depend on this step: the wave's first tile is fetched now.
  constexpr int KV16 = D / 32;          // 16-byte vectors of a K row per lane
  constexpr int NT = D / 16;            // k chunks of the score product = output column tiles of P.V
  constexpr int kTile = 16, kStep = kWaves * kTile;
  const int c16 = lane & 15, g4 = lane >> 4;
  const size_t tok_stride = static_cast<size_t>(M::NKV) * D;
  const size_t row_of_kvh = static_cast<size_t>(layer) * p.max_seq_len * tok_stride + static_cast<size_t>(kvh) * D;
  const u16* kbase = p.k_cache + row_of_kvh + g4 * (D / 4);
  const u16* vbase = p.v_cache + row_of_kvh + c16 * NT;
  struct Tile {
    v4u k[KV16];         // K[token c16][g4*D/4 ..]
    uint32_t v[4][NT / 2];  // V[token 4*g4 + j][c16*NT ..], two dims per word
  };
  // Tokens past the slice are fetched from its last row (finite data) and masked when scored.
  auto fetch = [&](Tile& tl, int tb) {
    const int tk = min(tb + c16, t1 - 1);
#pragma unroll
    for (int j = 0; j < KV16; ++j) tl.k[j] = reinterpret_cast<const v4u*>(kbase + static_cast<size_t>(tk) * tok_stride)[j];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int tv = min(tb + 4 * g4 + j, t1 - 1);
      const uint32_t* src = reinterpret_cast<const uint32_t*>(vbase + static_cast<size_t>(tv) * tok_stride);
#pragma unroll
      for (int i = 0; i < NT / 2; ++i) tl.v[j][i] = src[i];
    }
  };
  int tb = t0 + wave * kTile;
  Tile cur;
#pragma unroll
  for (int j = 0; j < KV16; ++j) cur.k[j] = v4u{0, 0, 0, 0};
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int i = 0; i < NT / 2; ++i) cur.v[j][i] = 0;
  if (tb < t1) fetch(cur, tb);

  // ---- stage q (and the appended K/V row) in LDS --------------------------------------------
  const bool tg = tagged(p);
  u16* stage16 = s.x;
  constexpr int kQ = 0, kK = GQA * D, kV = GQA * D + D;
  const size_t new_row = row_of_kvh + static_cast<size_t>(p.pos_id) * tok_stride;
  if (tg) {
    // q: GQA*D/2 units, two per thread of the first GQA*D/4 threads; K and V: D/2 units each, two per thread.
    constexpr int kQThreads = GQA * D / 4;
    static_assert(kQThreads + D / 2 <= kThreads, "one poller per unit pair");
    const uint32_t tag = tag_of(s.generation, layer);
    uint32_t* words = reinterpret_cast<uint32_t*>(stage16);
    bool arrived = true;
    uint32_t a = 0, b = 0;
    const int tid = c.tid;
    if (tid < kQThreads) {
      arrived = poll_tagged2(p.ws + kWsQ + kvh * (GQA * D / 2) + 2 * tid, tag, p.spin_limit, a, b);
      words[kQ / 2 + 2 * tid] = a;
      words[kQ / 2 + 2 * tid + 1] = b;
    } else if (tid < kQThreads + D / 2 && has_new) {
      const int j = tid - kQThreads;                       // [0, D/4): K, [D/4, D/2): V
      const bool is_v = j >= D / 4;
      const int u = 2 * (is_v ? j - D / 4 : j);
      arrived = poll_tagged2(p.ws + (is_v ? kWsV : kWsK) + kvh * (D / 2) + u, tag, p.spin_limit, a, b);
      words[(is_v ? kV : kK) / 2 + u] = a;
      words[(is_v ? kV : kK) / 2 + u + 1] = b;
    }
    if (!arrived) {
      s.ctl[0] = 1;
      report_error(p, QMK_DEV_WAIT_TIMEOUT, c.inst_idx, c.opcode, c.tid);
    }
    if (p.timeline != nullptr && c.tid == 0) {
      s.t_wait = wall_clock64();
      s.ctl[2] = 1;
    }
  } else {
    if (!wg_wait(p, s, c, GQA + 2,
                 [&](int i) {
                   const int slot = i < GQA ? kvh * GQA + i : (i == GQA ? M::NQ + kvh : M::NQ + M::NKV + kvh);
                   return counter_ptr(p, layer, ROW_QKV, slot);
                 },
                 p.qkv_blocks_per_head))
      return false;
    // 16-byte chunks: GQA*D/8 of q, then D/8 of K and of V (the row of this position only)
    const int tid = c.tid;
    constexpr int kQChunks = GQA * D / 8, kRowChunks = D / 8;
    const u16* q_src = M::QK_NORM ? p.qkv_raw + kvh * GQA * D : p.q_post_rope + kvh * GQA * D;
    const u16* k_src = M::QK_NORM ? p.qkv_raw + M::NQ * D + kvh * D : p.k_cache + new_row;
    const u16* v_src = M::QK_NORM ? p.qkv_raw + (M::NQ + M::NKV) * D + kvh * D : p.v_cache + new_row;
    if (tid < kQChunks) {
      reinterpret_cast<v4u*>(stage16 + kQ)[tid] = ld_shared128(q_src + tid * 8);
    } else if (tid < kQChunks + kRowChunks && has_new) {
      reinterpret_cast<v4u*>(stage16 + kK)[tid - kQChunks] = ld_shared128(k_src + (tid - kQChunks) * 8);
    } else if (tid < kQChunks + 2 * kRowChunks && has_new) {
      reinterpret_cast<v4u*>(stage16 + kV)[tid - kQChunks - kRowChunks] = ld_shared128(v_src + (tid - kQChunks - kRowChunks) * 8);
    }
  }
  __syncthreads();
  if (s.ctl[0]) return false;

  if constexpr (M::QK_NORM) {
    // One wave per vector: roles 0..GQA-1 are the query heads, role GQA the new K row; the new V row
    // (role GQA+1) goes to the cache as it is.  Lane l owns the rotation pair (2l, 2l+1).
    //   n = bf16(w * (x * rsqrt(mean(x^2) + eps)))   — fp32 throughout, one rounding
    uint32_t* words = reinterpret_cast<uint32_t*>(stage16);
    // A pass gives every wave one role; two passes cover the ten roles of a group of eight heads.
    if constexpr (GQA + 2 <= kWaves) {
      // (the helper's body, in place: called as a function — even a forced-inline one — this compiler allocates
      // the registers of the whole op differently and the dense Qwen3 kernel loses 1.3 %)
      if (wave <= GQA && (wave < GQA || has_new)) {
        const bool is_k = wave == GQA;
        const int at = is_k ? kK / 2 : (kQ + wave * D) / 2;
        const uint32_t raw = words[at + lane];
        const float x0 = bf_lo(raw), x1 = bf_hi(raw);
        const float ss = wave_sum(__builtin_fmaf(x1, x1, x0 * x0));
        const float rstd = 1.0f / sqrtf(ss / static_cast<float>(D) + p.rms_norm_eps);
        const uint32_t wn = reinterpret_cast<const uint32_t*>((is_k ? p.k_norm : p.q_norm) + static_cast<size_t>(layer) * D)[lane];
        const float n0 = round_bf16(bf_lo(wn) * (x0 * rstd)), n1 = round_bf16(bf_hi(wn) * (x1 * rstd));
        const float* cosr = p.rope_cos + static_cast<size_t>(p.pos_id) * D;
        const float* sinr = p.rope_sin + static_cast<size_t>(p.pos_id) * D;
        const uint32_t out = rope_pair(n0, n1, cosr, sinr, 2 * lane);
        words[at + lane] = out;
        if (has_new) {  // exactly one partial of this KV head holds the position: it owns the caller's copies
          if (is_k) st_shared32(p.k_cache + new_row + 2 * lane, out);
          else st_shared32(p.q_post_rope + (kvh * GQA + wave) * D + 2 * lane, out);
        }
      } else if (wave == GQA + 1 && has_new) {
        st_shared32(p.v_cache + new_row + 2 * lane, words[kV / 2 + lane]);
      }
    } else {
      qk_norm_rope_role<M>(p, words, wave, lane, layer, kvh, has_new, new_row);
      qk_norm_rope_role<M>(p, words, wave + kWaves, lane, layer, kvh, has_new, new_row);
    }
    __syncthreads();
  }

  // q as the B operand: column c16 is head c16 (zero beyond the GQA heads), k slots as for K.
  typedef short bf4 __attribute__((ext_vector_type(4)));
  typedef float f4 __attribute__((ext_vector_type(4)));
  typedef uint32_t u2 __attribute__((ext_vector_type(2)));
  const float qscale = p.attn_scale * 1.4426950408889634f;  // scores in the log2 domain
  bf4 qb[NT];
#pragma unroll
  for (int j = 0; j < KV16; ++j) {
    v4u qv = v4u{0, 0, 0, 0};
    if (c16 < GQA) qv = reinterpret_cast<const v4u*>(stage16 + kQ + c16 * D + g4 * (D / 4))[j];
    qb[2 * j] = __builtin_bit_cast(bf4, u2{qv.x, qv.y});
    qb[2 * j + 1] = __builtin_bit_cast(bf4, u2{qv.z, qv.w});
  }
  QMK_STAMP(0);  // q (and the appended row) have arrived

  // State of this wave: m (all four lanes of a column agree), this lane's share of l, and
  // O[head 4*g4 + i][dim c16*NT + tile] in acc[tile][i] (lane groups beyond the GQA heads hold nothing).
  float m_run = -INFINITY, l_run = 0.f;
  f4 acc[NT];
#pragma unroll
  for (int i = 0; i < NT; ++i) acc[i] = f4{0.f, 0.f, 0.f, 0.f};

  while (tb < t1) {
    Tile nxt = cur;
    if (tb + kStep < t1) fetch(nxt, tb + kStep);
    if (p.pos_id >= tb && p.pos_id < tb + kTile) {  // the row appended during this launch comes from LDS
      if (tb + c16 == p.pos_id) {
#pragma unroll
        for (int j = 0; j < KV16; ++j) cur.k[j] = reinterpret_cast<const v4u*>(stage16 + kK + g4 * (D / 4))[j];
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        if (tb + 4 * g4 + j == p.pos_id) {
#pragma unroll
          for (int i = 0; i < NT / 2; ++i) cur.v[j][i] = reinterpret_cast<const uint32_t*>(stage16 + kV + c16 * NT)[i];
        }
      }
    }
    // S^T[token 4*g4 + i][head c16]
    f4 sc = f4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < KV16; ++j) {
      sc = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(bf4, u2{cur.k[j].x, cur.k[j].y}), qb[2 * j], sc, 0, 0, 0);
      sc = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(bf4, u2{cur.k[j].z, cur.k[j].w}), qb[2 * j + 1], sc, 0, 0, 0);
    }
    float mt = -INFINITY;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      sc[i] = (tb + 4 * g4 + i < t1) ? sc[i] * qscale : -INFINITY;
      mt = fmaxf(mt, sc[i]);
    }
    mt = fmaxf(mt, __shfl_xor(mt, 16));
    mt = fmaxf(mt, __shfl_xor(mt, 32));      // the tile's maximum for head c16 (a tile has a valid token: finite)
    const float mn = fmaxf(m_run, mt);
    const float alpha = exp2_fast(m_run - mn);  // 0 on the first tile (m = -inf)
    m_run = mn;
    float pr[4], psum = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      pr[i] = (c16 < GQA) ? exp2_fast(sc[i] - mn) : 0.f;
      psum += pr[i];
    }
    l_run = __builtin_fmaf(l_run, alpha, psum);
    // P = hi + lo, both bf16: A operand rows = heads, k slots = the lane's four tokens.
    const uint32_t h01 = f2bf2(pr[0], pr[1]), h23 = f2bf2(pr[2], pr[3]);
    const uint32_t l01 = f2bf2(pr[0] - bf_lo(h01), pr[1] - bf_hi(h01)), l23 = f2bf2(pr[2] - bf_lo(h23), pr[3] - bf_hi(h23));
    const bf4 p_hi = __builtin_bit_cast(bf4, u2{h01, h23});
    const bf4 p_lo = __builtin_bit_cast(bf4, u2{l01, l23});
    // The accumulators of head h are scaled by that head's alpha (it lives in lane h); this lane
    // holds the heads 4*g4 .. 4*g4 + 3.
    float a_head[4];
    bool rescale = false;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      a_head[i] = i < GQA ? __int_as_float(__builtin_amdgcn_readlane(__float_as_int(alpha), i)) : 1.f;
      if constexpr (GQA > 4) {
        const float upper = 4 + i < GQA ? __int_as_float(__builtin_amdgcn_readlane(__float_as_int(alpha), 4 + i)) : 1.f;
        a_head[i] = g4 == 1 ? upper : a_head[i];
      }
      rescale = rescale || a_head[i] != 1.f;
    }
    if (rescale) {
#pragma unroll
      for (int tau = 0; tau < NT; ++tau)
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[tau][i] *= a_head[i];
    }
#pragma unroll
    for (int tau = 0; tau < NT; ++tau) {
      // B[token 4*g4 + j][column c16] = V[token][c16*NT + tau]
      const int w = tau / 2;
      uint32_t b0, b1;
      if (tau & 1) {
        b0 = (cur.v[0][w] >> 16) | (cur.v[1][w] & 0xffff0000u);
        b1 = (cur.v[2][w] >> 16) | (cur.v[3][w] & 0xffff0000u);
      } else {
        b0 = (cur.v[0][w] & 0xffffu) | (cur.v[1][w] << 16);
        b1 = (cur.v[2][w] & 0xffffu) | (cur.v[3][w] << 16);
      }
      const bf4 vb = __builtin_bit_cast(bf4, u2{b0, b1});
      acc[tau] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(p_hi, vb, acc[tau], 0, 0, 0);
      acc[tau] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(p_lo, vb, acc[tau], 0, 0, 0);
    }
    cur = nxt;
    tb += kStep;
  }

  QMK_STAMP(1);  // tokens scored
  // Every wave parks its state in LDS; GQA*D threads then merge the eight states, one output each.
  l_run += __shfl_xor(l_run, 16);
  l_run += __shfl_xor(l_run, 32);
  if constexpr (GQA <= 4) {
    if (lane < 16) {
#pragma unroll
      for (int tau = 0; tau < NT; ++tau)
#pragma unroll
        for (int i = 0; i < GQA; ++i) s.merge[wave][i][c16 * NT + tau] = acc[tau][i];
      if (c16 < GQA) {
        s.merge[wave][c16][D] = m_run;
        s.merge[wave][c16][D + 1] = l_run;
      }
    }
  } else if (lane < 32) {   // two lane groups hold the rows of heads 0..3 and 4..7
#pragma unroll
    for (int tau = 0; tau < NT; ++tau)
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (4 * g4 + i < GQA) s.merge[wave][4 * g4 + i][c16 * NT + tau] = acc[tau][i];
    if (g4 == 0 && c16 < GQA) {
      s.merge[wave][c16][D] = m_run;
      s.merge[wave][c16][D + 1] = l_run;
    }
  }
  __syncthreads();
  auto merge_output = [&](int o) {   // output o = (head, dim) of the partial: the eight wave states folded
    if (o >= GQA * D) return;
    const int h = o / D, d = o % D;
    float mx = -INFINITY;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) mx = fmaxf(mx, s.merge[w][h][D]);
    float den = 0.f, num = 0.f;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) {
      const float mw = s.merge[w][h][D];
      const float wgt = (mw == -INFINITY) ? 0.f : exp2_fast(mw - mx);
      den = __builtin_fmaf(s.merge[w][h][D + 1], wgt, den);
      num = __builtin_fmaf(s.merge[w][h][d], wgt, num);
    }
    const int head = kvh * GQA + h;
    const bool empty = !(den > 0.f);
    // Normalised partial output and log2-sum-exp; an empty slice contributes (0, -inf).
    st_shared_f32(p.attn_partial + (static_cast<size_t>(head) * p.max_splits + part) * D + d, empty ? 0.f : num / den);
    if (d == 0) st_shared_f32(p.attn_lse + static_cast<size_t>(head) * p.max_splits + part, empty ? -INFINITY : mx + log2f(den));
  };
  if constexpr (GQA * D <= kThreads) {
    if (c.tid < GQA * D) merge_output(c.tid);
  } else {
    // Two neighbouring dims of one head per thread: the head's maximum, weights and denominator once for both.
    static_assert(GQA * D == 2 * kThreads && D % 2 == 0, "one pair per thread");
    const int h = (2 * c.tid) / D, d = (2 * c.tid) % D;
    float mx = -INFINITY;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) mx = fmaxf(mx, s.merge[w][h][D]);
    float den = 0.f, num0 = 0.f, num1 = 0.f;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) {
      const float mw = s.merge[w][h][D];
      const float wgt = (mw == -INFINITY) ? 0.f : exp2_fast(mw - mx);
      const float2 a = *reinterpret_cast<const float2*>(&s.merge[w][h][d]);
      den = __builtin_fmaf(s.merge[w][h][D + 1], wgt, den);
      num0 = __builtin_fmaf(a.x, wgt, num0);
      num1 = __builtin_fmaf(a.y, wgt, num1);
    }
    const int head = kvh * GQA + h;
    const bool empty = !(den > 0.f);
    float* dst = p.attn_partial + (static_cast<size_t>(head) * p.max_splits + part) * D + d;
    __hip_atomic_store(reinterpret_cast<uint64_t*>(dst),
                       static_cast<uint64_t>(__float_as_uint(empty ? 0.f : num0 / den)) |
                           (static_cast<uint64_t>(__float_as_uint(empty ? 0.f : num1 / den)) << 32),
                       __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (d == 0) st_shared_f32(p.attn_lse + static_cast<size_t>(head) * p.max_splits + part, empty ? -INFINITY : mx + log2f(den));
  }

  QMK_STAMP(2);  // partial merged and stored
  release_stores();
  __syncthreads();
  QMK_STAMP(3);  // stores acknowledged
  if (merge_mode == 2) {  // one arrival per partial on the attention -> O-proj edge
    // (an arrival on every XCD's line where the launch has such lines: Llama shape 1 911 -> 1 931 tok/s)
    if (xcd_counters(p)) {
      if (c.tid < kXcds) publish(sub_counter(p, layer, ROW_REDUCE, c.tid), 1);
    } else if (p.flags & kFlagAttentionRows2To5) {
      if (c.tid < kXcds) publish(counter_ptr(p, layer, ROW_REDUCE, c.tid * kLineInts), 1);
    } else if (c.tid == 0) {
      publish(counter_ptr(p, layer, ROW_REDUCE, 0), 1);
    }
    return true;
  }
  if (!merge_in_last) {
    if (c.tid < M::GQA) publish(counter_ptr(p, layer, ROW_SPLITKV, kvh * M::GQA + c.tid), 1);
    return true;
  }
  // Arrive on the four head counters; whoever sees P-1 earlier arrivals is last.
  if (c.tid < M::GQA) {
    const int prev = __hip_atomic_fetch_add(counter_ptr(p, layer, ROW_SPLITKV, kvh * M::GQA + c.tid), 1,
                                            __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (c.tid == 0) s.ctl[3] = (prev == P - 1);
  }
  __syncthreads();
  if (s.ctl[3]) {  // uniform: every partial of this head group has been acknowledged in memory
    merge_partials<M>(p, kvh * M::GQA, P, nullptr, true, 0);
    release_stores();
    __syncthreads();
    if (p.flags & kFlagRowAttentionLines) {   // (p is the view of one row of a launch of several)
      if (c.tid < kXcds) publish(row_attention_line(p.ws, p.ws_row_units, c.tid), M::GQA);
    } else if (c.tid == 0) {
      publish(counter_ptr(p, layer, ROW_REDUCE, 0), M::GQA);
    }
  }
  return true;
}

// ===================================================================== 3 ==
// [3, layer, head_start, num_partials, len, list..., is_terminal, output_partial]
template <class M>
__device__ bool op_attn_reduce(const Params& p, Smem<M>& s, const Ctx& c) {
  const int layer = s.inst[1], head0 = s.inst[2], P = s.inst[3], n = s.inst[4];
  if (layer < 0 || layer >= p.num_layers) return bad_operand(p, s, c, 1);
  if (head0 < 0 || head0 + M::REDUCE_HEADS > M::NQ) return bad_operand(p, s, c, 2);
  if (n < 1 || n > kMaxPartials || P < 1) return bad_operand(p, s, c, 4);
  for (int i = 0; i < n; ++i)
    if (s.inst[5 + i] < 0 || s.inst[5 + i] >= p.max_splits) return bad_operand(p, s, c, 5 + i);
  const bool terminal = s.inst[5 + n] != 0;
  const int out_slot = s.inst[6 + n];
  if (!terminal && (out_slot < 0 || out_slot >= p.max_splits)) return bad_operand(p, s, c, 6 + n);

  if (!wg_wait(p, s, c, M::REDUCE_HEADS, [&](int i) { return counter_ptr(p, layer, ROW_SPLITKV, head0 + i); }, P)) return false;
  merge_partials<M, M::REDUCE_HEADS>(p, head0, n, &s.inst[5], terminal, out_slot);
  release_stores();
  __syncthreads();
  if (c.tid == 0) publish(counter_ptr(p, layer, ROW_REDUCE, 0), M::REDUCE_HEADS);
  return true;
}

// Two neighbouring residual-stream elements plus bf16(delta), as a bf16 pair.
__device__ __forceinline__ uint32_t residual_word(uint32_t old, float d0, float d1) {
  const uint32_t d = f2bf2(d0, d1);
  return f2bf2(bf_lo(old) + bf_lo(d), bf_hi(old) + bf_hi(d));
}

// The residual-stream pair `pair` of the rows [rs, ...) before this instruction adds to it: from
// the caller's buffer, or from the tagged copy `units` (tag `tag`) of the previous writer.
__device__ __forceinline__ bool residual_in(const Params& p, const uint64_t* units, uint32_t tag, int rs, int pair, uint32_t& old) {
  if (units == nullptr) {
    old = ld_shared32(p.hidden + rs + 2 * pair);
    return true;
  }
  return poll_tagged1(units + (rs + 2 * pair) / 2, tag, p.spin_limit, old);
}

// hidden[r0], hidden[r0+1] += bf16(delta): one coherent 32-bit read-modify-write.
__device__ __forceinline__ void residual_pair(u16* hidden_pair, float d0, float d1) {
  const uint32_t old = ld_shared32(hidden_pair);
  const uint32_t d = f2bf2(d0, d1);
  st_shared32(hidden_pair, f2bf2(bf_lo(old) + bf_lo(d), bf_hi(old) + bf_hi(d)));
}

// Rows kUpGateBuffers .. kUpGateBuffers + PARK_ROWS - 1 of every wave of the up/gate instruction `words` into LDS,
// through registers and one row at a time (16 registers; three rows at once spill): the wave stands here until each
// row has landed, which is why only a workgroup with a long wait ahead does this.
template <class M>
__device__ __forceinline__ void park_upgate_rows(const Params& p, Smem<M>& s, const int32_t* words, int layer, int lane, int wave) {
  if constexpr (M::PARK_ROWS > 0) {
    const int un = words[3], utile = words[5 + un];
#pragma unroll 1
    for (int k = 0; k < M::PARK_ROWS; ++k) {
      const int e = wave + (kUpGateBuffers + k) * kWaves;
      if (e < 2 * un * utile) {
        RowRegs<4> r;
        load_row(r, upgate_row<M>(p, words, layer, utile, e), lane);
#pragma unroll
        for (int j = 0; j < 4; ++j) s.park.v[k][wave][j][lane] = r.v[j];
      }
    }
  }
}

// ===================================================================== 4 ==
// [4, layer, tile_M, n_start, n_end, reduction_block, tile_M_g, tile_N_g]
// hidden[r] = bf16(hidden[r] + bf16(W_o[r] . attn_out))   (operations.py:251-262, 63-68)
template <class M>
__device__ bool op_oproj_residual(const Params& p, Smem<M>& s, const Ctx& c, Carried& carry, bool& carried, bool& parked) {
  constexpr int AW = M::AW;          // columns of W_o: all query heads side by side (= H for the dense models)
  constexpr int CH = AW / 512;
  static_assert(AW % (kThreads * 4) == 0 && AW <= M::F, "whole 8-byte pieces per thread; the vector fits the LDS buffer");
  const int layer = s.inst[1], nstart = s.inst[3], nend = s.inst[4], tile = s.inst[7];
  if (layer < 0 || layer >= p.num_layers) return bad_operand(p, s, c, 1);
  if (tile <= 0 || (tile & 1)) return bad_operand(p, s, c, 7);
  if (nstart < 0 || nend < nstart || static_cast<long>(nend) * tile > M::H) return bad_operand(p, s, c, 4);
  if ((nend - nstart) * tile > kResSlots) return bad_operand(p, s, c, 3);

  const int lane = c.tid & 63;
  const int rs = nstart * tile, nrows = (nend - nstart) * tile;
  const u16* W = p.o_w + (static_cast<size_t>(layer) * M::H + rs) * AW;
  auto src = [&](int r) { return W + static_cast<size_t>(r) * AW; };

  RowRegs<CH> buf[kOprojBuffers];
  preload<CH>(nrows, src, buf);
  // Tagged mode: the rows' residual values are those the previous layer's down projection
  // announced (layer 0: the caller's buffer); they are fetched now, long before they are needed.
  const bool tg = tagged(p);
  const uint32_t tag = tag_of(s.generation, layer);
  if (tg && nrows / 2 > kThreads) return bad_operand(p, s, c, 4);  // one residual pair per thread
  uint32_t res_old = 0;
  if (tg && c.tid < nrows / 2 &&
      !residual_in(p, layer > 0 ? p.ws + kWsHiddenOut : nullptr, tag - 1, rs, c.tid, res_old)) {
    s.ctl[0] = 1;  // seen by everybody after the barrier inside the wait below
    report_error(p, QMK_DEV_WAIT_TIMEOUT, c.inst_idx, c.opcode, c.tid);
  }
  // The next instruction's rows, if it is the up/gate GEMV of this layer (see Carried).
  // (`carried` comes in as "may": a workgroup that has just run this layer's attention starts late,
  // and its requests would stand in front of its own reads of the partials.)
  carried = carried && s.next[0] == OP_RMS_UPGATE_SILU && s.next[1] == layer && upgate_check<M>(p, s.next) < 0;
  if (carried) {
    const int un = s.next[3], utile = s.next[5 + un];
    const int wave = c.tid >> 6;
    static_assert(M::CARRY_ROWS <= kCarried, "the carried rows fit the up/gate ring");
#pragma unroll
    for (int k = 0; k < M::CARRY_ROWS; ++k) {
      const int e = wave + (k + 1) * kWaves;
      if (e < 2 * un * utile) load_row(carry.row[k], upgate_row<M>(p, s.next, layer, utile, e), lane);
    }
  } else {
    forget(carry);
  }
  // A workgroup that waits through the attention phase has LDS to spare as well: the rows behind the up/gate ring go
  // there, after the carried rows' requests (the other way round, and two rows per trip through the carried rows'
  // registers, measured 0.6 % slower).
  parked = parked && carried && M::PARK_ROWS > 0;
  if (parked) park_upgate_rows<M>(p, s, s.next, layer, lane, c.tid >> 6);
  const int self_merge = s.inst[5];  // reduction_block_idx: 0, or the split-KV fan-out P when this op merges
  if (self_merge == 0) {
    if (!wg_wait(p, s, c, 1, [&](int) { return counter_ptr(p, layer, ROW_REDUCE, 0); }, M::NQ)) return false;
#pragma unroll
    for (int k = 0; k < AW / (kThreads * 4); ++k)
      *reinterpret_cast<uint64_t*>(s.x + (c.tid + k * kThreads) * 4) = ld_shared64(p.attn_out + (c.tid + k * kThreads) * 4);
  } else {
    // Every O-proj workgroup merges the split-KV partials itself (python_vm.py:439-488 for all heads):
    // no merging workgroup, no attn_out round trip, one synchronisation hop less.  Item t (one or two
    // per thread) is dims 4*(t % (D/4)).. of head t / (D/4).
    const int P = self_merge;
    if (P < 1 || P > kMaxSelfMerge || P > p.max_splits) return bad_operand(p, s, c, 5);  // no list to fit: any fan-out the workspaces hold
    if (!wg_wait_all(p, s, c, layer, ROW_REDUCE, 0, M::NKV * P)) return false;
    constexpr int kItems = AW / (kThreads * 4);
    const float* lse[kItems];
    const float* part[kItems];
    float mx[kItems], den[kItems], n0[kItems], n1[kItems], n2[kItems], n3[kItems];
#pragma unroll
    for (int k = 0; k < kItems; ++k) {
      const int item = c.tid + k * kThreads;
      const int h = item / (M::D / 4), d0 = 4 * (item % (M::D / 4));
      lse[k] = p.attn_lse + static_cast<size_t>(h) * p.max_splits;
      part[k] = p.attn_partial + static_cast<size_t>(h) * p.max_splits * M::D + d0;
      mx[k] = -INFINITY;
      den[k] = n0[k] = n1[k] = n2[k] = n3[k] = 0.f;
    }
    for (int j0 = 0; j0 < P; j0 += 4) {   // four partials of every item per round, all loads first
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
      *reinterpret_cast<uint2*>(s.x + item * 4) = make_uint2(lo, hi);
      if (nstart == 0) {  // one workgroup also leaves attn_out in memory, as the reference does
        st_shared32(p.attn_out + item * 4, lo);
        st_shared32(p.attn_out + item * 4 + 2, hi);
      }
    }
  }
  __syncthreads();
  QMK_STAMP(0);
  v4u x[CH];
  load_x_from_lds(x, s.x, lane);
  stream<CH>(nrows, src, buf, [&](int r, const RowRegs<CH>& w) {
    const float sum = wave_sum(dot_row(w, x));
    if (lane == 0) s.res[r] = sum;
  });
  QMK_STAMP(1);
  __syncthreads();
  QMK_STAMP(2);
  if (tg) {
    // The new pair goes to the caller's buffer and, tagged, to the up/gate workgroups.
    if (c.tid < nrows / 2) {
      const int pair = c.tid;
      const uint32_t w = residual_word(res_old, s.res[2 * pair], s.res[2 * pair + 1]);
      st_tagged(p.ws + kWsHiddenMid + (rs + 2 * pair) / 2, w, tag);
      st_shared32(p.hidden + rs + 2 * pair, w);
    }
    QMK_STAMP(3);
    return true;
  }
  for (int pair = c.tid; pair < nrows / 2; pair += kThreads)
    residual_pair(p.hidden + rs + 2 * pair, s.res[2 * pair], s.res[2 * pair + 1]);

  release_stores();
  __syncthreads();
  if (c.tid == 0 && nend > nstart) arrive_all(p, layer, ROW_OPROJ, nend - nstart);
  return true;
}

// ===================================================================== 5 ==
// [5, layer, tile_M, n, block_0..block_{n-1}, tile_M_g, tile_N_g]
// up = bf16(W_u y), gate = bf16(W_g y), silu_out = bf16(bf16(silu(gate)) * up)   (operations.py:265-282)
template <class M>
__device__ bool op_rms_upgate_silu(const Params& p, Smem<M>& s, const Ctx& c, const Carried& carry, bool carried, bool parked) {
  constexpr int CH = M::H / 512;
  static_assert(CH == 4, "the carried rows are 4 KiB");
  const int bad = upgate_check<M>(p, s.inst);
  if (bad >= 0) return bad_operand(p, s, c, bad);
  const int layer = s.inst[1], n = s.inst[3];
  const int tile = s.inst[5 + n];

  const int lane = c.tid & 63;
  const int nout = n * tile;       // output elements of this instruction
  const int nrows = 2 * nout;      // streamed rows: element 2i = up row i, 2i+1 = gate row i
  const u16* Wu = p.up_w + static_cast<size_t>(layer) * M::F * M::H;
  const u16* Wg = p.gate_w + static_cast<size_t>(layer) * M::F * M::H;
  auto row_of = [&](int i) { return s.inst[4 + (i >> __builtin_ctz(static_cast<unsigned>(tile)))] * tile + (i & (tile - 1)); };
  auto src = [&](int e) { return upgate_row<M>(p, s.inst, layer, tile, e); };

  bool in_lds = false;   // the O-proj before this instruction has left rows kUpGateBuffers.. of every wave in LDS
  if constexpr (M::PARK_ROWS > 0) in_lds = parked && carried;
  RowRegs<CH> buf[kUpGateBuffers];
  if (carried) {  // the O-proj before this instruction has asked for the elements of buffers 1..
#pragma unroll
    for (int k = 0; k < M::CARRY_ROWS; ++k) buf[k + 1] = carry.row[k];
  }
  const bool tg = tagged(p);
  if (!rms_to_lds<M, kUpGateBuffers>(
          p, s, c, tg ? p.ws + kWsHiddenMid : nullptr, tag_of(s.generation, layer), p.mlp_norm + static_cast<size_t>(layer) * M::H,
          [&](auto k) {
            constexpr int kk = decltype(k)::value;
            if (kk == 0 || kk > M::CARRY_ROWS || !carried) preload_range<kk, kk + 1>(nrows, src, buf);
          },
          [&] { return wg_wait_all(p, s, c, layer, ROW_OPROJ, 0, p.oproj_blocks); }))
    return false;
  QMK_STAMP(0);
  v4u x[CH];
  load_x_from_lds(x, s.x, lane);
  auto use = [&](int e, const RowRegs<CH>& w) {
    const float sum = wave_sum(dot_row(w, x));
    if (lane == 0) s.res[e] = sum;
  };
  // The ring holds the wave's first kUpGateBuffers rows and, when they were parked, LDS the PARK_ROWS behind them: a
  // ring buffer is refilled with the row behind those, and the parked rows are used while the refills are on their
  // way.
  int pk = 0;
  if constexpr (M::PARK_ROWS > 0) pk = in_lds ? M::PARK_ROWS : 0;
  const int wave = c.tid >> 6;
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
  QMK_STAMP(1);
  __syncthreads();
  QMK_STAMP(2);
  // Two neighbouring outputs of a tile leave as one 32-bit word.
  for (int pair = c.tid; pair < nout / 2; pair += kThreads) {
    // elements 4 pair .. 4 pair + 3: up and gate of the pair's two outputs
    const uint32_t ug0 = f2bf2(s.res[4 * pair], s.res[4 * pair + 1]), ug1 = f2bf2(s.res[4 * pair + 2], s.res[4 * pair + 3]);
    const float g0 = bf_hi(ug0), g1 = bf_hi(ug1);
    const uint32_t act = f2bf2(g0 / (1.0f + expf(-g0)), g1 / (1.0f + expf(-g1)));
    const uint32_t word = f2bf2(bf_lo(act) * bf_lo(ug0), bf_hi(act) * bf_lo(ug1));
    st_shared32(p.silu_out + row_of(2 * pair), word);
    if (tg) st_tagged(p.ws + kWsSilu + row_of(2 * pair) / 2, word, tag_of(s.generation, layer));
  }
  QMK_STAMP(3);
  if (tg) return true;  // the down projection polls the units

  release_stores();
  __syncthreads();
  // One arrival per block, on the bucket (= down-projection K slice) it belongs to.
  if (xcd_counters(p)) {
    if (c.tid == 0 && n > 0) arrive_all(p, layer, ROW_UPGATE, n);
  } else if (c.tid < n) {
    publish(counter_ptr(p, layer, ROW_UPGATE, s.inst[4 + c.tid] / p.upgate_blocks_per_bucket), 1);
  }
  return true;
}

// ===================================================================== 6 ==
// bf16 add on one half of a 32-bit word, safe against concurrent adders of
// other K slices (only needed when the down projection is split along K).
__device__ __forceinline__ void atomic_add_bf16(u16* addr, float delta) {
  uint32_t* word = reinterpret_cast<uint32_t*>(reinterpret_cast<uintptr_t>(addr) & ~uintptr_t(3));
  const bool high = (reinterpret_cast<uintptr_t>(addr) & 2) != 0;
  uint32_t seen = ld_shared32(word);
  while (true) {
    const u16 cur = high ? static_cast<u16>(seen >> 16) : static_cast<u16>(seen & 0xffffu);
    const u16 nxt = f2bf(bf2f(cur) + delta);
    const uint32_t want = high ? ((seen & 0x0000ffffu) | (static_cast<uint32_t>(nxt) << 16))
                               : ((seen & 0xffff0000u) | nxt);
    if (__hip_atomic_compare_exchange_strong(word, &seen, want, __ATOMIC_RELAXED, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) break;
  }
}

// [6, layer, tile_M, n_start, n_end, split_K_idx, tile_M_g, tile_N_g, split_K_g]
// hidden[r] = bf16(hidden[r] + bf16(W_d[r, slice] . silu_out[slice]))   (operations.py:285-295;
// python_vm.py:137-171 for the sliced form).  With one slice this is the fused form exactly.
// A row's K slice is streamed as 2048-column segments: element e = (row e / segs, segment e % segs).
template <class M>
__device__ bool op_down_residual(const Params& p, Smem<M>& s, const Ctx& c) {
  constexpr int CH = 4;
  const int layer = s.inst[1], nstart = s.inst[3], nend = s.inst[4], split = s.inst[5];
  const int tile = s.inst[7], kg = s.inst[8];
  if (layer < 0 || layer >= p.num_layers) return bad_operand(p, s, c, 1);
  if (tile <= 0 || (tile & 1)) return bad_operand(p, s, c, 7);
  if (nstart < 0 || nend < nstart || static_cast<long>(nend) * tile > M::H) return bad_operand(p, s, c, 4);
  if ((nend - nstart) * tile > kResSlots) return bad_operand(p, s, c, 3);
  if (kg <= 0 || kg % (512 * CH) != 0 || kg > M::F) return bad_operand(p, s, c, 8);
  if (split < 0 || static_cast<long>(split + 1) * kg > M::F) return bad_operand(p, s, c, 5);
  if (split >= p.barrier_slots) return bad_operand(p, s, c, 5);

  const int lane = c.tid & 63, wave = c.tid >> 6;
  const int rs = nstart * tile, nrows = (nend - nstart) * tile, ks = split * kg;
  const int segs = kg / (512 * CH);
  // Element order is chosen per wave so that a wave owns whole rows: wave w streams the
  // segments of rows w, w+8, ...  Element index e (as seen by `stream`: e = w + 8*i) maps to
  // step i of wave w: row = w + 8*(i / segs), segment = i % segs.
  // (i / segs as a multiplication: exact for the few steps a wave has, and an integer division costs forty instructions)
  const int inv_segs = (65536 + segs - 1) / segs;
  auto step_row = [&](int e) { return ((e >> 3) * inv_segs) >> 16; };
  auto row_of = [&](int e) { return (e & (kWaves - 1)) + kWaves * step_row(e); };
  auto seg_of = [&](int e) { return (e >> 3) - step_row(e) * segs; };
  const u16* W = p.down_w + (static_cast<size_t>(layer) * M::H + rs) * M::F + ks;
  auto src = [&](int e) { return W + static_cast<size_t>(row_of(e)) * M::F + seg_of(e) * (512 * CH); };
  // Number of stream elements: waves with fewer rows simply run out earlier; bound by the largest.
  const int rows_w = (nrows - wave + kWaves - 1) / kWaves;          // rows owned by this wave (may be 0)
  const int n_elems = wave + kWaves * (rows_w * segs - 1) + 1;      // last element index of this wave + 1 (<= wave if none)

  RowRegs<CH> buf[kDepth];
  static_assert(kEarly <= kDepth, "early buffers are a subset of the ring");
  preload_range<0, kEarly>(rows_w > 0 ? n_elems : 0, src, buf);
  const bool tg = tagged(p);
  const uint32_t tag = tag_of(s.generation, layer);
  if ((xcd_counters(p) || tg) && (split != 0 || kg != M::F)) return bad_operand(p, s, c, 8);  // one K slice only
  if (tg && nrows / 2 > kThreads) return bad_operand(p, s, c, 4);  // one residual pair per thread
  // Tagged mode: the rows' residual values as the O-proj announced them, fetched ahead of time.
  uint32_t res_old = 0;
  if (tg && c.tid < nrows / 2 && !residual_in(p, p.ws + kWsHiddenMid, tag, rs, c.tid, res_old)) {
    s.ctl[0] = 1;  // seen by everybody after the barrier inside the wait below
    report_error(p, QMK_DEV_WAIT_TIMEOUT, c.inst_idx, c.opcode, c.tid);
  }
  if (tg) {
    // silu_out from its tagged units: thread t polls the unit pairs 2t + 1024k until they carry
    // this layer's tag; pairs already staged are not fetched again.
    static_assert(M::F % (4 * kThreads) == 0, "whole unit pairs per thread");
    constexpr int kPairs = M::F / (4 * kThreads);
    uint32_t* words = reinterpret_cast<uint32_t*>(s.x);
    const uint64_t* mine = p.ws + kWsSilu + 2 * c.tid;
    uint32_t polls = 0;
    bool have[kPairs];
#pragma unroll
    for (int k = 0; k < kPairs; ++k) have[k] = false;
    while (true) {
      uint64_t u[2 * kPairs];
#pragma unroll
      for (int k = 0; k < kPairs; ++k) {
        if (!have[k]) {
          u[2 * k] = ld_shared64(mine + 1024 * k);
          u[2 * k + 1] = ld_shared64(mine + 1024 * k + 1);
        }
      }
      bool all = true;
#pragma unroll
      for (int k = 0; k < kPairs; ++k) {
        if (!have[k] && static_cast<uint32_t>(u[2 * k] >> 32) == tag && static_cast<uint32_t>(u[2 * k + 1] >> 32) == tag) {
          words[2 * c.tid + 1024 * k] = static_cast<uint32_t>(u[2 * k]);
          words[2 * c.tid + 1024 * k + 1] = static_cast<uint32_t>(u[2 * k + 1]);
          have[k] = true;
        }
        all = all && have[k];
      }
      if (all) break;
      if (++polls > p.spin_limit) {
        s.ctl[0] = 1;
        report_error(p, QMK_DEV_WAIT_TIMEOUT, c.inst_idx, c.opcode, c.tid);
        break;
      }
      __builtin_amdgcn_s_sleep(8);
    }
    preload_range<kEarly, kDepth>(rows_w > 0 ? n_elems : 0, src, buf);
    if (p.timeline != nullptr && c.tid == 0) {
      s.t_wait = wall_clock64();
      s.ctl[2] = 1;
    }
    __syncthreads();
    if (s.ctl[0]) return false;
  } else {
  if (!wg_wait_all(p, s, c, layer, ROW_UPGATE, split, p.upgate_blocks_per_bucket)) return false;

  // The K slice of silu_out into LDS; the remaining row buffers are requested behind it.
  constexpr int kActLoads = (M::F / 4 + kThreads - 1) / kThreads;  // 8-byte loads per thread that cover the widest slice
  uint64_t act[kActLoads];
#pragma unroll
  for (int k = 0; k < kActLoads; ++k)
    if (c.tid + k * kThreads < kg / 4) act[k] = ld_shared64(p.silu_out + ks + (c.tid + k * kThreads) * 4);
  asm volatile("" ::: "memory");
  preload_range<kEarly, kDepth>(rows_w > 0 ? n_elems : 0, src, buf);
#pragma unroll
  for (int k = 0; k < kActLoads; ++k)
    if (c.tid + k * kThreads < kg / 4) reinterpret_cast<uint64_t*>(s.x)[c.tid + k * kThreads] = act[k];
  __syncthreads();
  }

  float acc = 0.f;
  stream<CH>(rows_w > 0 ? n_elems : 0, src, buf, [&](int e, const RowRegs<CH>& w) {
    const int seg = seg_of(e);
    v4u x[CH];
    load_x_from_lds(x, s.x + seg * (512 * CH), lane);
#pragma unroll
    for (int j = 0; j < CH; ++j) acc = dot8(w.v[j], x[j], acc);
    if (seg == segs - 1) {
      const float sum = wave_sum(acc);
      acc = 0.f;
      if (lane == 0) s.res[row_of(e)] = sum;
    }
  });
  QMK_STAMP(1);
  __syncthreads();
  QMK_STAMP(2);

  if (tg) {
    if (c.tid < nrows / 2) {
      const int pair = c.tid;
      const uint32_t w = residual_word(res_old, s.res[2 * pair], s.res[2 * pair + 1]);
      st_tagged(p.ws + kWsHiddenOut + (rs + 2 * pair) / 2, w, tag);
      st_shared32(p.hidden + rs + 2 * pair, w);
    }
    QMK_STAMP(3);
    return true;
  }
  if (kg == M::F) {  // one slice: every row has a single writer
    for (int pair = c.tid; pair < nrows / 2; pair += kThreads)
      residual_pair(p.hidden + rs + 2 * pair, s.res[2 * pair], s.res[2 * pair + 1]);
  } else {           // other slices add to the same rows concurrently
    for (int r = c.tid; r < nrows; r += kThreads) atomic_add_bf16(p.hidden + rs + r, round_bf16(s.res[r]));
  }

  release_stores();
  __syncthreads();
  if (c.tid == 0 && nend > nstart) arrive_all(p, layer, ROW_DOWN, nend - nstart);
  return true;
}

// ===================================================================== 7 ==
// [7, start_block, end_block, tile_M_g, tile_N_g]     logits = bf16(W_lm . rms(hidden))
template <class M>
__device__ bool op_rms_lmhead(const Params& p, Smem<M>& s, const Ctx& c) {
  constexpr int CH = M::H / 512;
  const int bstart = s.inst[1], bend = s.inst[2], tile = s.inst[4];
  if (tile <= 0) return bad_operand(p, s, c, 4);
  if (bstart < 0 || bend < bstart || static_cast<long>(bend) * tile > p.vocab_size) return bad_operand(p, s, c, 2);
  if (p.num_layers < 1) return bad_operand(p, s, c, 0);

  const int lane = c.tid & 63;
  const int rs = bstart * tile, nrows = (bend - bstart) * tile;
  const u16* W = p.lm_w + static_cast<size_t>(rs) * M::H;
  auto src = [&](int r) { return W + static_cast<size_t>(r) * M::H; };

  RowRegs<CH> buf[kDepth];
  preload<CH>(nrows, src, buf);
  const bool tg = tagged(p);
  if (!tg && !wg_wait_all(p, s, c, p.num_layers - 1, M::PREV_ROW, 0, p.down_arrivals)) return false;
  if (!rms_to_lds(p, s, c, tg ? p.ws + kWsHiddenOut : nullptr, tag_of(s.generation, p.num_layers - 1), p.lm_norm)) return false;
  v4u x[CH];
  load_x_from_lds(x, s.x, lane);
  // Terminal op: nothing inside the launch reads the logits, so ordinary stores do.  A wave sees
  // its rows in increasing order, so "strictly greater" keeps the first row of a tie.
  float best = -INFINITY;
  int best_row = 0x7fffffff;
  stream<CH>(nrows, src, buf, [&](int r, const RowRegs<CH>& w) {
    const float sum = wave_sum(dot_row(w, x));
    const u16 logit = f2bf(sum);
    if (lane == 0) p.logits[rs + r] = logit;
    const float v = bf2f(logit);
    if (v > best) {
      best = v;
      best_row = rs + r;
    }
  });
  if (p.token_out != nullptr) {  // greedy candidate of this workgroup (several LM-head instructions accumulate)
    if (lane == 0) {
      s.red[c.tid >> 6] = best;
      s.wave_idx[c.tid >> 6] = best_row;
    }
    __syncthreads();
    if (c.tid == 0) {
      float v = s.best_val;
      int i = s.best_idx;
      for (int w = 0; w < kWaves; ++w)
        if (s.red[w] > v || (s.red[w] == v && s.wave_idx[w] < i)) {
          v = s.red[w];
          i = s.wave_idx[w];
        }
      s.best_val = v;
      s.best_idx = i;
    }
  }
  return true;
}

}  // namespace qmk
