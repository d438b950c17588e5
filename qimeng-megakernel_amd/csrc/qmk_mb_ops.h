// The ten opcodes of the batch decode route (2..16 rows decoded together) as workgroup-wide device
// functions for gfx950.
//
// Semantics follow the reference's batch route: arithmetic and rounding points from its fused
// PyTorch operations run on [B, H] activations
// (qimeng_megakernel/models/LLM/llama/llama3_2__1b/A100/multi_batch/decode_schedule/fused/__init__.py,
//  …/single_batch/decode_schedule/fused/operations.py:126-321), operand layout, per-row state and the
// counter protocol from its instruction VM (…/multi_batch/decode_schedule/instructions/python_vm.py:139-730).
//
// The projections are GEMMs with a skinny activation side: a block is 16 weight rows, the batch
// rows are the (at most 16) columns.  v_mfma_f32_16x16x32_bf16 takes the 16 weight rows as A and the
// batch as B: lane l holds A[row l%16][k 8*(l/16)..+7], B[k 8*(l/16)..+7][column l%16] and
// C[row 4*(l/16)..+3][column l%16].  Which 8 columns of a 32-column chunk sit in which k slot is
// free as long as both operands agree, so a lane simply reads 16 contiguous bytes of its weight row
// and of its batch row.  The eight waves of a workgroup split K: wave w owns a 256-column segment
// (four of them for K = 8192) of the block, keeps its share of the activations in registers for the
// whole instruction and streams weight segments through a register ring; the eight partial 16x16
// tiles meet in LDS, where 128 threads add them up and apply the epilogue to two neighbouring
// outputs each.  Weights cross the memory system once per step whatever the batch size: the bound
// is still HBM.
#pragma once

#include "qmk_ops.h"

namespace qmk {
namespace mb {

constexpr int kTile = 16;       // weight rows per block (the reference's tile_N_granularity)
constexpr int kMaxBatch = 16;   // batch rows = columns of one matrix-core tile (tile_M_granularity)
constexpr int kChunk = 32;      // K per matrix-core instruction
constexpr int kSeg = 256;       // K columns of one segment: 8 chunks, 16 bytes per lane each
constexpr int kSegChunks = kSeg / kChunk;
constexpr int kMaxList = kInstWords - 10;  // reduction list: 6 leading and 4 trailing words
constexpr float kNoContribution = -79.0f;  // without a validity buffer: partials at or below do not count

enum Opcode {
  OP_NOOP = 0,
  OP_ATTN_RMS = 1,
  OP_QKV = 2,
  OP_SPLITKV = 3,
  OP_REDUCE = 4,
  OP_OPROJ = 5,
  OP_MLP_RMS = 6,
  OP_UPGATE = 7,
  OP_DOWN = 8,
  OP_LM_RMS = 9,
  OP_LMHEAD = 10,
};
// Counter rows: opcode - 1.
constexpr int ROW_ATTN_RMS = 0, ROW_QKV = 1, ROW_SPLITKV = 2, ROW_REDUCE = 3, ROW_OPROJ = 4, ROW_MLP_RMS = 5, ROW_UPGATE = 6,
              ROW_DOWN = 7, ROW_LM_RMS = 8;

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f4 __attribute__((ext_vector_type(4)));

// Two floats to a bf16 pair, round-to-nearest-even (v_cvt_pk_bf16_f32: the rounding torch applies on
// .to(bfloat16)), low half first.
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2{lo, hi}, bf16x2));
}
// old + bf16(delta) on a bf16 pair: the residual add of two neighbouring elements.
__device__ __forceinline__ uint32_t residual_add(uint32_t old, float d0, float d1) {
  const uint32_t d = pack_bf16(d0, d1);
  return pack_bf16(bf_lo(old) + bf_lo(d), bf_hi(old) + bf_hi(d));
}

// Validity flags are bytes that one workgroup writes and another reads within the launch.
__device__ __forceinline__ void st_shared8(uint8_t* p, uint8_t v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ uint8_t ld_shared8(const uint8_t* p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }

template <class M>
struct Smem {
  int32_t inst[kInstWords];
  int32_t ctl[8];                  // [0] abort, [1] last workgroup to retire, [2] a wait was timed
  int32_t pos[kMaxBatch];          // position of the token each row decodes
  int32_t active[kMaxBatch];       // rows that still generate
  float red[kWaves];
  float part[2][2][kWaves][kMaxBatch][kTile];  // [parity][unit][wave][batch row][weight row]: K-slice partial tiles
  alignas(16) u16 stage[M::GQA * M::D + 2 * M::D];  // attention: q heads, then the K and V row of this step
  float merge[kWaves][M::GQA][M::D + 4];
  unsigned long long t_wait;
  unsigned long long stamps[4];
  // One weight segment per wave ([wave][chunk][lane]) fetched before a wait that the registers have no room for: the
  // gate segment of an up/gate instruction's third block, the fourth segment of a down projection's first block.
  alignas(16) v4u seg_park[kWaves][kSegChunks][64];
};

#define QMK_MB_STAMP(k)                                                     \
  do {                                                                      \
    if (p.timeline != nullptr && c.tid == 0) s.stamps[k] = wall_clock64(); \
  } while (0)

template <class S>
__device__ __forceinline__ bool bad_operand(const Params& p, S& s, const Ctx& c, int operand) {
  if (c.tid == 0) report_error(p, QMK_DEV_BAD_OPERAND, c.inst_idx, c.opcode, operand);
  return false;
}

// Lanes 0..n-1 each poll the counter `ctr_of(i)` up to `expected(i)`; false (uniformly) on a timeout.
template <class S, class CtrOf, class Expected>
__device__ __forceinline__ bool wait_counters(const Params& p, S& s, const Ctx& c, int n, CtrOf ctr_of, Expected expected) {
  if (c.tid < n) {
    if (!poll_counter(ctr_of(c.tid), expected(c.tid), p.spin_limit)) {
      s.ctl[0] = 1;
      report_error(p, QMK_DEV_WAIT_TIMEOUT, c.inst_idx, c.opcode, c.tid);
    }
  }
  if (p.timeline != nullptr && c.tid == 0) {
    s.t_wait = wall_clock64();
    s.ctl[2] = 1;
  }
  __syncthreads();
  return s.ctl[0] == 0;
}
template <class S>
__device__ __forceinline__ bool wait_counter(const Params& p, S& s, const Ctx& c, int layer, int row, int expected) {
  return wait_counters(p, s, c, 1, [&](int) { return counter_ptr(p, layer, row, 0); }, [&](int) { return expected; });
}

// All stores of the workgroup are in memory; then thread 0 adds `amount` to one counter.
__device__ __forceinline__ void publish_after_stores(const Params& p, const Ctx& c, int layer, int row, int slot, int amount) {
  release_stores();
  __syncthreads();
  if (c.tid == 0) publish(counter_ptr(p, layer, row, slot), amount);
}

// ---- the all-to-all edges' arrivals on eight lines (QMK_FLAG_XCD_COUNTERS) ----
// The O-projection, the up/gate and the down projection each count 128..512 blocks on word 0 of their counter row, and
// every one of those arrivals is a read-modify-write of the same line from another XCD: the last of them is seen
// microseconds after it was sent.  With the flag an arrival goes to the sub-counter of the sender's XCD (workgroup % 8:
// word 32 * xcd of the same row, a line of its own; the rows have no other user, and word 0 is one of the eight), and a
// waiting workgroup's first eight lanes read the eight words and add them up.  A row needs 256 words for it.
constexpr int kSpread = kXcds;
__device__ __forceinline__ bool spread_counters(const Params& p) { return (p.flags & QMK_FLAG_XCD_COUNTERS) != 0; }
__device__ __forceinline__ void publish_edge_after_stores(const Params& p, const Ctx& c, int layer, int row, int amount) {
  publish_after_stores(p, c, layer, row, spread_counters(p) ? kLineInts * static_cast<int>(blockIdx.x & (kSpread - 1)) : 0, amount);
}
template <class S>
__device__ __forceinline__ bool wait_edge(const Params& p, S& s, const Ctx& c, int layer, int row, int expected) {
  if (!spread_counters(p)) return wait_counter(p, s, c, layer, row, expected);
  if (c.tid < kSpread) {
    const int32_t* mine = counter_ptr(p, layer, row, kLineInts * c.tid);
    uint32_t polls = 0;
    while (true) {
      int v = __hip_atomic_load(mine, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      v += __shfl_xor(v, 1, kSpread);
      v += __shfl_xor(v, 2, kSpread);
      v += __shfl_xor(v, 4, kSpread);
      if (v >= expected) break;
      if (++polls > p.spin_limit) {   // the same for all eight lanes
        if (c.tid == 0) {
          s.ctl[0] = 1;
          report_error(p, QMK_DEV_WAIT_TIMEOUT, c.inst_idx, c.opcode, 0);
        }
        break;
      }
      __builtin_amdgcn_s_sleep(2);
    }
  }
  if (p.timeline != nullptr && c.tid == 0) {
    s.t_wait = wall_clock64();
    s.ctl[2] = 1;
  }
  __syncthreads();
  return s.ctl[0] == 0;
}

// Counters that are neighbours in one line by the reference's layout (the 48 head counters of the QKV projection, the B
// row counters of the attention outputs) move a line apart with the flag: word i -> line i % 8, word i / 8 of it
// (Llama shape, 8 rows: +0.5 %).
__device__ __forceinline__ int apart(const Params& p, int i) { return spread_counters(p) ? kLineInts * (i & 7) + (i >> 3) : i; }

// The B rows of an RMSNorm round are few arrivals, but every workgroup of the next GEMM polls them: 128..256 pollers on
// one line stand in each other's way (and in the arrivals').  With the flag a row arrives on all eight lines, and a
// workgroup polls the line of its own XCD (Llama shape: 8 rows 8 890 -> 9 110 tok/s, 16 rows 15 550 -> 16 050).
template <class S>
__device__ __forceinline__ bool wait_rows_done(const Params& p, S& s, const Ctx& c, int layer, int row, int expected) {
  if (spread_counters(p))
    return wait_counters(p, s, c, 1, [&](int) { return counter_ptr(p, layer, row, kLineInts * static_cast<int>(blockIdx.x & (kSpread - 1))); },
                         [&](int) { return expected; });
  return wait_counter(p, s, c, layer, row, expected);
}

// ================================================================ 1, 6, 9 ==
// [op, layer, batch_size, -, -, -, batch_row]   (9: [op, batch_size, -, -, -, -, batch_row])
// dst[row] = RMSNorm(hidden[row]) for an active row, zeros otherwise   (python_vm.py:139-160, 614-634, 668-690)
template <class M>
__device__ bool op_rms_row(const Params& p, Smem<M>& s, const Ctx& c) {
  static_assert(M::H == kThreads * 4, "one thread normalises four elements");
  const bool lm = c.opcode == OP_LM_RMS;
  const int layer = lm ? p.num_layers - 1 : s.inst[1];
  const int B = lm ? s.inst[1] : s.inst[2], row = s.inst[6];
  if (layer < 0 || layer >= p.num_layers) return bad_operand(p, s, c, 1);
  if (B != p.batch) return bad_operand(p, s, c, lm ? 1 : 2);
  if (row < 0 || row >= B) return bad_operand(p, s, c, 6);
  const u16* weight;
  u16* dst;
  int my_row, wait_layer = layer, wait_row;
  if (c.opcode == OP_ATTN_RMS) {
    weight = p.attn_norm + static_cast<size_t>(layer) * M::H, dst = p.attn_rms_out, my_row = ROW_ATTN_RMS;
    wait_layer = layer - 1, wait_row = ROW_DOWN;
  } else if (c.opcode == OP_MLP_RMS) {
    weight = p.mlp_norm + static_cast<size_t>(layer) * M::H, dst = p.mlp_rms_out, my_row = ROW_MLP_RMS, wait_row = ROW_OPROJ;
  } else {
    weight = p.lm_norm, dst = p.lm_rms_out, my_row = ROW_LM_RMS, wait_row = ROW_DOWN;
  }
  const uint2 wv = *reinterpret_cast<const uint2*>(weight + c.tid * 4);
  const int produced = wait_row == ROW_OPROJ ? p.oproj_blocks : p.down_arrivals;   // blocks of the projection that completes the rows
  if (wait_layer >= 0 && !wait_edge(p, s, c, wait_layer, wait_row, produced)) return false;
  uint32_t lo = 0, hi = 0;
  if (s.active[row]) {
    const uint64_t hw = ld_shared64(p.hidden + static_cast<size_t>(row) * M::H + c.tid * 4);
    const float x0 = bf_lo(static_cast<uint32_t>(hw)), x1 = bf_hi(static_cast<uint32_t>(hw));
    const float x2 = bf_lo(static_cast<uint32_t>(hw >> 32)), x3 = bf_hi(static_cast<uint32_t>(hw >> 32));
    float ss = __builtin_fmaf(x3, x3, __builtin_fmaf(x2, x2, __builtin_fmaf(x1, x1, x0 * x0)));
    ss = block_sum(ss, s.red);
    const float rstd = 1.0f / sqrtf(ss / static_cast<float>(M::H) + p.rms_norm_eps);
    lo = static_cast<uint32_t>(f2bf(bf_lo(wv.x) * round_bf16(x0 * rstd))) | (static_cast<uint32_t>(f2bf(bf_hi(wv.x) * round_bf16(x1 * rstd))) << 16);
    hi = static_cast<uint32_t>(f2bf(bf_lo(wv.y) * round_bf16(x2 * rstd))) | (static_cast<uint32_t>(f2bf(bf_hi(wv.y) * round_bf16(x3 * rstd))) << 16);
  }
  __hip_atomic_store(reinterpret_cast<uint64_t*>(dst + static_cast<size_t>(row) * M::H + c.tid * 4), (static_cast<uint64_t>(hi) << 32) | lo,
                     __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  if (spread_counters(p)) {   // one arrival on every XCD's line: each consumer polls the line of its own XCD
    release_stores();
    __syncthreads();
    if (c.tid < kSpread) publish(counter_ptr(p, layer, my_row, kLineInts * c.tid), 1);
    return true;
  }
  publish_after_stores(p, c, layer, my_row, 0, 1);
  return true;
}

// ------------------------------------------------------------ GEMM core ----
// One lane's share of a 16-row x 256-column weight segment: row l%16, 16 bytes of each 64-byte chunk.
// Ordinary loads: an instruction takes 64 bytes of each of 16 rows, the next one the other half of the
// same 128-byte lines; with the streaming hint the second half misses again (measured: LM head 101 -> 90 us).
struct Seg {
  v4u a[kSegChunks];
};
__device__ __forceinline__ void load_seg(Seg& sg, const u16* lane_ptr) {
#pragma unroll
  for (int j = 0; j < kSegChunks; ++j) sg.a[j] = *reinterpret_cast<const v4u*>(lane_ptr + j * kChunk);
}
__device__ __forceinline__ f4 mma_seg(const Seg& sg, const v4u (&x)[kSegChunks], f4 acc) {
#pragma unroll
  for (int j = 0; j < kSegChunks; ++j)
    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, sg.a[j]), __builtin_bit_cast(bf16x8, x[j]), acc, 0, 0, 0);
  return acc;
}
// This lane's share of the activations [B, ld] for one segment: batch row l%16 (zeros beyond the
// batch), the same 16 bytes of every chunk as the weights.  The buffers are written during the launch
// by other workgroups, so the loads are device-coherent (sc1) like ld_shared128 — but as one 16-byte
// buffer load per chunk instead of two 8-byte ones: half the requests for the same bytes.
__device__ __forceinline__ void load_x(v4u (&x)[kSegChunks], const u16* act, int ld, int B, int k0, int lane) {
  const int n = lane & 15, g = lane >> 4;
  constexpr int kDeviceCoherent = 16;   // the sc1 bit of the cache policy operand
  // The descriptor is built where it is used: through an opaque copy of the pointer, so that the
  // descriptors of all five activation tensors are not computed once for all ops and kept in registers.
  u16* base = const_cast<u16*>(act);
  asm volatile("" : "+s"(base));
  const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(base, 0, 0x7fffffff, 0x00020000);
  const uint32_t at = (static_cast<uint32_t>(n) * ld + k0 + g * 8) * 2;
#pragma unroll
  for (int j = 0; j < kSegChunks; ++j) {
    x[j] = v4u{0, 0, 0, 0};
    if (n < B) x[j] = __builtin_bit_cast(v4u, __builtin_amdgcn_raw_buffer_load_b128(rsrc, at + j * kChunk * 2, 0, kDeviceCoherent));
  }
}
// The wave's partial tile (C layout: rows 4*(l/16)..+3, column l%16) into its LDS slot.
template <class M>
__device__ __forceinline__ void park(Smem<M>& s, int parity, int unit, int wave, int lane, f4 acc) {
  *reinterpret_cast<f4*>(&s.part[parity][unit][wave][lane & 15][4 * (lane >> 4)]) = acc;
}
// Outputs (2*rp, 2*rp + 1) of the block for batch row b: the eight K-slice partials added up.
template <class M>
__device__ __forceinline__ float2 gather(const Smem<M>& s, int parity, int unit, int b, int rp) {
  float2 v = float2{0.f, 0.f};
#pragma unroll
  for (int w = 0; w < kWaves; ++w) {
    const float2 t = *reinterpret_cast<const float2*>(&s.part[parity][unit][w][b][2 * rp]);
    v.x += t.x;
    v.y += t.y;
  }
  return v;
}

// Blocks 0..n-1 of NU weight matrices with K = 2048 (one segment per wave).  `src(j, u)` is the
// address of row 0, column 0 of block j in matrix u (rows are `M::H` apart); `before(j)` runs on
// all threads right after the block's tiles are parked (still before the barrier), `epi(j, parity,
// b, rp)` on threads 0..127 after it.  The ring holds NB blocks; the first NB are requested at once
// (the caller decides whether that is before or after its wait through `wait`).
// `rows` (16, or 8): weight rows per block; with 8 the upper half of the tile repeats the lower one
// (the same addresses: no extra traffic) and only outputs 0..7 are used.
// `PARK`: the first matrix's segment of block NB — the first one the ring has no room for — is fetched before the wait
// as well and waits in LDS (s.seg_park) until the ring's first slot is free.
template <class M, int NU, int NB, bool PARK = false, class Src, class Wait, class Epi>
__device__ __forceinline__ bool gemm_h(const Params& p, Smem<M>& s, const Ctx& c, int n, const u16* act, int B, Src src, Wait wait, Epi epi,
                                       int rows = kTile) {
  static_assert(M::H == kWaves * kSeg, "one segment per wave");
  const int lane = c.tid & 63, wave = c.tid >> 6;
  const size_t lane_off = static_cast<size_t>(lane & (rows - 1)) * M::H + wave * kSeg + (lane >> 4) * 8;
  Seg ring[NB][NU];
#pragma unroll
  for (int k = 0; k < NB; ++k)
    if (k < n)
#pragma unroll
      for (int u = 0; u < NU; ++u) load_seg(ring[k][u], src(k, u) + lane_off);
  if constexpr (PARK) {
    if (n > NB) {
      Seg extra;
      load_seg(extra, src(NB, 0) + lane_off);
#pragma unroll
      for (int j = 0; j < kSegChunks; ++j) s.seg_park[wave][j][lane] = extra.a[j];
    }
  }
  if (!wait()) return false;
  v4u x[kSegChunks];
  load_x(x, act, M::H, B, wave * kSeg, lane);
  int parity = 0;
  for (int j0 = 0; j0 < n; j0 += NB) {
#pragma unroll
    for (int k = 0; k < NB; ++k) {
      const int j = j0 + k;
      if (j < n) {  // uniform over the workgroup
#pragma unroll
        for (int u = 0; u < NU; ++u) {
          const f4 acc = mma_seg(ring[k][u], x, f4{0.f, 0.f, 0.f, 0.f});
          park(s, parity, u, wave, lane, acc);
          if (j + NB < n) {
            if (PARK && j == 0 && u == 0) {
#pragma unroll
              for (int q = 0; q < kSegChunks; ++q) ring[k][u].a[q] = s.seg_park[wave][q][lane];
            } else {
              load_seg(ring[k][u], src(j + NB, u) + lane_off);
            }
          }
        }
        __syncthreads();
        // Parity: a slot is written again two blocks later, behind the next barrier, which the
        // reading threads reach only after they are done with it.
        if (c.tid < 8 * rows) epi(j, parity, c.tid & 15, c.tid >> 4);
        parity ^= 1;
      }
    }
  }
  return true;
}

// ===================================================================== 2 ==
// [2, layer, batch_size, tile_M, n_start, n_end, tile_M_g, tile_N_g]
// QKV rows of blocks [n_start, n_end) for every batch row from attn_rms_out; RoPE at the row's
// position on q and k; q -> q_post_rope, k/v -> the row's cache line at its position
// (python_vm.py:163-266).  One arrival per block on the counter of the block's head.
template <class M>
__device__ bool op_qkv(const Params& p, Smem<M>& s, const Ctx& c) {
  const int layer = s.inst[1], B = s.inst[2], n0 = s.inst[4], n1 = s.inst[5];
  if (layer < 0 || layer >= p.num_layers) return bad_operand(p, s, c, 1);
  if (B != p.batch || s.inst[3] != 0) return bad_operand(p, s, c, 2);
  if (n0 < 0 || n1 < n0 || n1 > M::QKV / kTile) return bad_operand(p, s, c, 4);
  if (s.inst[6] != kMaxBatch || s.inst[7] != kTile) return bad_operand(p, s, c, 7);
  const u16* w = p.qkv_w + static_cast<size_t>(layer) * M::QKV * M::H;
  const size_t tok_stride = static_cast<size_t>(M::NKV) * M::D;
  const bool ok = gemm_h<M, 1, 3>(
      p, s, c, n1 - n0, p.attn_rms_out, B, [&](int j, int) { return w + static_cast<size_t>(n0 + j) * kTile * M::H; },
      [&] { return wait_rows_done(p, s, c, layer, ROW_ATTN_RMS, B); },
      [&](int j, int parity, int b, int rp) {
        if (b >= B || !s.active[b]) return;
        const float2 v = gather(s, parity, 0, b, rp);
        const uint32_t vb = pack_bf16(v.x, v.y);
        const float v0 = bf_lo(vb), v1 = bf_hi(vb);
        const int o = (n0 + j) * kTile + 2 * rp, d = o % M::D, pos = s.pos[b];
        if constexpr (M::QK_NORM) {   // Qwen3 op set: the raw vector; norm, RoPE and the cache rows belong to the attention prologue
          st_shared32(p.qkv_raw + static_cast<size_t>(b) * M::QKV + o, vb);
          return;
        }
        const size_t cache_row = ((static_cast<size_t>(layer) * B + b) * p.max_seq_len + pos) * tok_stride;
        if (o < M::NQ * M::D) {
          st_shared32(p.q_post_rope + static_cast<size_t>(b) * M::NQ * M::D + o,
                      rope_pair(v0, v1, p.rope_cos + static_cast<size_t>(pos) * M::D, p.rope_sin + static_cast<size_t>(pos) * M::D, d));
        } else if (o < (M::NQ + M::NKV) * M::D) {
          st_shared32(p.k_cache + cache_row + (o - M::NQ * M::D),
                      rope_pair(v0, v1, p.rope_cos + static_cast<size_t>(pos) * M::D, p.rope_sin + static_cast<size_t>(pos) * M::D, d));
        } else {
          st_shared32(p.v_cache + cache_row + (o - (M::NQ + M::NKV) * M::D), vb);
        }
      });
  if (!ok) return false;
  release_stores();
  __syncthreads();
  if (c.tid < n1 - n0) publish(counter_ptr(p, layer, ROW_QKV, apart(p, (n0 + c.tid) / (M::D / kTile))), 1);
  return true;
}

// Log-sum-exp merge (log2 domain) of partials list[0..n) (null: 0..n-1) of the GQA query heads from
// head0 of batch row b, over the valid ones only (python_vm.py:442-551).  Thread t < GQA*D/2
// produces two neighbouring dims.  All reads are issued before the first use.
template <class M>
__device__ __forceinline__ void merge_heads(const Params& p, const Ctx& c, int b, int head0, int n, const int32_t* list, bool terminal,
                                            int out_slot) {
  constexpr int D = M::D;
  if (c.tid >= M::GQA * D / 2) return;
  const int h = head0 + c.tid / (D / 2), d = 2 * (c.tid % (D / 2));
  const size_t row = (static_cast<size_t>(b) * M::NQ + h) * p.max_splits;
  const float* lse = p.attn_lse + row;
  const float* part = p.attn_partial + row * D + d;
  const uint8_t* valid = p.partial_valid ? p.partial_valid + row : nullptr;
  // Eight partials at a time (all eight reads in flight together; slots beyond n re-read the last
  // listed partial and get weight 0), folded into a running (max, numerators, denominator).
  constexpr int kGroup = 8;
  float mx = -INFINITY, num0 = 0.f, num1 = 0.f, den = 0.f;
  for (int base = 0; base < n; base += kGroup) {
    float e[kGroup];
    uint64_t two[kGroup];
    bool ok[kGroup];
#pragma unroll
    for (int i = 0; i < kGroup; ++i) {
      const int ii = min(base + i, n - 1);
      const int j = list ? list[ii] : ii;
      e[i] = ld_shared_f32(lse + j);
      two[i] = ld_shared64(part + static_cast<size_t>(j) * D);
      ok[i] = valid ? ld_shared8(valid + j) != 0 : true;
    }
    float gmx = mx;
#pragma unroll
    for (int i = 0; i < kGroup; ++i) {
      ok[i] = base + i < n && (valid ? ok[i] : (e[i] > kNoContribution && e[i] < INFINITY));
      if (ok[i]) gmx = fmaxf(gmx, e[i]);
    }
    const float keep = mx == -INFINITY ? 0.f : exp2_fast(mx - gmx);
    num0 *= keep, num1 *= keep, den *= keep;
    mx = gmx;
#pragma unroll
    for (int i = 0; i < kGroup; ++i) {
      const float f = ok[i] ? exp2_fast(e[i] - mx) : 0.f;
      num0 = __builtin_fmaf(__uint_as_float(static_cast<uint32_t>(two[i])), f, num0);
      num1 = __builtin_fmaf(__uint_as_float(static_cast<uint32_t>(two[i] >> 32)), f, num1);
      den += f;
    }
  }
  const bool any = den > 0.f;
  const float o0 = any ? num0 / den : 0.f, o1 = any ? num1 / den : 0.f;
  if (terminal) {
    st_shared32(p.attn_out + static_cast<size_t>(b) * M::NQ * D + static_cast<size_t>(h) * D + d,
                static_cast<uint32_t>(f2bf(o0)) | (static_cast<uint32_t>(f2bf(o1)) << 16));
  } else {
    float* dst = p.attn_partial + (row + out_slot) * D + d;
    st_shared_f32(dst, o0);
    st_shared_f32(dst + 1, o1);
    if (d == 0) {
      st_shared_f32(p.attn_lse + row + out_slot, any ? mx + log2f(den) : (valid ? 0.f : kNoContribution - 1.0f));
      if (p.partial_valid) st_shared8(p.partial_valid + row + out_slot, any ? 1 : 0);
    }
  }
}
// attn_out of the GQA heads from head0 of an inactive batch row.
template <class M>
__device__ __forceinline__ void zero_heads(const Params& p, const Ctx& c, int b, int head0) {
  if (c.tid < M::GQA * M::D / 2) st_shared32(p.attn_out + static_cast<size_t>(b) * M::NQ * M::D + head0 * M::D + 2 * c.tid, 0u);
}

// ===================================================================== 3 ==
// [3, layer, batch_row, kv_head, num_partials, partial_idx, seq_len, is_active, merge_in_last]
// Flash-decoding over one slice of one batch row's context for the GQA group of one KV head
// (python_vm.py:269-359).  seq_len < 0: the row's position + 1; is_active < 0: the row's flag.  The
// slices are whole KV blocks of `kv_block` tokens.  An inactive row or an empty slice leaves
// (0, -inf, not valid) and still counts.  Scoring as in the batch-1 kernel: a wave takes 16 tokens at
// a time on the matrix cores and keeps one running (max, sum, acc) per query head.
// merge_in_last (an extension; 0 in streams built by the reference scheduler): the workgroup whose
// arrival completes the head group's counters merges all partials itself (or zeroes the heads of an
// inactive row) and counts on the reduction row, so no reduction instruction and no second wait is needed.
template <class M>
__device__ bool op_splitkv(const Params& p, Smem<M>& s, const Ctx& c) {
  constexpr int D = M::D, GQA = M::GQA;
  static_assert(D % 64 == 0 && GQA <= 4 && GQA * D <= kThreads, "a lane owns whole 16-byte vectors of K; one thread per merged output");
  static_assert(M::AW == M::H, "the O-projection of this route reads an attention output as wide as the hidden state");
  const int layer = s.inst[1], b = s.inst[2], kvh = s.inst[3], P = s.inst[4], part = s.inst[5];
  if (layer < 0 || layer >= p.num_layers) return bad_operand(p, s, c, 1);
  if (b < 0 || b >= p.batch) return bad_operand(p, s, c, 2);
  if (kvh < 0 || kvh >= M::NKV) return bad_operand(p, s, c, 3);
  if (P < 1 || P > p.max_splits || part < 0 || part >= P) return bad_operand(p, s, c, 4);
  const int pos = s.pos[b];
  const int seq_len = s.inst[6] >= 0 ? s.inst[6] : pos + 1;
  if (seq_len > p.max_seq_len) return bad_operand(p, s, c, 6);
  const bool active = s.inst[7] == 0 ? false : (s.inst[7] == 1 ? true : s.active[b] != 0);
  const bool merge_in_last = s.inst[8] != 0;
  if (merge_in_last && P > kMaxList) return bad_operand(p, s, c, 8);
  const int lane = c.tid & 63, wave = c.tid >> 6;
  constexpr int kStride = M::NQ + 2 * M::NKV;   // counter slots per batch row

  const int total = max(1, (seq_len + p.kv_block - 1) / p.kv_block);
  const int per = max(1, (total + P - 1) / P);
  const int t0 = part * per * p.kv_block;
  const int t1 = min(min(part * per + per, total) * p.kv_block, seq_len);
  const bool empty = !active || t0 >= t1;
  const bool has_new = !empty && pos >= t0 && pos < t1;

  constexpr int KV16 = D / 32, NT = D / 16, kTok = 16, kStep = kWaves * kTok;
  const int c16 = lane & 15, g4 = lane >> 4;
  const size_t tok_stride = static_cast<size_t>(M::NKV) * D;
  const size_t row_of_kvh = (static_cast<size_t>(layer) * p.batch + b) * p.max_seq_len * tok_stride + static_cast<size_t>(kvh) * D;
  const u16* kbase = p.k_cache + row_of_kvh + g4 * (D / 4);
  const u16* vbase = p.v_cache + row_of_kvh + c16 * NT;
  struct Tile {
    v4u k[KV16];
    uint32_t v[4][NT / 2];
  };
  // Rows of earlier positions do not depend on this step; tokens past the slice are fetched from
  // its last row and masked when scored.
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
  // A wave's next kDepth tiles are in flight at any time, the first of them from before the wait below: a tile
  // costs a trip to memory and 16 tokens of arithmetic, so with one tile ahead every round paid most of the trip.
  constexpr int kDepth = 2;   // (4 and 8 measured 0.2 % and 0.4 % slower)
  int tb = t0 + wave * kTok;
  Tile ring[kDepth];
  static_for<0, kDepth>([&](auto i) {
#pragma unroll
    for (int j = 0; j < KV16; ++j) ring[i].k[j] = v4u{0, 0, 0, 0};
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int e = 0; e < NT / 2; ++e) ring[i].v[j][e] = 0;
    if (!empty && tb + i * kStep < t1) fetch(ring[i], tb + i * kStep);
  });

  if (!wait_counters(
          p, s, c, GQA + 2,
          [&](int i) {
            const int slot = i < GQA ? kvh * GQA + i : (i == GQA ? M::NQ + kvh : M::NQ + M::NKV + kvh);
            return counter_ptr(p, layer, ROW_QKV, apart(p, slot));
          },
          [&](int) { return D / kTile; }))
    return false;

  const int head0 = kvh * GQA;
  float* lse_out = p.attn_lse + (static_cast<size_t>(b) * M::NQ + head0) * p.max_splits + part;
  float* part_out = p.attn_partial + ((static_cast<size_t>(b) * M::NQ + head0) * p.max_splits + part) * D;
  uint8_t* valid_out = p.partial_valid ? p.partial_valid + (static_cast<size_t>(b) * M::NQ + head0) * p.max_splits + part : nullptr;
  auto arrive = [&] {
    release_stores();
    __syncthreads();
    if (!merge_in_last) {
      if (c.tid < GQA) publish(counter_ptr(p, layer, ROW_SPLITKV, b * kStride + head0 + c.tid), 1);
      return;
    }
    if (c.tid < GQA) {   // whoever sees P-1 earlier arrivals is last: every partial of the group is in memory
      const int prev = __hip_atomic_fetch_add(counter_ptr(p, layer, ROW_SPLITKV, b * kStride + head0 + c.tid), 1, __ATOMIC_RELAXED,
                                              __HIP_MEMORY_SCOPE_AGENT);
      if (c.tid == 0) s.ctl[3] = (prev == P - 1);
    }
    __syncthreads();
    if (s.ctl[3]) {  // uniform
      // the row's flag, not this slice's: an empty slice of a live row may well arrive last
      if (s.active[b]) merge_heads<M>(p, c, b, head0, P, nullptr, true, 0);
      else zero_heads<M>(p, c, b, head0);
      publish_after_stores(p, c, layer, ROW_REDUCE, apart(p, b), GQA);
    }
  };
  const bool alone = merge_in_last && P == 1 && !empty;
  if (empty) {  // uniform
    if (c.tid < GQA * D) {
      const int h = c.tid / D, d = c.tid % D;
      st_shared_f32(part_out + static_cast<size_t>(h) * p.max_splits * D + d, 0.f);
      if (d == 0) {
        st_shared_f32(lse_out + static_cast<size_t>(h) * p.max_splits, -INFINITY);
        if (valid_out) st_shared8(valid_out + static_cast<size_t>(h) * p.max_splits, 0);
      }
    }
    arrive();
    return true;
  }

  // q of the GQA group and, if the slice holds it, the K/V row this launch appended: bf16 in LDS.
  u16* stage16 = s.stage;
  constexpr int kQ = 0, kK = GQA * D, kV = GQA * D + D;
  {
    const size_t new_row = row_of_kvh + static_cast<size_t>(pos) * tok_stride;
    constexpr int kQChunks = GQA * D / 8, kRowChunks = D / 8;
    const int tid = c.tid;
    if constexpr (M::QK_NORM) {
      // Qwen3 op set (qwen3__0_6b/…/fused/operations.py:52-120): the raw vectors are staged; then one wave per
      // vector applies the per-head RMSNorm and RoPE in place (every lane one rotation pair), and the workgroup
      // whose slice holds the row's position also writes q_post_rope and the cache row.
      static_assert(D == 2 * kWaveSize && GQA + 2 <= kWaves, "one wave per vector, one rotation pair per lane");
      const u16* raw = p.qkv_raw + static_cast<size_t>(b) * M::QKV;
      if (tid < kQChunks) {
        reinterpret_cast<v4u*>(stage16 + kQ)[tid] = ld_shared128(raw + head0 * D + tid * 8);
      } else if (tid < kQChunks + kRowChunks && has_new) {
        reinterpret_cast<v4u*>(stage16 + kK)[tid - kQChunks] = ld_shared128(raw + (M::NQ + kvh) * D + (tid - kQChunks) * 8);
      } else if (tid < kQChunks + 2 * kRowChunks && has_new) {
        reinterpret_cast<v4u*>(stage16 + kV)[tid - kQChunks - kRowChunks] =
            ld_shared128(raw + (M::NQ + M::NKV + kvh) * D + (tid - kQChunks - kRowChunks) * 8);
      }
      __syncthreads();
      uint32_t* words = reinterpret_cast<uint32_t*>(stage16);
      if (wave <= GQA && (wave < GQA || has_new)) {
        const bool is_k = wave == GQA;
        const int at = is_k ? kK / 2 : (kQ + wave * D) / 2;
        const uint32_t rw = words[at + lane];
        const float x0 = bf_lo(rw), x1 = bf_hi(rw);
        const float ss = wave_sum(__builtin_fmaf(x1, x1, x0 * x0));
        const float rstd = 1.0f / sqrtf(ss / static_cast<float>(D) + p.rms_norm_eps);
        const uint32_t wn = reinterpret_cast<const uint32_t*>((is_k ? p.k_norm : p.q_norm) + static_cast<size_t>(layer) * D)[lane];
        const float n0 = round_bf16(bf_lo(wn) * (x0 * rstd)), n1 = round_bf16(bf_hi(wn) * (x1 * rstd));
        const uint32_t out = rope_pair(n0, n1, p.rope_cos + static_cast<size_t>(pos) * D, p.rope_sin + static_cast<size_t>(pos) * D, 2 * lane);
        words[at + lane] = out;
        if (has_new) {
          if (is_k) st_shared32(p.k_cache + new_row + 2 * lane, out);
          else st_shared32(p.q_post_rope + static_cast<size_t>(b) * M::NQ * D + (head0 + wave) * D + 2 * lane, out);
        }
      } else if (wave == GQA + 1 && has_new) {
        st_shared32(p.v_cache + new_row + 2 * lane, words[kV / 2 + lane]);
      }
    } else if (tid < kQChunks) {
      reinterpret_cast<v4u*>(stage16 + kQ)[tid] = ld_shared128(p.q_post_rope + static_cast<size_t>(b) * M::NQ * D + head0 * D + tid * 8);
    } else if (tid < kQChunks + kRowChunks && has_new) {
      reinterpret_cast<v4u*>(stage16 + kK)[tid - kQChunks] = ld_shared128(p.k_cache + new_row + (tid - kQChunks) * 8);
    } else if (tid < kQChunks + 2 * kRowChunks && has_new) {
      reinterpret_cast<v4u*>(stage16 + kV)[tid - kQChunks - kRowChunks] = ld_shared128(p.v_cache + new_row + (tid - kQChunks - kRowChunks) * 8);
    }
  }
  __syncthreads();

  typedef short bf4 __attribute__((ext_vector_type(4)));
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
  QMK_MB_STAMP(0);

  float m_run = -INFINITY, l_run = 0.f;
  f4 acc[NT];
#pragma unroll
  for (int i = 0; i < NT; ++i) acc[i] = f4{0.f, 0.f, 0.f, 0.f};

  auto round = [&](Tile& cur) {
    if (pos >= tb && pos < tb + kTok) {  // the row appended during this launch comes from LDS
      // (also where a token past the slice was redirected to this row: what the cache holds there is not defined yet)
      if (min(tb + c16, t1 - 1) == pos) {
#pragma unroll
        for (int j = 0; j < KV16; ++j) cur.k[j] = reinterpret_cast<const v4u*>(stage16 + kK + g4 * (D / 4))[j];
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        if (min(tb + 4 * g4 + j, t1 - 1) == pos) {
#pragma unroll
          for (int i = 0; i < NT / 2; ++i) cur.v[j][i] = reinterpret_cast<const uint32_t*>(stage16 + kV + c16 * NT)[i];
        }
      }
    }
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
    mt = fmaxf(mt, __shfl_xor(mt, 32));
    const float mn = fmaxf(m_run, mt);
    const float alpha = exp2_fast(m_run - mn);
    m_run = mn;
    float pr[4], psum = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      pr[i] = (c16 < GQA) ? exp2_fast(sc[i] - mn) : 0.f;
      psum += pr[i];
    }
    l_run = __builtin_fmaf(l_run, alpha, psum);
    // the weights as bf16 pairs hi + lo (lo = what the rounding of hi left): two conversions per pair
    const u2 hi = u2{pack_bf16(pr[0], pr[1]), pack_bf16(pr[2], pr[3])};
    const u2 lo = u2{pack_bf16(pr[0] - bf_lo(hi.x), pr[1] - bf_hi(hi.x)), pack_bf16(pr[2] - bf_lo(hi.y), pr[3] - bf_hi(hi.y))};
    const bf4 p_hi = __builtin_bit_cast(bf4, hi);
    const bf4 p_lo = __builtin_bit_cast(bf4, lo);
    float a_head[4];
    bool rescale = false;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      a_head[i] = i < GQA ? __int_as_float(__builtin_amdgcn_readlane(__float_as_int(alpha), i)) : 1.f;
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
    if (tb + kDepth * kStep < t1) fetch(cur, tb + kDepth * kStep);   // the tile that takes this one's place
    tb += kStep;
  };
  while (tb < t1) {
    static_for<0, kDepth>([&](auto i) {
      if (tb < t1) round(ring[i]);
    });
  }
  QMK_MB_STAMP(1);

  l_run += __shfl_xor(l_run, 16);
  l_run += __shfl_xor(l_run, 32);
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
  __syncthreads();
  if (c.tid < GQA * D) {
    const int h = c.tid / D, d = c.tid % D;
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
    const bool none = !(den > 0.f);
    st_shared_f32(part_out + static_cast<size_t>(h) * p.max_splits * D + d, none ? 0.f : num / den);
    // the only slice of its heads: what the merge of one partial leaves (weight 2^0, denominator 1) is the partial itself
    // (whole waves are here: GQA * D is a multiple of the wave size, and the even lane stores its neighbour's half too)
    const uint32_t half = f2bf(none ? 0.f : num / den);
    const uint32_t next = __shfl_down(half, 1);
    if (alone && !(d & 1)) st_shared32(p.attn_out + static_cast<size_t>(b) * M::NQ * D + static_cast<size_t>(head0 + h) * D + d, half | (next << 16));
    if (d == 0) {
      st_shared_f32(lse_out + static_cast<size_t>(h) * p.max_splits, none ? -INFINITY : mx + log2f(den));
      if (valid_out) st_shared8(valid_out + static_cast<size_t>(h) * p.max_splits, none ? 0 : 1);
    }
  }
  QMK_MB_STAMP(2);
  if (alone) {   // no trip for the count of arrivals, none to read the partial back
    release_stores();
    __syncthreads();
    if (c.tid < GQA) publish(counter_ptr(p, layer, ROW_SPLITKV, b * kStride + head0 + c.tid), 1);
    if (c.tid == 0) publish(counter_ptr(p, layer, ROW_REDUCE, apart(p, b)), GQA);
    return true;
  }
  arrive();
  return true;
}

// ===================================================================== 4 ==
// [4, layer, batch_row, head_start, num_partials, len, list..., is_terminal, output_partial, valid_partials, is_active]
// Log-sum-exp merge (log2 domain) of the listed partials of four query heads of one batch row,
// over the valid ones only (python_vm.py:442-551).  Thread t < GQA*D/2 produces two neighbouring dims.
template <class M>
__device__ bool op_reduce(const Params& p, Smem<M>& s, const Ctx& c) {
  constexpr int D = M::D, R = M::GQA;
  constexpr int kStride = M::NQ + 2 * M::NKV;
  const int layer = s.inst[1], b = s.inst[2], head0 = s.inst[3], P = s.inst[4], n = s.inst[5];
  if (layer < 0 || layer >= p.num_layers) return bad_operand(p, s, c, 1);
  if (b < 0 || b >= p.batch) return bad_operand(p, s, c, 2);
  if (head0 < 0 || head0 + R > M::NQ) return bad_operand(p, s, c, 3);
  if (n < 1 || n > kMaxList || P < 1) return bad_operand(p, s, c, 5);
  for (int i = 0; i < n; ++i)
    if (s.inst[6 + i] < 0 || s.inst[6 + i] >= p.max_splits) return bad_operand(p, s, c, 6 + i);
  const bool terminal = s.inst[6 + n] != 0;
  const int out_slot = s.inst[7 + n];
  if (!terminal && (out_slot < 0 || out_slot >= p.max_splits)) return bad_operand(p, s, c, 7 + n);
  const int flag = s.inst[9 + n];
  const bool active = flag == 0 ? false : (flag == 1 ? true : s.active[b] != 0);
  if (!active) {
    zero_heads<M>(p, c, b, head0);
    publish_after_stores(p, c, layer, ROW_REDUCE, apart(p, b), R);
    return true;
  }
  if (!wait_counters(p, s, c, R, [&](int i) { return counter_ptr(p, layer, ROW_SPLITKV, b * kStride + head0 + i); }, [&](int) { return P; }))
    return false;
  merge_heads<M>(p, c, b, head0, n, &s.inst[6], terminal, out_slot);
  publish_after_stores(p, c, layer, ROW_REDUCE, apart(p, b), R);
  return true;
}

// ===================================================================== 5 ==
// [5, layer, batch_size, tile_M, n_start, n_end, reduction_block, tile_M_g, tile_N_g]
// hidden[b, r] = bf16(hidden[b, r] + bf16(W_o[r] . attn_out[b])) for active rows   (python_vm.py:554-611)
template <class M>
__device__ bool op_oproj(const Params& p, Smem<M>& s, const Ctx& c) {
  const int layer = s.inst[1], B = s.inst[2], n0 = s.inst[4], n1 = s.inst[5];
  if (layer < 0 || layer >= p.num_layers) return bad_operand(p, s, c, 1);
  if (B != p.batch || s.inst[3] != 0) return bad_operand(p, s, c, 2);
  const int R = s.inst[8];   // rows per block: 16 (the reference's), or 8 (one block per workgroup on 256 CUs)
  if (s.inst[7] != kMaxBatch || (R != kTile && R != kTile / 2)) return bad_operand(p, s, c, 8);
  if (n0 < 0 || n1 < n0 || n1 > M::H / R) return bad_operand(p, s, c, 4);
  if (s.inst[6] != 0) return bad_operand(p, s, c, 6);
  const u16* w = p.o_w + static_cast<size_t>(layer) * M::H * M::H;
  // The residual pair this thread adds to in the first block is asked for together with the activations.
  u16* const mine = p.hidden + static_cast<size_t>(c.tid & 15) * M::H + 2 * (c.tid >> 4);
  const bool adds = c.tid < 8 * R && (c.tid & 15) < B && s.active[c.tid & 15];
  uint32_t old0 = 0;
  const bool ok = gemm_h<M, 1, 3>(
      p, s, c, n1 - n0, p.attn_out, B, [&](int j, int) { return w + static_cast<size_t>(n0 + j) * R * M::H; },
      [&] {
        if (!wait_counters(p, s, c, B, [&](int i) { return counter_ptr(p, layer, ROW_REDUCE, apart(p, i)); }, [&](int) { return M::NQ; })) return false;
        if (adds && n0 < n1) old0 = ld_shared32(mine + n0 * R);
        return true;
      },
      [&](int j, int parity, int b, int rp) {
        if (!adds) return;
        const float2 v = gather(s, parity, 0, b, rp);
        const uint32_t old = j == 0 ? old0 : ld_shared32(mine + (n0 + j) * R);
        st_shared32(mine + (n0 + j) * R, residual_add(old, v.x, v.y));
      },
      R);
  if (!ok) return false;
  publish_edge_after_stores(p, c, layer, ROW_OPROJ, n1 - n0);
  return true;
}

// ===================================================================== 7 ==
// [7, layer, batch_size, tile_M, len, blocks..., tile_M_g, tile_N_g]
// silu_out[b, r] = bf16(bf16(silu(bf16(W_g[r] . y_b))) * bf16(W_u[r] . y_b)), zero for inactive rows
// (python_vm.py:637-665; operations.py:265-282)
template <class M>
__device__ bool op_upgate(const Params& p, Smem<M>& s, const Ctx& c) {
  const int layer = s.inst[1], B = s.inst[2], n = s.inst[4];
  if (layer < 0 || layer >= p.num_layers) return bad_operand(p, s, c, 1);
  if (B != p.batch || s.inst[3] != 0) return bad_operand(p, s, c, 2);
  if (n < 0 || n > kInstWords - 7) return bad_operand(p, s, c, 4);
  for (int i = 0; i < n; ++i)
    if (s.inst[5 + i] < 0 || s.inst[5 + i] >= M::F / kTile) return bad_operand(p, s, c, 5 + i);
  if (s.inst[5 + n] != kMaxBatch || s.inst[6 + n] != kTile) return bad_operand(p, s, c, 6 + n);
  const u16* wg = p.gate_w + static_cast<size_t>(layer) * M::F * M::H;
  const u16* wu = p.up_w + static_cast<size_t>(layer) * M::F * M::H;
  const bool ok = gemm_h<M, 2, 2, true>(
      p, s, c, n, p.mlp_rms_out, B, [&](int j, int u) { return (u ? wu : wg) + static_cast<size_t>(s.inst[5 + j]) * kTile * M::H; },
      [&] { return wait_rows_done(p, s, c, layer, ROW_MLP_RMS, B); },
      [&](int j, int parity, int b, int rp) {
        if (b >= B) return;
        uint32_t word = 0;
        if (s.active[b]) {
          const float2 g = gather(s, parity, 0, b, rp), u = gather(s, parity, 1, b, rp);
          const uint32_t gb = pack_bf16(g.x, g.y), ub = pack_bf16(u.x, u.y);
          const float g0 = bf_lo(gb), g1 = bf_hi(gb);
          const uint32_t ab = pack_bf16(g0 / (1.0f + expf(-g0)), g1 / (1.0f + expf(-g1)));
          word = pack_bf16(bf_lo(ab) * bf_lo(ub), bf_hi(ab) * bf_hi(ub));
        }
        st_shared32(p.silu_out + static_cast<size_t>(b) * M::F + s.inst[5 + j] * kTile + 2 * rp, word);
      });
  if (!ok) return false;
  publish_edge_after_stores(p, c, layer, ROW_UPGATE, n);
  return true;
}

// The down projection of a 16-row block for at most 8 batch rows.  With 8 batch rows half of the tile's
// columns are empty, and so is half of every activation register: here a tile is 8 weight rows x 8 batch rows, twice —
// lanes m < 8 of the A operand hold rows 0..7 of one 32-column chunk, lanes m >= 8 the same rows of the NEXT chunk, and
// the B operand's columns n < 8 / n >= 8 hold the batch rows' shares of those two chunks: C[m][n] is then the first
// chunk's product for m, n < 8, the second's for m, n >= 8 (the other two quadrants mix chunks and are dropped), and
// an output is the sum of the two.  A register set covers 8 rows x 512 columns instead of 16 x 256 (F = 8192; 8 x 384
// for F = 6144): a wave's columns of both 8-row halves are four weight sets as before, but ALL of its activations are
// two sets, which fit beside three (F = 6144: all four) of them — one round of activation loads behind the wait instead
// of two dependent ones.  Weight loads take 128 contiguous bytes of 8 rows per instruction (64 bytes of 16 before).
template <class M>
__device__ __forceinline__ bool op_down_packed(const Params& p, Smem<M>& s, const Ctx& c, int layer, int B, int n0, int n1) {
  constexpr int kPair = 2 * kChunk;                      // columns of a chunk pair
  constexpr int NP = M::F / (kWaves * 2 * kPair);        // chunk pairs of a set: 8 (F = 8192: 512 columns), 6 (F = 6144: 384)
  constexpr int kSetCols = NP * kPair;
  static_assert(M::F == kWaves * 2 * kSetCols && NP <= kSegChunks, "a wave owns two sets of each half");
  // Four weight sets of 8 pairs and the activations do not fit the registers: the fourth waits in LDS; four of 6 do.
  constexpr bool kPark = NP == kSegChunks;
  struct Set {
    v4u a[NP];
  };
  const int lane = c.tid & 63, wave = c.tid >> 6;
  const u16* w = p.down_w + static_cast<size_t>(layer) * M::H * M::F;
  const int k0 = wave * 2 * kSetCols;
  const int sub = (lane >> 3) & 1, g = lane >> 4;   // which chunk of the pair, which 8 columns of it
  const size_t lane_off = static_cast<size_t>(lane & 7) * M::F + k0 + sub * kChunk + g * 8;
  auto load_set = [&](Set& sg, const u16* at) {
#pragma unroll
    for (int j = 0; j < NP; ++j) {
      // whole 128-byte lines per instruction: the streaming hint pays here (+0.4 %), unlike on the 64-byte pieces of load_seg
      sg.a[j] = __builtin_nontemporal_load(reinterpret_cast<const v4u*>(at + j * kPair));
    }
  };
  auto mma_set = [&](const Set& sg, const v4u (&x)[NP], f4 acc) {
#pragma unroll
    for (int j = 0; j < NP; ++j)
      acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, sg.a[j]), __builtin_bit_cast(bf16x8, x[j]), acc, 0, 0, 0);
    return acc;
  };
  // set q of a block: half q >> 1 (rows 8 * half ..), columns k0 + kSetCols * (q & 1) ..
  auto wptr = [&](int block, int q) { return w + (static_cast<size_t>(block) * kTile + 8 * (q >> 1)) * M::F + lane_off + (q & 1) * kSetCols; };
  Set a0, a1, a2, a3;
  auto request = [&](int block) {
    load_set(a0, wptr(block, 0));
    load_set(a1, wptr(block, 1));
    load_set(a2, wptr(block, 2));
    if constexpr (!kPark) load_set(a3, wptr(block, 3));
  };
  if (n0 < n1) {
    request(n0);
    if constexpr (kPark) {
      load_set(a3, wptr(n0, 3));
#pragma unroll
      for (int j = 0; j < NP; ++j) s.seg_park[wave][j][lane] = a3.a[j];
    }
  }
  if (!wait_edge(p, s, c, layer, ROW_UPGATE, M::F / kTile)) return false;
  u16* const mine = p.hidden + static_cast<size_t>(c.tid & 15) * M::H + 2 * (c.tid >> 4);
  const bool adds = c.tid < 8 * kTile && (c.tid & 15) < B && s.active[c.tid & 15];
  // this lane's share of silu_out: batch row l % 8, the chunk of the pair its weight lanes hold
  v4u xa[NP], xb[NP];
  {
    u16* base = p.silu_out;
    asm volatile("" : "+s"(base));
    const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(base, 0, 0x7fffffff, 0x00020000);
    // (a lane beyond the batch reads row 0 again: its column of the tile is finite and nobody looks at it)
    const uint32_t row = (lane & 7) < B ? static_cast<uint32_t>(lane & 7) : 0u;
    const uint32_t at = (row * M::F + k0 + sub * kChunk + g * 8) * 2;
#pragma unroll
    for (int j = 0; j < NP; ++j) {
      xa[j] = __builtin_bit_cast(v4u, __builtin_amdgcn_raw_buffer_load_b128(rsrc, at + j * kPair * 2, 0, 16));
      xb[j] = __builtin_bit_cast(v4u, __builtin_amdgcn_raw_buffer_load_b128(rsrc, at + (kSetCols + j * kPair) * 2, 0, 16));
    }
  }
  int parity = 0;
  for (int blk = n0; blk < n1; ++blk) {
    const uint32_t old = adds ? ld_shared32(mine + blk * kTile) : 0u;   // the pair this thread adds to, in time for the epilogue
    f4 lo = mma_set(a0, xa, f4{0.f, 0.f, 0.f, 0.f});   // rows 0..7
    f4 hi = mma_set(a2, xa, f4{0.f, 0.f, 0.f, 0.f});   // rows 8..15
    lo = mma_set(a1, xb, lo);
    if constexpr (kPark) {
      if (blk == n0) {
#pragma unroll
        for (int j = 0; j < NP; ++j) a3.a[j] = s.seg_park[wave][j][lane];
      } else {
        load_set(a3, wptr(blk, 3));
      }
    }
    hi = mma_set(a3, xb, hi);
    park(s, parity, 0, wave, lane, lo);
    park(s, parity, 1, wave, lane, hi);
    QMK_MB_STAMP(0);
    if (blk + 1 < n1) request(blk + 1);
    __syncthreads();
    QMK_MB_STAMP(1);
    if (adds) {
      // outputs (2 rp, 2 rp + 1) of the block for batch row b: half rp / 4, the two quadrants of every wave's tile
      const int b = c.tid & 15, rp = c.tid >> 4, half = rp >> 2, r = 2 * (rp & 3);
      float2 v = float2{0.f, 0.f};
#pragma unroll
      for (int wv = 0; wv < kWaves; ++wv) {
        const float2 t0 = *reinterpret_cast<const float2*>(&s.part[parity][half][wv][b][r]);
        const float2 t1 = *reinterpret_cast<const float2*>(&s.part[parity][half][wv][b + 8][r + 8]);
        v.x += t0.x + t1.x;
        v.y += t0.y + t1.y;
      }
      st_shared32(mine + blk * kTile, residual_add(old, v.x, v.y));
    }
    QMK_MB_STAMP(2);
    parity ^= 1;
  }
  publish_edge_after_stores(p, c, layer, ROW_DOWN, n1 - n0);
  return true;
}

// ===================================================================== 8 ==
// [8, layer, batch_size, tile_M, n_start, n_end, tile_M_g, tile_N_g]
// hidden[b, r] = bf16(hidden[b, r] + bf16(W_d[r] . silu_out[b])) for active rows, the whole K in
// one instruction (python_vm.py:554-611).  A wave owns F/8 columns: F/2048 segments per block (four for
// F = 8192, three for 6144); its share of silu_out follows the wait, two segments at a time.
template <class M>
__device__ bool op_down(const Params& p, Smem<M>& s, const Ctx& c) {
  constexpr int NS = M::F / (kWaves * kSeg);   // segments per wave and block
  static_assert(M::F % (kWaves * kSeg) == 0, "whole segments");
  const int layer = s.inst[1], B = s.inst[2], n0 = s.inst[4], n1 = s.inst[5];
  if (layer < 0 || layer >= p.num_layers) return bad_operand(p, s, c, 1);
  if (B != p.batch || s.inst[3] != 0) return bad_operand(p, s, c, 2);
  const int R = s.inst[7];   // rows per block: 16 (the reference's), or 8 (one block per workgroup on 256 CUs)
  if (s.inst[6] != kMaxBatch || (R != kTile && R != kTile / 2)) return bad_operand(p, s, c, 7);
  if (n0 < 0 || n1 < n0 || n1 > M::H / R) return bad_operand(p, s, c, 4);
  // at most 8 batch rows: half-tiles, all activations in one round (Llama shape, 8 rows: +1.4 %)
  if (B <= kMaxBatch / 2 && R == kTile) return op_down_packed<M>(p, s, c, layer, B, n0, n1);   // uniform
  const int lane = c.tid & 63, wave = c.tid >> 6;
  const u16* w = p.down_w + static_cast<size_t>(layer) * M::H * M::F;
  const int k0 = wave * NS * kSeg;
  const size_t lane_off = static_cast<size_t>(lane & (R - 1)) * M::F + k0 + (lane >> 4) * 8;
  static_assert(NS == 3 || NS == 4, "the segments below are handled by name");
  // Three weight segments of a block are requested before the wait and land during it; with four segments
  // the last follows the first activations (all four beside two activation segments do not fit the registers).
  Seg a0, a1, a2, a3;
  auto wptr = [&](int block, int q) { return w + static_cast<size_t>(block) * R * M::F + lane_off + q * kSeg; };
  auto request = [&](int block) {
    load_seg(a0, wptr(block, 0));
    load_seg(a1, wptr(block, 1));
    load_seg(a2, wptr(block, 2));
  };
  if (n0 < n1) {
    request(n0);
    if constexpr (NS == 4) {
      // The fourth segment of the first block goes to LDS through a3's registers: it lands during the wait instead of
      // behind the first activations (the registers hold three weight and two activation segments, not four and two).
      load_seg(a3, wptr(n0, 3));
#pragma unroll
      for (int j = 0; j < kSegChunks; ++j) s.seg_park[wave][j][lane] = a3.a[j];
    }
  }
  if (!wait_edge(p, s, c, layer, ROW_UPGATE, M::F / kTile)) return false;
  u16* const mine = p.hidden + static_cast<size_t>(c.tid & 15) * M::H + 2 * (c.tid >> 4);
  const bool adds = c.tid < 8 * R && (c.tid & 15) < B && s.active[c.tid & 15];
  int parity = 0;
  for (int blk = n0; blk < n1; ++blk) {
    f4 acc = f4{0.f, 0.f, 0.f, 0.f};
    uint32_t old = 0u;
    {
      v4u xa[kSegChunks], xb[kSegChunks];
      load_x(xa, p.silu_out, M::F, B, k0, lane);
      load_x(xb, p.silu_out, M::F, B, k0 + kSeg, lane);
      if constexpr (NS == 4) {
        if (blk != n0) load_seg(a3, wptr(blk, 3));
      }
      acc = mma_seg(a0, xa, acc);
      load_x(xa, p.silu_out, M::F, B, k0 + 2 * kSeg, lane);
      acc = mma_seg(a1, xb, acc);
      if constexpr (NS == 4) load_x(xb, p.silu_out, M::F, B, k0 + 3 * kSeg, lane);
      old = adds ? ld_shared32(mine + blk * R) : 0u;   // the pair this thread adds to, in time for the epilogue
      acc = mma_seg(a2, xa, acc);
      if constexpr (NS == 4) {
        if (blk == n0) {
#pragma unroll
          for (int j = 0; j < kSegChunks; ++j) a3.a[j] = s.seg_park[wave][j][lane];
        }
        acc = mma_seg(a3, xb, acc);
      }
    }
    park(s, parity, 0, wave, lane, acc);
    QMK_MB_STAMP(0);  // thread 0's weights and activations have all arrived
    if (blk + 1 < n1) request(blk + 1);
    __syncthreads();
    QMK_MB_STAMP(1);  // ... and everybody's
    if (adds) {
      const float2 v = gather(s, parity, 0, c.tid & 15, c.tid >> 4);
      st_shared32(mine + blk * R, residual_add(old, v.x, v.y));
    }
    QMK_MB_STAMP(2);
    parity ^= 1;
  }
  publish_edge_after_stores(p, c, layer, ROW_DOWN, n1 - n0);
  return true;
}

// The LM head for at most 8 batch rows on the half-tiles of op_down_packed: a 16-row block is two 8-row halves, a lane
// of the A operand holds rows 0..7 of one 32-column chunk (m < 8) or of the next (m >= 8), the B operand the batch rows'
// shares of the two chunks: 128 contiguous bytes of 8 rows per load instruction, half the activation registers.  With
// whole lines per instruction the weights can carry the streaming hint (8 rows: +0.8 %; the layout alone: -0.4 %).
template <class M>
__device__ __forceinline__ bool op_lmhead_packed(const Params& p, Smem<M>& s, const Ctx& c, int B, int n0, int n1) {
  constexpr int kPair = 2 * kChunk, NP = M::H / (kWaves * kPair), NB = 4;
  static_assert(M::H == kWaves * NP * kPair, "whole chunk pairs per wave");
  struct Half {
    v4u a[NP];
  };
  const int lane = c.tid & 63, wave = c.tid >> 6, n = n1 - n0;
  const int sub = (lane >> 3) & 1, g = lane >> 4;
  const int col = wave * NP * kPair + sub * kChunk + g * 8;
  const int last = p.vocab_size - 1;
  auto load_half = [&](Half& h, int j, int half) {   // rows past the vocabulary re-read its last row and are not stored
    const u16* at = p.lm_w + static_cast<size_t>(min((n0 + j) * kTile + 8 * half + (lane & 7), last)) * M::H + col;
#pragma unroll
    for (int q = 0; q < NP; ++q) {
      h.a[q] = __builtin_nontemporal_load(reinterpret_cast<const v4u*>(at + q * kPair));
    }
  };
  Half ring[NB][2];
#pragma unroll
  for (int k = 0; k < NB; ++k)
    if (k < n) {
      load_half(ring[k][0], k, 0);
      load_half(ring[k][1], k, 1);
    }
  if (!wait_rows_done(p, s, c, p.num_layers - 1, ROW_LM_RMS, B)) return false;
  v4u x[NP];
  {
    u16* base = p.lm_rms_out;
    asm volatile("" : "+s"(base));
    const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(base, 0, 0x7fffffff, 0x00020000);
    const uint32_t row = (lane & 7) < B ? static_cast<uint32_t>(lane & 7) : 0u;   // (a lane beyond the batch: row 0 again, unused)
    const uint32_t at = (row * M::H + col) * 2;
#pragma unroll
    for (int q = 0; q < NP; ++q) x[q] = __builtin_bit_cast(v4u, __builtin_amdgcn_raw_buffer_load_b128(rsrc, at + q * kPair * 2, 0, 16));
  }
  int parity = 0;
  for (int j0 = 0; j0 < n; j0 += NB) {
#pragma unroll
    for (int k = 0; k < NB; ++k) {
      const int j = j0 + k;
      if (j < n) {  // uniform over the workgroup
#pragma unroll
        for (int half = 0; half < 2; ++half) {
          f4 acc = f4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int q = 0; q < NP; ++q)
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, ring[k][half].a[q]), __builtin_bit_cast(bf16x8, x[q]), acc, 0, 0, 0);
          park(s, parity, half, wave, lane, acc);
          if (j + NB < n) load_half(ring[k][half], j + NB, half);
        }
        __syncthreads();
        if (c.tid < 8 * kTile && (c.tid & 15) < B) {
          const int b = c.tid & 15, rp = c.tid >> 4, half = rp >> 2, r = 2 * (rp & 3);
          float2 v = float2{-1e9f, -1e9f};
          if (s.active[b]) {
            v = float2{0.f, 0.f};
#pragma unroll
            for (int wv = 0; wv < kWaves; ++wv) {
              const float2 t0 = *reinterpret_cast<const float2*>(&s.part[parity][half][wv][b][r]);
              const float2 t1 = *reinterpret_cast<const float2*>(&s.part[parity][half][wv][b + 8][r + 8]);
              v.x += t0.x + t1.x;
              v.y += t0.y + t1.y;
            }
          }
          const int o = (n0 + j) * kTile + 2 * rp;
          u16* dst = p.logits + static_cast<size_t>(b) * p.vocab_size + o;
          if (o + 1 < p.vocab_size && (reinterpret_cast<uintptr_t>(dst) & 3) == 0) {
            st_shared32(dst, pack_bf16(v.x, v.y));
          } else {
            if (o < p.vocab_size) st_shared16(dst, f2bf(v.x));
            if (o + 1 < p.vocab_size) st_shared16(dst + 1, f2bf(v.y));
          }
        }
        parity ^= 1;
      }
    }
  }
  return true;
}

// ==================================================================== 10 ==
// [10, batch_size, start_block, end_block, tile_M_g, tile_N_g]
// logits[b, r] = bf16(W_lm[r] . lm_head_rms_out[b]); -1e9 for inactive rows   (python_vm.py:693-715)
template <class M>
__device__ bool op_lmhead(const Params& p, Smem<M>& s, const Ctx& c) {
  const int B = s.inst[1], n0 = s.inst[2], n1 = s.inst[3];
  if (B != p.batch) return bad_operand(p, s, c, 1);
  if (n0 < 0 || n1 < n0 || static_cast<long>(n1 - 1) * kTile >= p.vocab_size) return bad_operand(p, s, c, 3);
  if (s.inst[4] != kMaxBatch || s.inst[5] != kTile) return bad_operand(p, s, c, 5);
  if (B <= kMaxBatch / 2) return op_lmhead_packed<M>(p, s, c, B, n0, n1);   // uniform
  const int last = p.vocab_size - 1;
  const int lane_row = c.tid & 15;
  // The last block may be ragged: its missing rows re-read the last row and are not stored.
  return gemm_h<M, 1, 4>(
      p, s, c, n1 - n0, p.lm_rms_out, B,
      [&](int j, int) {
        const int r0 = (n0 + j) * kTile;
        return p.lm_w + static_cast<size_t>(min(r0 + lane_row, last) - lane_row) * M::H;
      },
      [&] { return wait_rows_done(p, s, c, p.num_layers - 1, ROW_LM_RMS, B); },
      [&](int j, int parity, int b, int rp) {
        if (b >= B) return;
        const int o = (n0 + j) * kTile + 2 * rp;
        const float2 v = s.active[b] ? gather(s, parity, 0, b, rp) : float2{-1e9f, -1e9f};
        u16* dst = p.logits + static_cast<size_t>(b) * p.vocab_size + o;
        if (o + 1 < p.vocab_size && (reinterpret_cast<uintptr_t>(dst) & 3) == 0) {
          st_shared32(dst, pack_bf16(v.x, v.y));
        } else {
          if (o < p.vocab_size) st_shared16(dst, f2bf(v.x));
          if (o + 1 < p.vocab_size) st_shared16(dst + 1, f2bf(v.y));
        }
      });
}

}  // namespace mb
}  // namespace qmk
