// Output pass of the bf16 matrix-core prefill for groups of four query heads per kv-head (K == V == D
// in {64, 128}, M == 64): same mathematics as mfma_out_kernel (prefill_mfma.hip; chunk algebra of
// nha_fla/ops/nha/chunk_fused.py:186-283, one softmax over [slots | window] as in
// nha_fla/ops/nha/chunk.py:459-470), different data movement and order.
//
//  * Every operand tile goes from global memory straight into LDS (global_load_lds_dwordx4, 1 KB
//    per wave instruction): no staging registers, no LDS stores, and the loads of the slot branch
//    are requested at the start and land while the window loop runs.
//  * The sliding window is walked first, in units of 32 keys through a ring of NR unit buffers; the
//    slot branch (which only needs the chunk-start states and the chunk's own rows) is folded into
//    the running softmax afterwards.
//  * The window loop is software-pipelined inside each wave: while the matrix core forms the scores
//    of unit u+1, the VALU exponentiates unit u.  The scale and the softmax reference are folded into
//    the score product itself (pre-scaled queries, accumulator started at -reference), so a score
//    needs one v_exp_f32 and half a v_cvt_pk_bf16_f32 and nothing else.
//  * The softmax reference of a query row is fixed once, from the first unit (the row's own and
//    nearest keys; 0 for rows that unit does not reach): fp32 sums relative to a fixed reference are
//    exact while every score stays within 2^+-100 of it, and the loop carries no maxima, no
//    comparisons and no rescaling of the accumulators.  A row whose window sum leaves that range
//    (overflowed, or below 2^-100) is flagged for mfma_repair_kernel, which recomputes it exactly.
//
// LDS layouts (no padding, which a 1 KB wave load cannot produce; the 16-byte pieces of a wave load may
// come from anywhere, so any order of pieces inside a 1 KB block is free): a 32-row unit is cut into
// 16-row x 32-column blocks of 1 KB.  "K layout" (row fragments, ds_read_b128): the 16-byte piece c of
// row r sits at 256 c + 16 r, which is exactly 16 x the number of the lane that reads it as its MFMA
// operand, so a wave reads a block as 1 KB of consecutive bytes (with 64-byte rows and the piece index
// XORed with (row / 4) % 4 a read took 12 LDS cycles instead of 4: SQ_LDS_BANK_CONFLICT 3.9e7 -> 5.1e6,
// SQ_LDS_IDX_ACTIVE 1.12e8 -> 7.8e7 cycles per launch at the T = 8192 shape).  "V layout" (transposing
// ds_read_b64_tr_b16, which takes 16 columns = 32 bytes of each of 16 rows per wave instruction): the
// block is two planes of 16 rows x 32 bytes, columns 0..15 then columns 16..31, so that the 512 bytes
// of one instruction are contiguous (with 64-byte rows: SQ_LDS_BANK_CONFLICT 9.8e7 -> 3.9e7).
#include "mfma_common.h"

#include <mutex>

namespace nha {
namespace {
using namespace mf;

typedef NHA_LDS unsigned char lbyte;
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

// nothing crosses: the instruction order of the loop is the source order
#define NHA_FENCE() __builtin_amdgcn_sched_barrier(0)
// keeps a value, and the arithmetic that made it, where the source has it
#define NHA_PIN(x) asm volatile("" : "+v"(x))

__device__ __forceinline__ unsigned cvt2(float a, float b) {
  bf16x2 t;
  t[0] = (__bf16)a;
  t[1] = (__bf16)b;
  return __builtin_bit_cast(unsigned, t);
}

// 16 bytes per lane from global memory into LDS at lds_base + 16 * lane (lds_base wave-uniform).
// Issued outside the compiler's memory model: every wait on these loads is written by hand.
__device__ __forceinline__ void g2l16(const void* gbase, uint32_t voff_bytes, uint32_t lds_base) {
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(voff_bytes), "s"(gbase), "s"(lds_base) : "memory");
}
template <int N>
__device__ __forceinline__ void wait_vm() {
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}
// 16 bytes per lane from global memory into registers, outside the compiler's memory model like the loads above: the
// wait the compiler writes for a load of its own does not know of the LDS-direct requests behind it and waits for
// all of them.  The value is there after wait_vm<N> with at most N younger requests pending; until then nothing may
// read or move the register, so its first use is claim_reg, placed behind that wait and a scheduling fence (a copy
// the register allocator makes for the claim then comes after the wait as well).
__device__ __forceinline__ u32x4 gload16(const void* ptr) {
  u32x4 x;
  asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(x) : "v"(ptr) : "memory");
  return x;
}
__device__ __forceinline__ void claim_reg(u32x4& x) { asm volatile("" : "+v"(x)::"memory"); }

template <int D>
struct RingCfg {
  static constexpr int KS = D / 32;            // 32-column blocks per row == contraction steps of q.k
  static constexpr int DB = D / 16;            // 16-row blocks of O^T
  static constexpr int UB = 32 * D * 2;        // bytes of a 32-row unit
  static constexpr int HB = UB / 2;            // bytes of its 16-row half
  static constexpr int NR = 512 / D;           // ring slots (64 KB of K and V units together)
  static constexpr int LPW = KS / 2;           // LDS-direct loads per wave for a unit (K and V) or a 64-row tile
  static constexpr int RING_K = 0, RING_V = NR * UB;
  static constexpr int TA = 2 * NR * UB;       // chunk-start k-state [m][d], K layout
  static constexpr int TB = TA + 2 * UB;       // k_gsa rows, K layout
  static constexpr int TC = TB + 2 * UB;       // chunk-start v-state [m][d], V layout
  static constexpr int TD = TC + 2 * UB;       // v rows, V layout
  static constexpr int GC = TD + 2 * UB;       // gate cumsum fp32 [64][64], pieces XORed with row % 16
  static constexpr int SS = GC + 16384;        // s bf16 [64][64], pieces XORed with row % 8
  static constexpr int BYTES = SS + 8192;
  static constexpr int ETAB = 0;               // decay tables (6 units of 4 KB), over the ring once the window is done
  static constexpr int NSLOT_LOADS = 4 * LPW + 3;   // per wave: four tiles, two gate blocks, one s block
  static constexpr int EGI = ETAB + 6 * 4096;  // exp(gc_i[m]) fp32 [64][64], laid out like GC
  static constexpr int EGR = EGI + 16384;      // exp(gc_i[m] - gr[m]) fp32 [64][64], gr = gate cumsum before the row's 16-row block
  static_assert(6 * 4096 + 2 * 16384 <= 2 * NR * UB, "decay tables must fit the ring");
};

// SINK: the window branch alone, with p.sinks zero-logit, zero-value keys in front of every sequence of which query t
// (position in its sequence) still sees clamp(p.wl - t, 0, p.sinks): the "full attention" layers of the hybrid models
// (nha_fla/models/qwen3_moe_nha/qwennha.py:323-336, :400-413).  No slot operands are requested, the slot branch and its
// tables are skipped, and the sinks join the denominator in the epilogue with the weight 2^(-reference) each.
template <int D, bool SINK = false>
__global__ __launch_bounds__(512, 1) void ring_out_kernel(const MP p) {
  using C = RingCfg<D>;
  constexpr int KS = C::KS, DB = C::DB, UB = C::UB, HB = C::HB, NR = C::NR, LPW = C::LPW;
  constexpr int RQB = 2;                        // 16-row query blocks per wave
  constexpr int NPRE = NR - 1;                  // units requested before the loop
  extern __shared__ __align__(1024) unsigned char smem_[];
  lbyte* const lds = (lbyte*)smem_;
  const uint32_t lds0 = (uint32_t)(uintptr_t)lds;
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l16 = lane & 15, kb = lane >> 4;
  const int H = p.H, HQ = p.HQ, NG = p.NG;
  // grid = (kv-head x group of four q-heads, chunk), chunks from the last to the first (prefill_mfma.hip)
  const int ngrp = NG / 4;
  int vx, vy;
  xcd_tile(ngrp, p.NT, vx, vy);   // with 8 (kv-head, group) pairs this is the launch order itself
  const int chunk = p.NT - 1 - vy;
  const int h = vx / ngrp, grp = vx % ngrp;
  const int hq = h * NG + grp * 4 + wave / 2;
  // rows 0..31 or 32..63 of the chunk: the later rows have more intra-chunk work in the slot branch, so the two
  // waves that share a SIMD (w and w + 4) take one half each
  const int qb0 = ((wave ^ (wave >> 2)) & 1) * RQB;
  const int n = p.cidx[2 * chunk], it = p.cidx[2 * chunk + 1];
  const int bos = p.cu[n], eos = p.cu[n + 1];
  const int c0 = bos + it * BT;
  const int rows = (eos - c0) < BT ? (eos - c0) : BT;
  const float cs = p.scale * LOG2E;
  const int64_t cg = (int64_t)chunk * H + h;

  // window units: unit u covers keys [c0 + 32 - 32 u, c0 + 64 - 32 u); c0 - bos is a multiple of 64, so no
  // unit starts before its sequence; units 0 and 1 are the chunk's own rows and may run past eos
  int lowest = bos;
  if (p.wl >= 0 && c0 - p.wl > bos) lowest = c0 - p.wl;
  const int nunits = (c0 + 64 - lowest + 31) / 32;   // >= 2

  // ---- load descriptors of this wave: LDS-direct load i of a unit / a 64-row tile ------------------
  // block index b = wave + 8 i; K layout: the lane's 16 bytes are piece lane / 16 of row lane % 16 of the block
  const int lrow16 = lane & 15, lswz = lane >> 4;
  // V layout: the lane's 16 bytes are piece lane % 2 of plane lane / 32, row (lane % 32) / 2
  const int lrowv = (lane & 31) >> 1, lpv = 2 * (lane >> 5) + (lane & 1);
  uint32_t u_off[LPW];          // byte offset from the unit's first row (token rows, stride H*D)
  uint32_t u_lds[LPW];          // LDS address of the block inside ring slot 0
  bool u_isv[LPW];
#pragma unroll
  for (int i = 0; i < LPW; ++i) {
    const int b = wave + 8 * i;
    const bool isv = b >= 2 * KS;
    const int bb = isv ? b - 2 * KS : b;
    const int rh = bb / KS, cq = bb % KS;
    u_isv[i] = isv;
    u_off[i] = ((uint32_t)(16 * rh + (isv ? lrowv : lrow16)) * (uint32_t)(H * D) + (uint32_t)(4 * cq + (isv ? lpv : lswz)) * 8) * 2;
    u_lds[i] = lds0 + (isv ? C::RING_V : C::RING_K) + rh * HB + cq * 1024;
  }
  // request unit u; rows past eos (units 0 and 1 only) are read from row eos - 1: always masked, always finite
  auto issue_unit_checked = [&](int u) {
    const int key0 = c0 + 32 - 32 * u;
    const int slot = u & (NR - 1);
#pragma unroll
    for (int i = 0; i < LPW; ++i) {
      const int b = wave + 8 * i;
      const bool isv = b >= 2 * KS;
      const int bb = isv ? b - 2 * KS : b;
      const int rh = bb / KS, cq = bb % KS;
      int row = key0 + 16 * rh + (isv ? lrowv : lrow16);
      row = row < eos ? row : eos - 1;
      const uint32_t off = ((uint32_t)(row - bos) * (uint32_t)(H * D) + (uint32_t)(4 * cq + (isv ? lpv : lswz)) * 8) * 2;
      const bf16_t* base = (isv ? p.v : p.k_swa) + ((int64_t)bos * H + h) * D;
      g2l16(base, off, u_lds[i] + slot * UB);
    }
  };
  // 64-row tile of the slot branch: kind 0 = K layout, 1 = V layout; rows of `src` with `stride` elements,
  // row r of the tile is global row rowmap(r)
  auto issue_tile = [&](int lds_tile, bool vlay, const bf16_t* src, uint32_t stride, auto rowmap) {
#pragma unroll
    for (int i = 0; i < LPW; ++i) {
      const int b = wave + 8 * i;            // < 4 KS
      const int unit = b / (2 * KS), bb = b % (2 * KS);
      const int rh = bb / KS, cq = bb % KS;
      const int r = 32 * unit + 16 * rh + (vlay ? lrowv : lrow16);
      const uint32_t off = ((uint32_t)rowmap(r) * stride + (uint32_t)(4 * cq + (vlay ? lpv : lswz)) * 8) * 2;
      g2l16(src, off, lds0 + lds_tile + unit * UB + rh * HB + cq * 1024);
    }
  };

  // ---- requests, in the order of their first use: the query fragments and unit 0 (first scores), then the other
  //      first units.  A CU serves the loads of its waves in the order they were issued: the barrier keeps the
  //      other units of the early waves from queueing in front of the last wave's queries and unit 0 ----
  u32x4 qraw[RQB][KS];
#pragma unroll
  for (int qb = 0; qb < RQB; ++qb) {
    // rows past the end of the sequence read its last row (the waits below count the loads) and are zeroed afterwards
    const int irow = 16 * (qb0 + qb) + l16;
    const bf16_t* qp = p.q_swa + ((int64_t)(c0 + (irow < rows ? irow : rows - 1)) * HQ + hq) * D + 8 * kb;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) qraw[qb][ks] = gload16(qp + 32 * ks);
  }
  issue_unit_checked(0);
  __builtin_amdgcn_s_barrier();
#pragma unroll
  for (int u = 1; u < NPRE; ++u)
    if (u < nunits) issue_unit_checked(u);
  // the queries and unit 0 have landed for this wave once no more than the units requested after them are in
  // flight (with a ring of four: one or two units; longer rings wait for everything)
  if constexpr (NR == 4) {
    if (nunits > 2) wait_vm<2 * LPW>();
    else wait_vm<LPW>();
  } else {
    wait_vm<0>();
  }
  NHA_FENCE();

  // window-query fragments, pre-scaled by scale * log2(e): scores come out of the matrix core in the
  // units the exponential wants
  bf16x8 qs[RQB][KS];
#pragma unroll
  for (int qb = 0; qb < RQB; ++qb) {
    const int irow = 16 * (qb0 + qb) + l16;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      claim_reg(qraw[qb][ks]);
      const u32x4 x = irow < rows ? qraw[qb][ks] : (u32x4){0u, 0u, 0u, 0u};
      const uint32_t w[4] = {x[0], x[1], x[2], x[3]};
      bf16x8 r;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float f = __uint_as_float((e & 1) ? (w[e >> 1] & 0xffff0000u) : (w[e >> 1] << 16));
        r[e] = (__bf16)(f * cs);
      }
      qs[qb][ks] = r;
    }
  }

  // ---- requests of the slot branch: made in the first loop iteration, they land while the window loop runs
  const int vlo = (p.shift - it * BT) < 0 ? 0 : (p.shift - it * BT);   // first row of the chunk whose source token exists
  auto issue_slot_operands = [&]() {
    const int grow_s = c0 - p.shift;   // source token of row 0
    auto tok = [&](int r) {            // source token of row r, kept inside the sequence (rows outside [vlo, rows) carry no weight)
      int t = grow_s + r;
      t = t < bos ? bos : t;
      t = t < eos ? t : eos - 1;
      return t - bos;
    };
    auto ident = [&](int r) { return r; };
    // in the order of their first use: the gate blocks (the decay tables are built from them), then the four tiles
    // gate cumsums: 16 blocks of 4 rows; rows >= `rows` were never written by the state pass and stay unused
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int b = wave + 8 * i;
      const int r = 4 * b + (lane >> 4);
      const int c = (lane & 15) ^ (r & 15);
      g2l16(p.gc + cg * BT * MS, (uint32_t)(r * MS + 4 * c) * 4, lds0 + C::GC + b * 1024);
    }
    {
      const int r = 8 * wave + (lane >> 3);
      const int c = (lane & 7) ^ (r & 7);
      g2l16(p.s + ((int64_t)bos * H + h) * MS, ((uint32_t)tok(r) * (uint32_t)(H * MS) + (uint32_t)c * 8) * 2, lds0 + C::SS + wave * 1024);
    }
    issue_tile(C::TA, false, p.hkT + cg * MS * D, (uint32_t)D, ident);
    issue_tile(C::TB, false, p.k_gsa + ((int64_t)bos * H + h) * D, (uint32_t)(H * D), tok);
    issue_tile(C::TC, true, p.hvc + cg * MS * D, (uint32_t)D, ident);
    issue_tile(C::TD, true, p.v + ((int64_t)bos * H + h) * D, (uint32_t)(H * D), tok);
  };

  // ---- window loop state ------------------------------------------------------------------------
  f32x4 O[DB][RQB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int qb = 0; qb < RQB; ++qb) O[db][qb] = (f32x4){0.f, 0.f, 0.f, 0.f};
  f32x4 Lw[RQB];
  float nm[RQB];     // minus the softmax reference of the row, log2 units
  f32x4 nmv[RQB];    // nm broadcast: the accumulator the score products start from
#pragma unroll
  for (int qb = 0; qb < RQB; ++qb) {
    Lw[qb] = (f32x4){0.f, 0.f, 0.f, 0.f};
    nm[qb] = 0.f;
    nmv[qb] = (f32x4){0.f, 0.f, 0.f, 0.f};
  }
  bf16x8 ones;
#pragma unroll
  for (int e = 0; e < 8; ++e) ones[e] = (__bf16)1.0f;
  // the reference is taken from unit 0 when a score there exceeds 2^THR, and kept from then on
  constexpr float THR = 8.f;

  const uint32_t kaddr = (uint32_t)(lane * 16);
  const uint32_t vaddr = (uint32_t)((4 * kb + (l16 >> 2)) * 32 + 8 * (l16 & 3));
  // row fragment (rows 16 kk + l16 of a unit, columns 32 ks + 8 kb ..) of a K-layout unit at byte address a
  auto kfrag = [&](uint32_t a, int kk, int ks) -> bf16x8 {
    return *reinterpret_cast<const NHA_LDS bf16x8*>(lds + a + kk * HB + ks * 1024);
  };
  // transposed fragment of a V-layout unit: X[4 kb + e][16 db + l16] (e < 4) and X[16 + 4 kb + e - 4][..]
  auto vfrag = [&](uint32_t a, int db) -> bf16x8 {
    const lbyte* pa = lds + a + (db >> 1) * 1024 + (db & 1) * 512;
    struct { s16x4 a, b; } t;
    t.a = __builtin_amdgcn_ds_read_tr16_b64_v4i16((NHA_LDS s16x4*)pa);
    t.b = __builtin_amdgcn_ds_read_tr16_b64_v4i16((NHA_LDS s16x4*)(pa + HB));
    return __builtin_bit_cast(bf16x8, t);
  };
  auto mask_unit = [&](f32x4 (&S)[2][RQB], int u) {
    const int xbase = 32 - 32 * u;
#pragma unroll
    for (int kk = 0; kk < 2; ++kk)
#pragma unroll
      for (int qb = 0; qb < RQB; ++qb) {
        const int y = 16 * (qb0 + qb) + l16;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int x = xbase + 16 * kk + 4 * kb + r;
          const bool ok = (x <= y) && (p.wl < 0 || x >= y - p.wl);
          if (!ok) S[kk][qb][r] = -INFINITY;
        }
      }
  };
  auto is_edge = [&](int u) -> bool { return (63 - 32 * u > 0) || (p.wl >= 0 && 32 - 32 * u < 63 - p.wl); };
  // the reference of column qb moves up by delta: everything accumulated so far shrinks by 2^-delta
  auto rescale_acc = [&](int qb, float delta) {
    const float alpha = fexp2(-delta);
    nm[qb] -= delta;
    nmv[qb] = (f32x4){nm[qb], nm[qb], nm[qb], nm[qb]};
#pragma unroll
    for (int r = 0; r < 4; ++r) Lw[qb][r] *= alpha;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int r = 0; r < 4; ++r) O[db][qb][r] *= alpha;
  };
  auto rescale = [&](f32x4 (&S)[2][RQB], const float (&rmax)[RQB]) {
#pragma unroll
    for (int qb = 0; qb < RQB; ++qb) {
      const float delta = fmaxf(max_over_rows(rmax[qb]), 0.f);
      rescale_acc(qb, delta);
#pragma unroll
      for (int kk = 0; kk < 2; ++kk)
#pragma unroll
        for (int r = 0; r < 4; ++r) S[kk][qb][r] -= delta;
    }
  };

  f32x4 Sc[2][RQB], Sn[2][RQB];
  bf16x8 kf[KS][2];
  bf16x8 vf[DB];
  // ---- prologue: scores of unit 0, K fragments of unit 1 -----------------------------------------------
  // unit 0 has landed for this wave (waited for above), then for everybody
  lds_barrier();
  {
    const uint32_t k0 = C::RING_K + kaddr;
#pragma unroll
    for (int kk = 0; kk < 2; ++kk)
#pragma unroll
      for (int qb = 0; qb < RQB; ++qb) Sc[kk][qb] = nmv[qb];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const bf16x8 a0 = kfrag(k0, 0, ks), a1 = kfrag(k0, 1, ks);
#pragma unroll
      for (int qb = 0; qb < RQB; ++qb) {
        Sc[0][qb] = mfma16(a0, qs[qb][ks], Sc[0][qb]);
        Sc[1][qb] = mfma16(a1, qs[qb][ks], Sc[1][qb]);
      }
    }
    mask_unit(Sc, 0);   // unit 0 is always an edge unit
    float rmax[RQB];
    bool need = false;
#pragma unroll
    for (int qb = 0; qb < RQB; ++qb) {
      float x = fmaxf(fmaxf(Sc[0][qb][0], Sc[0][qb][1]), fmaxf(Sc[0][qb][2], Sc[0][qb][3]));
      x = fmaxf(x, fmaxf(fmaxf(Sc[1][qb][0], Sc[1][qb][1]), fmaxf(Sc[1][qb][2], Sc[1][qb][3])));
      rmax[qb] = x;
      need |= x > THR;
    }
    if (__any(need)) rescale(Sc, rmax);
    // unit 1 has landed, for this wave and then for everybody (the last of the first units may still be in flight)
    if constexpr (NR == 4) {
      if (nunits > 2) wait_vm<LPW>();
      else wait_vm<0>();
      lds_barrier();
    }
    const uint32_t k1 = C::RING_K + (1 & (NR - 1)) * UB + kaddr;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      kf[ks][0] = kfrag(k1, 0, ks);
      kf[ks][1] = kfrag(k1, 1, ks);
    }
  }
  // global position of the next unit to request (unit NPRE at u = 0), 32 rows back per iteration
  const bf16_t* kreq = p.k_swa + (((int64_t)c0 + 32 - 32 * NPRE) * H + h) * D;
  const bf16_t* vreq = p.v + (((int64_t)c0 + 32 - 32 * NPRE) * H + h) * D;
  const int64_t ustep = (int64_t)32 * H * D;

  // slot-branch query fragments of one query block (requested while the last unit is worked on)
  auto load_qg = [&](bf16x8 (&q)[KS], int qb) {
    const int irow = 16 * (qb0 + qb) + l16;
    const bf16_t* qp = p.q_gsa + ((int64_t)(c0 + irow) * HQ + hq) * D + 8 * kb;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      uint4 x = make_uint4(0, 0, 0, 0);
      if (irow < rows) x = *reinterpret_cast<const uint4*>(qp + 32 * ks);
      q[ks] = as_bf16x8(x);
    }
  };
  // exponentials of the current unit's block for contraction step ks, element j (see phase A)
  auto exp_step = [&](int ks, int j) {
    if (KS == 4) {
      Sc[ks & 1][ks >> 1][j] = fexp2(Sc[ks & 1][ks >> 1][j]);
      NHA_PIN(Sc[ks & 1][ks >> 1][j]);
    } else {
      Sc[0][ks][j] = fexp2(Sc[0][ks][j]);
      NHA_PIN(Sc[0][ks][j]);
      Sc[1][ks][j] = fexp2(Sc[1][ks][j]);
      NHA_PIN(Sc[1][ks][j]);
    }
  };
  auto pack_p = [&](bf16x8 (&Pq)[RQB]) {
#pragma unroll
    for (int qb = 0; qb < RQB; ++qb) {
      const u32x4 t = {cvt2(Sc[0][qb][0], Sc[0][qb][1]), cvt2(Sc[0][qb][2], Sc[0][qb][3]), cvt2(Sc[1][qb][0], Sc[1][qb][1]),
                       cvt2(Sc[1][qb][2], Sc[1][qb][3])};
      Pq[qb] = __builtin_bit_cast(bf16x8, t);
      NHA_PIN(Pq[qb]);
    }
  };

  for (int u = 0; u + 1 < nunits; ++u) {
    const uint32_t k_nn = C::RING_K + ((u + 2) & (NR - 1)) * UB + kaddr;   // K of unit u+2 (after the barrier)
    const uint32_t v_c = C::RING_V + (u & (NR - 1)) * UB + vaddr;           // V of unit u
    // ---- phase A: scores of unit u+1 on the matrix core, exponentials of unit u on the VALU,
    //      V fragments of unit u requested from LDS ----
    NHA_FENCE();
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int kk = j & 1, qb = j >> 1;
        // DB / (4 KS) = 1/2 V fragment per score product
        if ((j & 1) == 0) vf[2 * ks + (j >> 1)] = vfrag(v_c, 2 * ks + (j >> 1));
        Sn[kk][qb] = mfma16(kf[ks][kk], qs[qb][ks], ks == 0 ? nmv[qb] : Sn[kk][qb]);
        // a score block of the current unit per contraction step: with KS = 4 block (ks & 1, ks >> 1),
        // with KS = 2 blocks (0, ks) and (1, ks)
        exp_step(ks, j);
        NHA_FENCE();
      }
    }
    bf16x8 Pq[RQB];
    pack_p(Pq);
    NHA_FENCE();
    // unit u+2 has landed (this wave's part), then everybody's; after the barrier the slot of unit u-1
    // is free and takes unit u+NPRE.  Requests younger than unit u+2 may stay in flight: units
    // u+3 .. u+NR-2, and the slot-branch operands while u <= NR-3 (queued behind unit NR-1 in iteration 0)
    if (u + 2 < nunits) {
      if (u + NR - 2 < nunits) {
        if (!SINK && u >= 1 && u <= NR - 3) wait_vm<LPW * (NR - 4) + C::NSLOT_LOADS>();
        else wait_vm<LPW * (NR - 4)>();
      } else {
        wait_vm<0>();
      }
    }
    lds_barrier();
    if (u + NPRE < nunits) {
      const int slot = (u + NPRE) & (NR - 1);
#pragma unroll
      for (int i = 0; i < LPW; ++i) g2l16(u_isv[i] ? vreq : kreq, u_off[i], u_lds[i] + slot * UB);
    }
    if (!SINK && u == 0) issue_slot_operands();
    kreq -= ustep;
    vreq -= ustep;
    NHA_FENCE();
    // ---- phase B: value products of unit u on the matrix core,
    //      K fragments of unit u+2 requested from LDS ----
#pragma unroll
    for (int qb = 0; qb < RQB; ++qb) {
      Lw[qb] = mfma16(ones, Pq[qb], Lw[qb]);
      NHA_FENCE();
    }
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      kf[db >> 1][db & 1] = kfrag(k_nn, db & 1, db >> 1);
      NHA_FENCE();
#pragma unroll
      for (int qb = 0; qb < RQB; ++qb) {
        O[db][qb] = mfma16(vf[db], Pq[qb], O[db][qb]);
        NHA_FENCE();
      }
    }
    if (is_edge(u + 1)) mask_unit(Sn, u + 1);
#pragma unroll
    for (int kk = 0; kk < 2; ++kk)
#pragma unroll
      for (int qb = 0; qb < RQB; ++qb) Sc[kk][qb] = Sn[kk][qb];
  }
  // ---- the last unit: no further scores; the slot-branch queries of the first query block are
  //      requested into the registers the window queries leave ----
  bf16x8 qg[KS];
  {
    const int u = nunits - 1;
    const uint32_t v_c = C::RING_V + (u & (NR - 1)) * UB + vaddr;
#pragma unroll
    for (int db = 0; db < DB; ++db) vf[db] = vfrag(v_c, db);
    if (!SINK) load_qg(qg, 0);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
#pragma unroll
      for (int j = 0; j < 4; ++j) exp_step(ks, j);
    bf16x8 Pq[RQB];
    pack_p(Pq);
#pragma unroll
    for (int qb = 0; qb < RQB; ++qb) Lw[qb] = mfma16(ones, Pq[qb], Lw[qb]);
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int qb = 0; qb < RQB; ++qb) O[db][qb] = mfma16(vf[db], Pq[qb], O[db][qb]);
  }

  // a window sum outside 2^+-100 of the fixed reference (overflowed sums are +inf: beyond the upper bound):
  // products with the values may have left fp32, or bf16 probabilities may have been flushed to zero
  // that matter against the sum; the exact pass redoes the rows of the sub-block
#pragma unroll
  for (int qb = 0; qb < RQB; ++qb) {
    const bool bad = (16 * (qb0 + qb) + l16 < rows) && (Lw[qb][0] >= 0x1p100f || Lw[qb][0] < 0x1p-100f);
    if (__any(bad) && lane == 0) atomicOr(p.flags + cg * 4, 1 << (qb0 + qb));
  }
  float lg[RQB];
  if constexpr (SINK) {
    // the sinks still in view: logit 0, i.e. 2^(0 - reference) each relative to the row's reference; value 0
#pragma unroll
    for (int qb = 0; qb < RQB; ++qb) {
      const int irow = 16 * (qb0 + qb) + l16;
      int n0 = p.wl - (c0 - bos + irow);
      n0 = n0 < 0 ? 0 : (n0 > p.sinks ? p.sinks : n0);
      lg[qb] = (float)n0 * fexp2(nm[qb]);
      if (p.lse_swa && kb == 0 && irow < rows)
        p.lse_swa[(int64_t)(c0 + irow) * HQ + hq] = (__builtin_amdgcn_logf(Lw[qb][0] + lg[qb]) - nm[qb]) * LN2;
    }
  } else {
  // ================= slot branch, folded into the running softmax =================================
  // The gate blocks have landed and every wave is done with the ring.  With a window of at most NR units the slot
  // operands were the last requests (the tiles the last of all): the decay tables are built while the tiles are
  // still on their way.  Longer windows requested units after them, and the loop has waited for those.
  if (nunits <= NR) wait_vm<4 * LPW>();
  else wait_vm<0>();
  lds_barrier();
  auto gc_at = [&](int j, int m) -> const lfloat* { return (const lfloat*)(lds + C::GC + j * 256 + (((m >> 2) ^ (j & 15)) * 16) + (m & 3) * 4); };
  auto s_at = [&](int j, int m) -> const lbf16* { return (const lbf16*)(lds + C::SS + j * 128 + (((m >> 3) ^ (j & 7)) * 16) + (m & 7) * 2); };
  // decay tables E_Q[j][m] = s_j[m] exp(min(gr_Q[m] - gc_j[m], DECAY_CLAMP)) for the rows j of the 16-row
  // blocks jb <= Q, zero elsewhere: query sub-block Q (16 rows) references the gate cumsum gr_Q of the
  // row before it (0 for Q = 0), so the exponent is <= 0 for rows of earlier blocks and bounded by the
  // block's own decay on the diagonal.  Rows whose source token does not exist (before the sequence,
  // past its end) carry no weight.  Stored as 32-row units in the V layout (64 columns): the logit
  // update reads them transposed (rows = slots), the slot-read weights row by row (rows = tokens).
  // Units: E_0 -> 0, E_1 -> 1, E_2 -> 2,3, E_3 -> 4,5; a thread makes 8 consecutive slots of a row.
  for (int item = tid; item < 6 * 256; item += 512) {
    const int U = item >> 8, r32 = (item >> 3) & 31, m = (item & 7) * 8;
    const int Q = U == 0 ? 0 : U == 1 ? 1 : U < 4 ? 2 : 3;
    const int pr = (U == 3 || U == 5) ? 1 : 0;
    const int j = 32 * pr + r32;
    const bool ok = (j >> 4) <= Q && j >= vlo && j < rows;
    bf16x8 out;
#pragma unroll
    for (int e = 0; e < 8; ++e) out[e] = (__bf16)0.f;
    if (ok) {
      f32x4 gv[2], gr[2];
#pragma unroll
      for (int hh = 0; hh < 2; ++hh) {
        gv[hh] = *reinterpret_cast<const NHA_LDS f32x4*>(gc_at(j, m + 4 * hh));
        gr[hh] = (f32x4){0.f, 0.f, 0.f, 0.f};
        if (Q > 0) gr[hh] = *reinterpret_cast<const NHA_LDS f32x4*>(gc_at(16 * Q - 1, m + 4 * hh));
      }
      const bf16x8 sv = *reinterpret_cast<const NHA_LDS bf16x8*>(s_at(j, m));
#pragma unroll
      for (int e = 0; e < 8; ++e) out[e] = (__bf16)((float)sv[e] * fexp(fminf(gr[e >> 2][e & 3] - gv[e >> 2][e & 3], DECAY_CLAMP)));
    }
    *reinterpret_cast<NHA_LDS bf16x8*>(lds + C::ETAB + U * 4096 + (r32 >> 4) * 2048 + (m >> 5) * 1024 + ((m >> 4) & 1) * 512 + (r32 & 15) * 32 + (m & 15) * 2) = out;
  }
  // exp(gc_i[m]) and exp(gc_i[m] - gr[m]) of the chunk's rows: the same for the four query heads of the
  // workgroup, so they are formed once here instead of by every wave for its own rows
  for (int item = tid; item < 64 * 16; item += 512) {
    const int j = item >> 4, m = 4 * (item & 15);
    const f32x4 gi = *reinterpret_cast<const NHA_LDS f32x4*>(gc_at(j, m));
    f32x4 gr4 = (f32x4){0.f, 0.f, 0.f, 0.f};
    if (j >= 16) gr4 = *reinterpret_cast<const NHA_LDS f32x4*>(gc_at((j & ~15) - 1, m));
    f32x4 ei, er;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      ei[r] = fexp(gi[r]);
      er[r] = fexp(gi[r] - gr4[r]);
    }
    const uint32_t off = (uint32_t)(j * 256 + (((m >> 2) ^ (j & 15)) * 16));
    *reinterpret_cast<NHA_LDS f32x4*>(lds + C::EGI + off) = ei;
    *reinterpret_cast<NHA_LDS f32x4*>(lds + C::EGR + off) = er;
  }
  wait_vm<0>();   // the four tiles
  __syncthreads();

  // E_Q transposed: rows = slots 16 mb + l16, contraction over the tokens 32 pr + {4 kb + e, 16 + 4 kb + e - 4}
  auto etab_tr = [&](int Q, int pr, int mb) -> bf16x8 {
    const lbyte* pa = lds + C::ETAB + ((Q < 2 ? Q : 2 * Q - 2) + pr) * 4096 + (mb >> 1) * 1024 + (mb & 1) * 512 + vaddr;
    struct { s16x4 a, b; } t;
    t.a = __builtin_amdgcn_ds_read_tr16_b64_v4i16((NHA_LDS s16x4*)pa);
    t.b = __builtin_amdgcn_ds_read_tr16_b64_v4i16((NHA_LDS s16x4*)(pa + 2048));
    return __builtin_bit_cast(bf16x8, t);
  };
  // E_Q by rows: row = token 16 jb + l16, contraction over the slots 32 pr + {4 kb + e, 16 + 4 kb + e - 4}
  auto etab_row = [&](int Q, int jb, int pr) -> bf16x8 {
    const lbyte* pa = lds + C::ETAB + ((Q < 2 ? Q : 2 * Q - 2) + (jb >> 1)) * 4096 + (jb & 1) * 2048 + pr * 1024 + l16 * 32 + 8 * kb;
    struct { bf16x4 a, b; } t;
    t.a = *reinterpret_cast<const NHA_LDS bf16x4*>(pa);
    t.b = *reinterpret_cast<const NHA_LDS bf16x4*>(pa + 512);
    return __builtin_bit_cast(bf16x8, t);
  };
  // No barrier holds the two waves of a SIMD together from here on, and the older one (w < 4) is served
  // first: left alone it ends about 5 k cycles before the younger, which then has the SIMD to itself.  The
  // younger wave gets the higher priority for the first of the two query blocks, so that both end together.
  if (wave >= 4) __builtin_amdgcn_s_setprio(1);
#pragma unroll
  for (int qb = 0; qb < RQB; ++qb) {
    if (qb == RQB - 1) __builtin_amdgcn_s_setprio(0);
    const int Q = qb0 + qb;                // sub-block index inside the chunk
    const int irow = 16 * Q + l16;         // this lane's query row inside the chunk
    // the window's own log-sum-exp, taken before the slots join: afterwards the window sum is only known
    // relative to the joint maximum and underflows when the slot logits top the window's by 2^126
    if (p.lse_swa && kb == 0 && irow < rows) p.lse_swa[(int64_t)(c0 + irow) * HQ + hq] = (__builtin_amdgcn_logf(Lw[qb][0]) - nm[qb]) * LN2;
    // inter-chunk slot logits: okT[m][i] = sum_d hkT[m][d] q[i][d]
    f32x4 ok[4];
#pragma unroll
    for (int mb = 0; mb < 4; ++mb) ok[mb] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
#pragma unroll
      for (int mb = 0; mb < 4; ++mb) ok[mb] = mfma16(kfrag(C::TA + (mb >> 1) * UB + kaddr, mb & 1, ks), qg[ks], ok[mb]);
    // intra-chunk scores AT[j][i] = sum_d k_gsa[j][d] q[i][d] for row blocks jb <= Q, masked j <= i
    bf16x8 bA[2];
    {
      f32x4 at[4];
#pragma unroll
      for (int jb = 0; jb < 4; ++jb) at[jb] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
#pragma unroll
        for (int jb = 0; jb < 4; ++jb)
          if (jb <= Q) at[jb] = mfma16(kfrag(C::TB + (jb >> 1) * UB + kaddr, jb & 1, ks), qg[ks], at[jb]);
#pragma unroll
      for (int jb = 0; jb < 4; ++jb)
        if (jb == Q) {
#pragma unroll
          for (int r = 0; r < 4; ++r)
            if (4 * kb + r > l16) at[jb][r] = 0.f;
        }
      bA[0] = pack8(at[0], at[1]);
      bA[1] = pack8(at[2], at[3]);
    }
    if (qb + 1 < RQB) load_qg(qg, qb + 1);
    // okT_intra[m][i] = sum_j s_j[m] exp(gr[m] - gc_j[m]) AT[j][i]
    f32x4 oki[4];
#pragma unroll
    for (int mb = 0; mb < 4; ++mb) {
      oki[mb] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int pr = 0; pr < 2; ++pr)
        if (2 * pr <= Q) {
          oki[mb] = mfma16(etab_tr(Q, pr, mb), bA[pr], oki[mb]);
        }
    }
    // combine; the slot logits join the running softmax as one more set of keys
    f32x4 egi[4], egr[4];   // exp(gc_i[m]) and exp(gc_i[m] - gr[m]) in accumulator layout
    float xmax = -INFINITY;
#pragma unroll
    for (int mb = 0; mb < 4; ++mb) {
      const uint32_t off = (uint32_t)(irow * 256 + (((4 * mb + kb) ^ (irow & 15)) * 16));
      egi[mb] = *reinterpret_cast<const NHA_LDS f32x4*>(lds + C::EGI + off);
      egr[mb] = *reinterpret_cast<const NHA_LDS f32x4*>(lds + C::EGR + off);
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        ok[mb][r] = (ok[mb][r] * egi[mb][r] + oki[mb][r] * egr[mb][r]) * cs;   // slot logit, log2 units
        xmax = fmaxf(xmax, ok[mb][r]);
      }
    }
    // relative to the reference of the window pass; the reference moves if a slot logit tops it by 2^THR
    if (__any(xmax + nm[qb] > THR)) {
      const float delta = fmaxf(max_over_rows(xmax) + nm[qb], 0.f);
      rescale_acc(qb, delta);
    }
    float psum = 0.f;
    f32x4 sl[4];
#pragma unroll
    for (int mb = 0; mb < 4; ++mb) sl[mb] = ok[mb];
#pragma unroll
    for (int mb = 0; mb < 4; ++mb)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        ok[mb][r] = fexp2(ok[mb][r] + nm[qb]);   // unnormalised slot probabilities
        psum += ok[mb][r];
      }
    psum += __shfl_xor(psum, 16, 64);
    psum += __shfl_xor(psum, 32, 64);
    lg[qb] = psum;
    if (p.lse_gsa) {
      // the slots' own log-sum-exp, relative to their own maximum (log2 units; logits were saved in `sl`)
      const float ms = max_over_rows(xmax);
      float pown = 0.f;
#pragma unroll
      for (int mb = 0; mb < 4; ++mb)
#pragma unroll
        for (int r = 0; r < 4; ++r) pown += fexp2(sl[mb][r] - ms);
      pown += __shfl_xor(pown, 16, 64);
      pown += __shfl_xor(pown, 32, 64);
      if (kb == 0 && irow < rows) p.lse_gsa[(int64_t)(c0 + irow) * HQ + hq] = (__builtin_amdgcn_logf(pown) + ms) * LN2;
    }
    bf16x8 bp[2], bpr[2];   // slot probabilities x exp(gc_i) and x exp(gc_i - gr), B operands
#pragma unroll
    for (int pr = 0; pr < 2; ++pr) {
      f32x4 x0, x1, y0, y1;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        x0[r] = ok[2 * pr][r] * egi[2 * pr][r];
        x1[r] = ok[2 * pr + 1][r] * egi[2 * pr + 1][r];
        y0[r] = ok[2 * pr][r] * egr[2 * pr][r];
        y1[r] = ok[2 * pr + 1][r] * egr[2 * pr + 1][r];
      }
      bp[pr] = pack8(x0, x1);
      bpr[pr] = pack8(y0, y1);
    }
    // slot read, inter-chunk part: O^T[d][i] += sum_m hv[m][d] (p[i][m] exp(gc_i[m]))
#pragma unroll
    for (int pr = 0; pr < 2; ++pr)
#pragma unroll
      for (int db = 0; db < DB; ++db) O[db][qb] = mfma16(vfrag(C::TC + pr * UB + vaddr, db), bp[pr], O[db][qb]);
    // intra-chunk part: AvT[j][i] = sum_m s_j[m] exp(gr[m]-gc_j[m]) (p[i][m] exp(gc_i[m]-gr[m])), j <= i
    bf16x8 bAv[2];
    {
      f32x4 av[4];
#pragma unroll
      for (int jb = 0; jb < 4; ++jb) {
        av[jb] = (f32x4){0.f, 0.f, 0.f, 0.f};
        if (jb <= Q) {
#pragma unroll
          for (int pr = 0; pr < 2; ++pr) {
            av[jb] = mfma16(etab_row(Q, jb, pr), bpr[pr], av[jb]);
          }
          if (jb == Q) {
#pragma unroll
            for (int r = 0; r < 4; ++r)
              if (4 * kb + r > l16) av[jb][r] = 0.f;
          }
        }
      }
      bAv[0] = pack8(av[0], av[1]);
      bAv[1] = pack8(av[2], av[3]);
    }
#pragma unroll
    for (int pr = 0; pr < 2; ++pr)
      if (2 * pr <= Q) {
#pragma unroll
        for (int db = 0; db < DB; ++db) O[db][qb] = mfma16(vfrag(C::TD + pr * UB + vaddr, db), bAv[pr], O[db][qb]);
      }
  }
  }   // !SINK

  // ---- epilogue: 16-byte stores (the lanes of an even 16-lane row keep block db, those of the odd
  //      row block db + 1, and the two trade their halves) -------------------------------------------
#pragma unroll
  for (int qb = 0; qb < RQB; ++qb) {
    const int irow = 16 * (qb0 + qb) + l16;
    const float lwt = Lw[qb][0];
    const float inv = 1.f / (lwt + lg[qb]);
    bf16_t* op = p.o + ((int64_t)(c0 + irow) * HQ + hq) * D;
#pragma unroll
    for (int db = 0; db < DB; db += 2) {
      unsigned a[2], b[2];
      a[0] = cvt2(O[db][qb][0] * inv, O[db][qb][1] * inv);
      a[1] = cvt2(O[db][qb][2] * inv, O[db][qb][3] * inv);
      b[0] = cvt2(O[db + 1][qb][0] * inv, O[db + 1][qb][1] * inv);
      b[1] = cvt2(O[db + 1][qb][2] * inv, O[db + 1][qb][3] * inv);
#pragma unroll
      for (int e = 0; e < 2; ++e) {
        const auto sw = __builtin_amdgcn_permlane16_swap(a[e], b[e], false, false);
        a[e] = sw[0];
        b[e] = sw[1];
      }
      const int dcol = 16 * (db + (kb & 1)) + 8 * (kb >> 1);
      if (irow < rows) *reinterpret_cast<uint4*>(op + dcol) = make_uint4(a[0], a[1], b[0], b[1]);
    }
  }
}

template <int D, bool SINK>
int launch_ring(const MP& p, hipStream_t st) {
  static std::once_flag once;
  static hipError_t attr_err = hipSuccess;
  // the window-only launch has no slot operands: the ring is all the LDS it uses
  const size_t lds = SINK ? (size_t)RingCfg<D>::TA : (size_t)RingCfg<D>::BYTES;
  std::call_once(once, [&] { attr_err = hipFuncSetAttribute((const void*)ring_out_kernel<D, SINK>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds); });
  if (attr_err != hipSuccess) {
    set_error("nha_prefill_fwd(mfma): cannot reserve %zu bytes of LDS: %s", lds, hipGetErrorString(attr_err));
    return NHA_ERR_LAUNCH;
  }
  hipLaunchKernelGGL((ring_out_kernel<D, SINK>), dim3(p.H * (p.NG / 4), p.NT), dim3(512), lds, st, p);
  NHA_CHECK_LAUNCH("nha_prefill_fwd(mfma output pass, ring)");
  return NHA_OK;
}

__global__ __launch_bounds__(256) void zero_flags_kernel(int* flags, int n) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i < n) flags[i] = 0;
}

// Exact rows for the window-only launch: the rows of 16-row blocks whose window sums left the range of their fixed
// softmax reference (flags set by ring_out_kernel<D, true>) are recomputed key by key in fp32 with a running maximum,
// the sinks in view joining as keys of logit 0 and value 0.  grid (chunk, kv-head); workgroups of unflagged chunks
// read four words and leave.
template <int D>
__global__ __launch_bounds__(256) void sink_repair_kernel(const MP p) {
  const int chunk = blockIdx.x, h = blockIdx.y;
  const int H = p.H, HQ = p.HQ;
  const int* fl = p.flags + ((int64_t)chunk * H + h) * 4;
  const int bits = fl[0] | fl[1] | fl[2] | fl[3];
  if (bits == 0) return;
  __shared__ float qs[D];
  __shared__ float pw[256];
  __shared__ float red[4];
  const int tid = threadIdx.x;
  const int n = p.cidx[2 * chunk], it = p.cidx[2 * chunk + 1];
  const int bos = p.cu[n], eos = p.cu[n + 1];
  const int c0 = bos + it * BT;
  const int rows = (eos - c0) < BT ? (eos - c0) : BT;
  for (int hq = h * p.NG; hq < (h + 1) * p.NG; ++hq)
    for (int r = 0; r < rows; ++r) {
      if (!((bits >> (r >> 4)) & 1)) continue;
      const int t = c0 + r;
      __syncthreads();   // the previous row is finished
      const bf16_t* qsw = p.q_swa + ((int64_t)t * HQ + hq) * D;
      for (int i = tid; i < D; i += 256) qs[i] = bf16_to_f32(qsw[i]) * p.scale;
      __syncthreads();
      int n0 = p.wl - (t - bos);
      n0 = n0 < 0 ? 0 : (n0 > p.sinks ? p.sinks : n0);
      const int lo = p.wl < 0 ? bos : (t - p.wl > bos ? t - p.wl : bos);
      float wm = -INFINITY, wsum = 0.f;
      for (int j = lo + tid; j <= t; j += 256) {
        const float d = dot_row<bf16_t>(qs, p.k_swa + ((int64_t)j * H + h) * D, D);
        if (d > wm) {
          wsum = wsum * expf(wm - d) + 1.f;
          wm = d;
        } else {
          wsum += expf(d - wm);
        }
      }
      float mt = block_max(wm, red);
      if (n0 > 0) mt = fmaxf(mt, 0.f);
      const float lw = block_sum(wm == -INFINITY ? 0.f : wsum * expf(wm - mt), red) + (float)n0 * expf(-mt);
      if (tid == 0 && p.lse_swa) p.lse_swa[(int64_t)t * HQ + hq] = mt + logf(lw);
      const float inv = 1.f / lw;
      float acc = 0.f;   // value column tid (D <= 256 == threads)
      for (int jb = lo; jb <= t; jb += 256) {
        const int j = jb + tid;
        __syncthreads();
        pw[tid] = j <= t ? expf(dot_row<bf16_t>(qs, p.k_swa + ((int64_t)j * H + h) * D, D) - mt) * inv : 0.f;
        __syncthreads();
        const int cnt = (t - jb + 1) < 256 ? (t - jb + 1) : 256;
        if (tid < D)
          for (int x = 0; x < cnt; ++x) acc += pw[x] * bf16_to_f32(p.v[((int64_t)(jb + x) * H + h) * D + tid]);
      }
      if (tid < D) p.o[((int64_t)t * HQ + hq) * D + tid] = f32_to_bf16(acc);
    }
}

}  // namespace

// Served: four (or a multiple of four) query heads per kv-head at D = 64 or 128.  The per-lane byte
// offsets of the LDS-direct loads are 32 bits: the tensors of one sequence must stay below 4 GiB, which
// the caller's 32-bit token count times the row size decides.
bool prefill_ring_supported(const mf::MP& p, int D) {
  if (!(D == 64 || D == 128) || p.NG % 4 != 0) return false;
  return (int64_t)p.T_tot * p.H * D * 2 < ((int64_t)1 << 32) && (int64_t)p.T_tot * p.H * MS * 2 < ((int64_t)1 << 32);
}

int prefill_ring_launch(const mf::MP& p, int D, hipStream_t st) {
  return D == 64 ? launch_ring<64, false>(p, st) : launch_ring<128, false>(p, st);
}

// Sliding-window attention with zero sinks (nha_sink_window_fwd): the window loop of ring_out_kernel alone.  The scratch
// holds the flags of the 16-row blocks that go to the exact pass.
size_t sink_window_scratch_bytes(const NhaSinkWindowArgs* a) { return ((size_t)a->NT * a->H * 4 * sizeof(int) + 255) & ~(size_t)255; }

int sink_window_impl(const NhaSinkWindowArgs* a) {
  mf::MP p = {};
  p.q_swa = (const bf16_t*)a->q; p.k_swa = (const bf16_t*)a->k; p.v = (const bf16_t*)a->v;
  p.o = (bf16_t*)a->o;
  p.lse_swa = a->lse;
  p.cu = a->cu_seqlens; p.cidx = a->chunk_indices; p.coff = a->chunk_offsets;
  p.flags = (int*)a->scratch;
  p.T_tot = a->T_tot; p.N = a->N; p.NT = a->NT; p.HQ = a->HQ; p.H = a->H; p.NG = a->HQ / a->H;
  p.wl = a->window - 1; p.shift = 0; p.scale = a->scale; p.sinks = a->sinks;
  if (a->dtype != NHA_DTYPE_BF16 || !prefill_ring_supported(p, a->D) || p.NT > 65535) {
    set_error("nha_sink_window_fwd: built for bf16, head size 64 or 128, a multiple of four query heads per kv-head, "
              "at most 65535 chunks and tensors below 4 GiB (dtype=%d D=%d HQ/H=%d NT=%d)", a->dtype, a->D, p.NG, p.NT);
    return NHA_ERR_UNSUPPORTED;
  }
  hipStream_t st = (hipStream_t)a->stream;
  const int nflags = a->NT * a->H * 4;
  hipLaunchKernelGGL(zero_flags_kernel, dim3((nflags + 255) / 256), dim3(256), 0, st, p.flags, nflags);
  NHA_CHECK_LAUNCH("nha_sink_window_fwd(flags)");
  const int rc = a->D == 64 ? launch_ring<64, true>(p, st) : launch_ring<128, true>(p, st);
  if (rc != NHA_OK) return rc;
  if (a->D == 64) hipLaunchKernelGGL((sink_repair_kernel<64>), dim3(p.NT, p.H), dim3(256), 0, st, p);
  else hipLaunchKernelGGL((sink_repair_kernel<128>), dim3(p.NT, p.H), dim3(256), 0, st, p);
  NHA_CHECK_LAUNCH("nha_sink_window_fwd(exact rows)");
  return NHA_OK;
}

}  // namespace nha
