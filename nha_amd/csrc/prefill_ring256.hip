// Output pass of the bf16 matrix-core prefill at head size 256 (K == V == 256, M == 64), one query head
// per workgroup: the data movement and loop of prefill_ring.hip (operands straight from global memory
// into LDS, the window walked first in 32-key units, the slot branch folded into the running softmax
// afterwards; chunk algebra of nha_fla/ops/nha/chunk_fused.py:186-283, one softmax over
// [slots | window] as in nha_fla/ops/nha/chunk.py:459-470) re-proportioned for rows of 512 bytes:
//
//  * One workgroup = NCH consecutive 64-row chunks of a sequence for one query head, 4 NCH waves of 16 query
//    rows: the accumulators of 16 rows x 256 columns are 64 registers, those of 32 rows would not leave room
//    for the fragments.  Launched with NCH = 2: the two chunks walk one window (20 units at a window of 512
//    where two workgroups of one chunk fetch 18 each) with two waves per SIMD; the slot branch, whose tiles
//    and tables are one chunk's, runs chunk by chunk.
//  * A unit of 32 keys is 16 KB of K and 16 KB of V.  K and V units live in two rings of three buffers
//    with their own schedules: iteration u forms the scores of unit u + 1 and the products of unit u, so
//    after its barrier the K buffer of unit u + 1 and the V buffer of unit u - 1 are free and take K of
//    unit u + 4 and V of unit u + 2; both have two iterations to land.
//  * Fragments are read from LDS a few matrix instructions before their use and not earlier: sixteen K
//    and sixteen V fragments held at once (128 registers) would push the accumulators out of the
//    register file.
//  * The slot-branch operands (four 64 x 256 tiles, 128 KB) do not fit beside the rings: they pass
//    through the ring buffers.  The two halves of the chunk-start k-state and the first half of the
//    chunk's k_gsa rows are requested into the K buffers the last iterations of the loop retire, the
//    second half of the rows into the V buffer the last iteration retires, the halves of the v-state after
//    the loop; the chunk's v rows replace the k-state once the slot logits are formed.
//  * The softmax reference of a row is fixed by the prologue (the chunk's own keys): rescaling 64
//    accumulator registers inside the loop costs the loop its registers whether or not the branch is
//    taken.  A unit whose maximum tops the reference by 2^96 hands the wave's 16 rows to the exact pass
//    (mfma_repair_kernel) and is clamped.
#include "mfma_common.h"

#include <mutex>

namespace nha {
namespace {
using namespace mf;

typedef NHA_LDS unsigned char lbyte;
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

#define NHA_FENCE() __builtin_amdgcn_sched_barrier(0)
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

template <int NCH>
struct Cfg {
  static constexpr int D = 256;
  static constexpr int KS = D / 32;            // 32-column blocks per row == contraction steps of q.k
  static constexpr int DB = D / 16;            // 16-row blocks of O^T
  static constexpr int UB = 32 * D * 2;        // bytes of a 32-row unit buffer (16 KB)
  static constexpr int HB = UB / 2;            // bytes of its 16-row half
  static constexpr int NR = 3;                 // buffers per ring
  static constexpr int NW = 4 * NCH;           // waves: four 16-row sub-blocks per chunk
  static constexpr int BPU = 2 * KS;           // 1 KB blocks of a unit buffer (16)
  static constexpr int LPB = BPU / NW;         // LDS-direct loads per wave for one buffer (4 or 2)
  static constexpr int RING_K = 0, RING_V = NR * UB;
  static constexpr int GC = 2 * NR * UB;       // gate cumsum fp32 [64][64], pieces XORed with row % 16
  static constexpr int SS = GC + 16384;        // s bf16 [64][64], pieces XORed with row % 8
  static constexpr int ETAB = SS + 8192;       // decay tables, 6 units of 4 KB
  static constexpr int GC2 = ETAB + 6 * 4096;  // gate cumsums of the second chunk (NCH == 2)
  static constexpr int BYTES = GC2 + (NCH - 1) * 16384;
};

// Two chunks per workgroup: launch index -> (query head, chunk).  The grid has a workgroup per (query head, chunk);
// those of a sequence's odd chunks leave at once.  The even chunk indices come first in the launch order (in sequences
// of even chunk counts they are the working ones), from the last chunk to the first, and as in xcd_tile XCD k (launch
// index % 8) takes the k-th eighth of each class, so that neighbouring pairs of a kv-head meet in one L2.
__device__ __forceinline__ void pair_tile(int ngrp, int nchunks, int& vx, int& chunk) {
  const int nev = (nchunks + 1) >> 1, nod = nchunks >> 1;
  const int L = blockIdx.y * gridDim.x + blockIdx.x;
  const int tot_e = gridDim.x * nev, tot_o = gridDim.x * nod;
  // each class is dealt to the XCDs in eighths; the up to seven workgroups a class has beyond a multiple of 8 keep
  // their place at its end
  int v, nn, par;
  const int pe = tot_e >> 3, po = tot_o >> 3;
  if (L < 8 * (pe + po)) {
    const int k = L & 7, w = L >> 3;
    if (w < pe) {
      v = k * pe + w, nn = nev, par = 0;
    } else {
      v = k * po + (w - pe), nn = nod, par = 1;
    }
  } else {
    const int r = L - 8 * (pe + po);   // < (tot_e & 7) + (tot_o & 7)
    if (r < (tot_e & 7)) {
      v = 8 * pe + r, nn = nev, par = 0;
    } else {
      v = 8 * po + r - (tot_e & 7), nn = nod, par = 1;
    }
  }
  const int g = v % ngrp, rest = v / ngrp;
  vx = (rest / nn) * ngrp + g;
  chunk = 2 * (nn - 1 - rest % nn) + par;
}

// LDS layouts as in prefill_ring.hip: a 32-row buffer is cut into 16-row x 32-column blocks of 1 KB
// (half h, column block c at h * HB + c * 1024).  K layout: 16-byte piece c of row r at 256 c + 16 r (a wave's
// row fragments are 1 KB of consecutive bytes).  V layout: two planes of 16 rows x 32 bytes (columns 0..15, then 16..31).
template <int NCH>
__global__ __launch_bounds__(256 * NCH, 1) void ring256_out_kernel(const MP p) {
  using C = Cfg<NCH>;
  constexpr int XB0 = 64 * NCH - 32;           // first key of unit 0, relative to the workgroup's first row
  constexpr int D = C::D, KS = C::KS, DB = C::DB, UB = C::UB, HB = C::HB, NR = C::NR, NW = C::NW, LPB = C::LPB;
  extern __shared__ __align__(1024) unsigned char smem_[];
  lbyte* const lds = (lbyte*)smem_;
  const uint32_t lds0 = (uint32_t)(uintptr_t)lds;
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l16 = lane & 15, kb = lane >> 4;
  const int H = p.H, HQ = p.HQ, NG = p.NG;
  // grid = (query head, chunk), tiles dealt so that an XCD works on neighbouring chunks of one kv-head
  // (xcd_tile); chunks from the last to the first
  int vx, chunk;
  if constexpr (NCH == 1) {
    int vy;
    xcd_tile(NG, p.NT, vx, vy);
    chunk = p.NT - 1 - vy;
  } else {
    pair_tile(NG, p.NT, vx, chunk);
  }
  const int hq = vx, h = hq / NG;
  const int ch = wave >> 2;                    // this wave's chunk of the workgroup's NCH
  const int Q = wave & 3;                      // its 16-row sub-block of that chunk
  const int n = p.cidx[2 * chunk], it = p.cidx[2 * chunk + 1];
  // two chunks per workgroup: the workgroup of a sequence's even chunk takes that chunk and the next one of the
  // same sequence, if there is one; the workgroups of the odd chunks leave at once
  if (NCH == 2 && (it & 1)) return;
  const int bos = p.cu[n], eos = p.cu[n + 1];
  const int c0 = bos + it * BT;                // first row of the workgroup (its first chunk)
  const int rows_wg = (eos - c0) < NCH * BT ? (eos - c0) : NCH * BT;
  const int rows = rows_wg - BT * ch < 0 ? 0 : (rows_wg - BT * ch < BT ? rows_wg - BT * ch : BT);   // rows of this wave's chunk
  const float cs = p.scale * LOG2E;
  const int64_t cg = (int64_t)chunk * H + h;   // (chunk, kv-head) of the first chunk; the second one is H further
  const int irow = 16 * Q + l16;               // this lane's query row inside its chunk
  const int yrow = BT * ch + irow;             // ... and inside the workgroup's rows
  const int r0w = BT * ch + 16 * Q;            // first row of this wave

  // window units: unit u covers keys [c0 + XB0 - 32 u, c0 + XB0 + 32 - 32 u); c0 - bos is a multiple of 64, so no
  // unit starts before its sequence; units 0 .. 2 NCH - 1 are the workgroup's own rows and may run past eos
  int lowest = bos;
  if (p.wl >= 0 && c0 - p.wl > bos) lowest = c0 - p.wl;
  const int nunits = (c0 + BT * NCH - lowest + 31) / 32;   // >= 2 NCH

  // ---- LDS-direct loads: block b = wave + NW i of a buffer; per lane a row of the block and a 16-byte piece
  const int lrow16 = lane & 15, lswz = lane >> 4;          // K layout
  const int lrowv = (lane & 31) >> 1, lpv = 2 * (lane >> 5) + (lane & 1);         // V layout
  // one 32-row buffer from rows of `src` (row stride in elements): row r of the buffer is global row rowmap(r)
  auto issue_buffer = [&](uint32_t lds_buf, bool vlay, const bf16_t* src, uint32_t stride, auto rowmap) {
#pragma unroll
    for (int i = 0; i < LPB; ++i) {
      const int b = wave + NW * i;           // < 16
      const int rh = b / KS, cq = b % KS;
      const int r = 16 * rh + (vlay ? lrowv : lrow16);
      const uint32_t off = ((uint32_t)rowmap(r) * stride + (uint32_t)(4 * cq + (vlay ? lpv : lswz)) * 8) * 2;
      g2l16(src, off, lds0 + lds_buf + rh * HB + cq * 1024);
    }
  };
  const bf16_t* const kbase = p.k_swa + ((int64_t)bos * H + h) * D;
  const bf16_t* const vbase = p.v + ((int64_t)bos * H + h) * D;
  // rows past eos (the workgroup's own units only) are read from row eos - 1: always masked, always finite
  auto unit_row = [&](int u) {
    const int key0 = c0 + XB0 - 32 * u - bos;
    const int last = eos - 1 - bos;
    return [=](int r) { return key0 + r < last ? key0 + r : last; };
  };
  auto issue_k = [&](int u) { issue_buffer(C::RING_K + (u % NR) * UB, false, kbase, (uint32_t)(H * D), unit_row(u)); };
  auto issue_v = [&](int u) { issue_buffer(C::RING_V + (u % NR) * UB, true, vbase, (uint32_t)(H * D), unit_row(u)); };
  // units >= 2 NCH lie wholly before the workgroup's rows (never past eos): fixed per-lane offsets from a wave-uniform row pointer
  uint32_t koff[LPB], voff[LPB], boff[LPB];
#pragma unroll
  for (int i = 0; i < LPB; ++i) {
    const int b = wave + NW * i;
    const int rh = b / KS, cq = b % KS;
    koff[i] = ((uint32_t)(16 * rh + lrow16) * (uint32_t)(H * D) + (uint32_t)(4 * cq + lswz) * 8) * 2;
    voff[i] = ((uint32_t)(16 * rh + lrowv) * (uint32_t)(H * D) + (uint32_t)(4 * cq + lpv) * 8) * 2;
    boff[i] = lds0 + rh * HB + cq * 1024;
  }
  auto issue_k_fast = [&](int u, uint32_t slot_off) {
    if (NCH > 1 && u < 2 * NCH) {
      issue_buffer(C::RING_K + slot_off, false, kbase, (uint32_t)(H * D), unit_row(u));
      return;
    }
    const bf16_t* src = p.k_swa + (((int64_t)c0 + XB0 - 32 * u) * H + h) * D;
#pragma unroll
    for (int i = 0; i < LPB; ++i) g2l16(src, koff[i], boff[i] + C::RING_K + slot_off);
  };
  auto issue_v_fast = [&](int u, uint32_t slot_off) {
    if (NCH > 1 && u < 2 * NCH) {
      issue_buffer(C::RING_V + slot_off, true, vbase, (uint32_t)(H * D), unit_row(u));
      return;
    }
    const bf16_t* src = p.v + (((int64_t)c0 + XB0 - 32 * u) * H + h) * D;
#pragma unroll
    for (int i = 0; i < LPB; ++i) g2l16(src, voff[i], boff[i] + C::RING_V + slot_off);
  };

  // The slot branch runs chunk by chunk (its tables and tiles are one chunk's): cc is the chunk it is at, and these
  // are that chunk's first row whose source token exists, its number of rows and the source token of its row 0
  int cc = 0;
  int vlo = (p.shift - it * BT) < 0 ? 0 : (p.shift - it * BT);
  int rows_c = rows_wg < BT ? rows_wg : BT;
  int grow_s = c0 - p.shift;
  uint32_t gco = C::GC;   // where that chunk's gate cumsums lie
  auto tok_from = [&](int gs, int r) {   // source token of row r of a chunk whose row 0 has source token gs, kept inside the sequence
    int t = gs + r;
    t = t < bos ? bos : t;
    t = t < eos ? t : eos - 1;
    return t - bos;
  };
  auto tok = [&](int r) { return tok_from(grow_s, r); };   // rows outside [vlo, rows_c) carry no weight
  // gate cumsums of chunk c of the workgroup (16 blocks of 4 rows; rows past the chunk's last were never written by the
  // state pass and stay unused) and the s rows of its source tokens
  auto issue_gc = [&](int c_, uint32_t dst) {
#pragma unroll
    for (int i = 0; i < 16 / NW; ++i) {
      const int b = wave + NW * i;
      const int r = 4 * b + (lane >> 4);
      const int c = (lane & 15) ^ (r & 15);
      g2l16(p.gc + (cg + (int64_t)c_ * H) * BT * MS, (uint32_t)(r * MS + 4 * c) * 4, lds0 + dst + b * 1024);
    }
  };
  auto issue_s = [&](int gs) {
#pragma unroll
    for (int i = 0; i < 8 / NW; ++i) {
      const int b = wave + NW * i;
      const int r = 8 * b + (lane >> 3);
      const int c = (lane & 7) ^ (r & 7);
      g2l16(p.s + ((int64_t)bos * H + h) * MS, ((uint32_t)tok_from(gs, r) * (uint32_t)(H * MS) + (uint32_t)c * 8) * 2, lds0 + C::SS + b * 1024);
    }
  };

  auto gc_at = [&](int j, int m) -> const lfloat* { return (const lfloat*)(lds + gco + j * 256 + (((m >> 2) ^ (j & 15)) * 16) + (m & 3) * 4); };
  auto s_at = [&](int j, int m) -> const lbf16* { return (const lbf16*)(lds + C::SS + j * 128 + (((m >> 3) ^ (j & 7)) * 16) + (m & 7) * 2); };
  // decay tables E_Q[j][m] = s_j[m] exp(min(gr_Q[m] - gc_j[m], DECAY_CLAMP)) for the rows j of the 16-row
  // blocks jb <= Q, zero elsewhere (gr_Q: gate cumsum of the row before sub-block Q, 0 for Q = 0); rows
  // whose source token does not exist carry no weight.  32-row units in the V layout (64 columns):
  // E_0 -> unit 0, E_1 -> 1, E_2 -> 2,3, E_3 -> 4,5; a thread makes 8 consecutive slots of a row.
  auto build_decay_tables = [&]() {
    for (int item = tid; item < 6 * 256; item += 64 * NW) {
      const int U = item >> 8, r32 = (item >> 3) & 31, m = (item & 7) * 8;
      const int Qt = U == 0 ? 0 : U == 1 ? 1 : U < 4 ? 2 : 3;
      const int pr = (U == 3 || U == 5) ? 1 : 0;
      const int j = 32 * pr + r32;
      const bool ok = (j >> 4) <= Qt && j >= vlo && j < rows_c;
      bf16x8 out;
#pragma unroll
      for (int e = 0; e < 8; ++e) out[e] = (__bf16)0.f;
      if (ok) {
        f32x4 gv[2], gr[2];
#pragma unroll
        for (int hh = 0; hh < 2; ++hh) {
          gv[hh] = *reinterpret_cast<const NHA_LDS f32x4*>(gc_at(j, m + 4 * hh));
          gr[hh] = (f32x4){0.f, 0.f, 0.f, 0.f};
          if (Qt > 0) gr[hh] = *reinterpret_cast<const NHA_LDS f32x4*>(gc_at(16 * Qt - 1, m + 4 * hh));
        }
        const bf16x8 sv = *reinterpret_cast<const NHA_LDS bf16x8*>(s_at(j, m));
#pragma unroll
        for (int e = 0; e < 8; ++e) out[e] = (__bf16)((float)sv[e] * fexp(fminf(gr[e >> 2][e & 3] - gv[e >> 2][e & 3], DECAY_CLAMP)));
      }
      *reinterpret_cast<NHA_LDS bf16x8*>(lds + C::ETAB + U * 4096 + (r32 >> 4) * 2048 + (m >> 5) * 1024 + ((m >> 4) & 1) * 512 + (r32 & 15) * 32 + (m & 15) * 2) = out;
    }
  };
  // ---- requests: the gate blocks (the decay tables are built from them while the units are still on their
  //      way; the second chunk's gate cumsums wait in a place of their own), K and V of the first units, then the
  //      query fragments -------------------------------------
  const bool second = rows_wg > BT;   // the workgroup has a second chunk
  issue_gc(0, C::GC);
  issue_s(grow_s);
  if (NCH == 2 && second) issue_gc(1, C::GC2);
  issue_k(0);
  issue_v(0);
  issue_k(1);
  issue_v(1);
  if (2 < nunits) issue_k_fast(2, 2 * UB);
  // window-query fragments, pre-scaled by scale * log2(e)
  bf16x8 qs[KS];
  uint4 qraw[KS];
  {
    // rows past the end of the sequence read the last row (the number of loads must not depend on the lane:
    // the wait below counts them) and are zeroed afterwards
    const bf16_t* qp = p.q_swa + ((int64_t)(c0 + (yrow < rows_wg ? yrow : rows_wg - 1)) * HQ + hq) * D + 8 * kb;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) qraw[ks] = *reinterpret_cast<const uint4*>(qp + 32 * ks);
  }
  NHA_FENCE();
  // the gate blocks were requested first: they have landed once no more than the requests made after them
  // are outstanding (four or five unit buffers and the query loads)
  if (2 < nunits) wait_vm<5 * LPB + KS>();
  else wait_vm<4 * LPB + KS>();
  lds_barrier();
  build_decay_tables();
  NHA_FENCE();
  {
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const uint4 x = irow < rows ? qraw[ks] : make_uint4(0, 0, 0, 0);
      const uint32_t w[4] = {x.x, x.y, x.z, x.w};
      bf16x8 r;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float f = __uint_as_float((e & 1) ? (w[e >> 1] & 0xffff0000u) : (w[e >> 1] << 16));
        r[e] = (__bf16)(f * cs);
      }
      qs[ks] = r;
    }
  }

  // ---- window loop state ------------------------------------------------------------------------
  f32x4 O[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db) O[db] = (f32x4){0.f, 0.f, 0.f, 0.f};
  f32x4 Lw = {0.f, 0.f, 0.f, 0.f};
  float nm = 0.f;                      // minus the running reference maximum, log2 units
  f32x4 nmv = {0.f, 0.f, 0.f, 0.f};    // nm broadcast: the accumulator the score products start from
  bf16x8 ones;
#pragma unroll
  for (int e = 0; e < 8; ++e) ones[e] = (__bf16)1.0f;
  constexpr float THR = 8.f;           // the reference moves (prologue, slot branch) when a score tops it by more than 2^THR
  constexpr float BIG = 96.f;          // scores this far above the reference leave the matrix-core path

  const uint32_t kaddr = (uint32_t)(lane * 16);
  const uint32_t vaddr = (uint32_t)((4 * kb + (l16 >> 2)) * 32 + 8 * (l16 & 3));
  // row fragment (rows 16 kk + l16 of a buffer, columns 32 ks + 8 kb ..) of a K-layout buffer at byte address a
  auto kfrag = [&](uint32_t a, int kk, int ks) -> bf16x8 {
    const lbyte* base = lds + (a + kaddr);     // one address per buffer; the fragment is a constant offset from it
    return *reinterpret_cast<const NHA_LDS bf16x8*>(base + (kk * HB + ks * 1024));
  };
  // transposed fragment of a V-layout buffer: X[4 kb + e][16 db + l16] (e < 4) and X[16 + 4 kb + e - 4][..]
  auto vfrag = [&](uint32_t a, int db) -> bf16x8 {
    const lbyte* base = lds + (a + vaddr);
    const lbyte* pa = base + ((db >> 1) * 1024 + (db & 1) * 512);
    struct { s16x4 a, b; } t;
    t.a = __builtin_amdgcn_ds_read_tr16_b64_v4i16((NHA_LDS s16x4*)pa);
    t.b = __builtin_amdgcn_ds_read_tr16_b64_v4i16((NHA_LDS s16x4*)(pa + HB));
    return __builtin_bit_cast(bf16x8, t);
  };
  auto mask_unit = [&](f32x4 (&S)[2], int u) {
    const int xbase = XB0 - 32 * u;
#pragma unroll
    for (int kk = 0; kk < 2; ++kk)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int x = xbase + 16 * kk + 4 * kb + r;
        const bool ok = (x <= yrow) && (p.wl < 0 || x >= yrow - p.wl);
        if (!ok) S[kk][r] = -INFINITY;
      }
  };
  // a unit needs the mask when its last key lies after this wave's first row or its first key before the window of
  // this wave's last row
  auto is_edge = [&](int u) -> bool { return (XB0 + 31 - 32 * u > r0w) || (p.wl >= 0 && XB0 - 32 * u < r0w + 15 - p.wl); };

  // the reference moves up by delta: everything accumulated so far shrinks by 2^-delta
  auto rescale_acc = [&](float delta) {
    const float alpha = fexp2(-delta);
    nm -= delta;
    nmv = (f32x4){nm, nm, nm, nm};
#pragma unroll
    for (int r = 0; r < 4; ++r) Lw[r] *= alpha;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int r = 0; r < 4; ++r) O[db][r] *= alpha;
  };
  auto rescale = [&](f32x4 (&S)[2], float rmax) {
    const float delta = fmaxf(max_over_rows(rmax), 0.f);
    rescale_acc(delta);
#pragma unroll
    for (int kk = 0; kk < 2; ++kk)
#pragma unroll
      for (int r = 0; r < 4; ++r) S[kk][r] -= delta;
  };
  auto max8 = [&](const f32x4 (&S)[2]) -> float {
    const float a = fmaxf(fmaxf(S[0][0], S[0][1]), fmaxf(S[0][2], S[0][3]));
    return fmaxf(a, fmaxf(fmaxf(S[1][0], S[1][1]), fmaxf(S[1][2], S[1][3])));
  };

  f32x4 Sc[2], Sn[2];
  // fragments requested from LDS ahead of the matrix instruction that takes them: with one wave per SIMD 4 to 14 measure
  // the same; with two (the other wave fills the waits) 2 is best by 1.5 % (1, 3, 4: 0 - 1 %; 8, 10: slower)
  constexpr int PD = NCH == 2 ? 2 : 6;
  // ---- prologue: scores of unit 0, K fragments of unit 1 -----------------------------------------------
  wait_vm<0>();
  lds_barrier();
  {
    Sc[0] = nmv;
    Sc[1] = nmv;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      Sc[0] = mfma16(kfrag(C::RING_K, 0, ks), qs[ks], Sc[0]);
      Sc[1] = mfma16(kfrag(C::RING_K, 1, ks), qs[ks], Sc[1]);
    }
    mask_unit(Sc, 0);   // unit 0 is always an edge unit
    const float x = max8(Sc);
    if (__any(x > THR)) rescale(Sc, x);
  }
  // every wave has read the K buffer of unit 0: unit 3 takes it; every wave has built its part of the first chunk's
  // decay tables, the last readers of its s rows: the second chunk's s rows take their place (one load per wave,
  // older than everything the loop's waits leave in flight)
  lds_barrier();
  if (NCH == 2 && second) issue_s(c0 + BT - p.shift);
  if (3 < nunits) issue_k_fast(3, 0);

  // slot-branch query fragments (requested while the last unit is worked on)
  bf16x8 qg[KS];
  auto load_qg = [&]() {
    const bf16_t* qp = p.q_gsa + ((int64_t)(c0 + yrow) * HQ + hq) * D + 8 * kb;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      uint4 x = make_uint4(0, 0, 0, 0);
      if (irow < rows) x = *reinterpret_cast<const uint4*>(qp + 32 * ks);
      qg[ks] = as_bf16x8(x);
    }
  };
  auto pack_p = [&]() -> bf16x8 {
    const u32x4 t = {cvt2(Sc[0][0], Sc[0][1]), cvt2(Sc[0][2], Sc[0][3]), cvt2(Sc[1][0], Sc[1][1]), cvt2(Sc[1][2], Sc[1][3])};
    bf16x8 P = __builtin_bit_cast(bf16x8, t);
    NHA_PIN(P);
    return P;
  };

  // The slot-branch tiles (k-state, k_gsa rows, v-state as two 32-row halves each) take ring buffers as the
  // window loop retires them: with at least five units the last three K buffers and the last V buffer to
  // come free receive four of the six halves while the loop still runs (a half is as many loads as a
  // unit buffer, so the in-flight counts of the loop stay what they are); the two v-state halves follow
  // after the loop, and shorter windows request everything then.
  const bf16_t* const t_kg = p.k_gsa + ((int64_t)bos * H + h) * D;
  auto issue_ta = [&](uint32_t off, int half) { issue_buffer(off, false, p.hkT + (cg + (int64_t)cc * H) * MS * D, (uint32_t)D, [=](int r) { return 32 * half + r; }); };
  auto issue_tb = [&](uint32_t off, int half) { issue_buffer(off, false, t_kg, (uint32_t)(H * D), [&](int r) { return tok(32 * half + r); }); };
  auto issue_tc = [&](uint32_t off, int half) { issue_buffer(off, true, p.hvc + (cg + (int64_t)cc * H) * MS * D, (uint32_t)D, [=](int r) { return 32 * half + r; }); };
  const bool early = nunits >= 5;
  uint32_t oA0 = C::RING_K, oA1 = C::RING_K + UB, oB0 = C::RING_K + 2 * UB, oB1 = C::RING_V;   // where the halves lie
  uint32_t oC0 = C::RING_V + UB, oC1 = C::RING_V + 2 * UB;
  // ring positions as rotating buffer offsets: s0 = buffer of unit u, s1 of unit u+1, s2 of unit u+2
  uint32_t s0 = 0, s1 = UB, s2 = 2 * UB;
  for (int u = 0; u + 1 < nunits; ++u) {
    const uint32_t k_n = C::RING_K + s1;    // K of unit u+1
    const uint32_t v_c = C::RING_V + s0;    // V of unit u
    // ---- phase A: scores of unit u+1 on the matrix core (two accumulators in turn), exponentials of
    //      unit u on the VALU (one per two products); K fragment i = 2 ks + kk is read PD products ahead ----
    bf16x8 kfr[2 * KS];
    NHA_FENCE();
#pragma unroll
    for (int i = 0; i < PD; ++i) kfr[i] = kfrag(k_n, i & 1, i >> 1);
    NHA_FENCE();
#pragma unroll
    for (int i = 0; i < 2 * KS; ++i) {
      const int ks = i >> 1, kk = i & 1;
      if (i + PD < 2 * KS) kfr[i + PD] = kfrag(k_n, (i + PD) & 1, (i + PD) >> 1);
      Sn[kk] = mfma16(kfr[i], qs[ks], ks == 0 ? nmv : Sn[kk]);
      if (kk == 1) {
        Sc[ks >> 2][ks & 3] = fexp2(Sc[ks >> 2][ks & 3]);
        NHA_PIN(Sc[ks >> 2][ks & 3]);
      }
      NHA_FENCE();
    }
    const bf16x8 Pq = pack_p();
    NHA_FENCE();
    // K of unit u+2 and V of unit u (requested two iterations ago) have landed for this wave, then for
    // everybody.  What may stay in flight: the requests of the previous iteration.
    if (u >= 1) {
      if (early) {                    // every iteration requests two buffers' worth, V side first
        if (u + 2 == nunits) wait_vm<LPB>();   // last iteration: also V of the last unit; the tile half behind it may fly
        else wait_vm<2 * LPB>();
      } else {
        wait_vm<0>();
      }
    }
    lds_barrier();
    if (u + 2 < nunits) {
      issue_v_fast(u + 2, s2);
    } else if (early) {
      oB1 = C::RING_V + s2;
      issue_tb(oB1, 1);
    }
    if (u + 4 < nunits) {
      issue_k_fast(u + 4, s1);   // unit u+4 takes the buffer of unit u+1
    } else if (early) {
      const uint32_t off = C::RING_K + s1;
      if (u + 4 == nunits) {
        oA0 = off;
        issue_ta(off, 0);
      } else if (u + 3 == nunits) {
        oA1 = off;
        issue_ta(off, 1);
      } else {
        oB0 = off;
        issue_tb(off, 0);
      }
    }
    NHA_FENCE();
    // ---- phase B: value products of unit u on the matrix core, row maximum of unit u+1 on the VALU;
    //      V fragment db is read PD products ahead ----
    float m0 = 0.f, m1 = 0.f;
    auto max_step = [&](int s2) {
      if (s2 == 0) m0 = fmaxf(Sn[0][0], Sn[0][1]);
      if (s2 == 1) m1 = fmaxf(Sn[0][2], Sn[0][3]);
      if (s2 == 2) m0 = fmaxf(fmaxf(m0, Sn[1][0]), Sn[1][1]);
      if (s2 == 3) m1 = fmaxf(fmaxf(m1, Sn[1][2]), Sn[1][3]);
      if (s2 == 4) m0 = fmaxf(m0, m1);
      if (s2 == 0 || s2 == 2 || s2 == 4) NHA_PIN(m0);
      if (s2 == 1 || s2 == 3) NHA_PIN(m1);
    };
    bf16x8 vfr[DB];
#pragma unroll
    for (int i = 0; i < PD; ++i) vfr[i] = vfrag(v_c, i);
    Lw = mfma16(ones, Pq, Lw);
    NHA_FENCE();
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      if (db + PD < DB) vfr[db + PD] = vfrag(v_c, db + PD);
      O[db] = mfma16(vfr[db], Pq, O[db]);
      if (db % 3 == 0 && db / 3 < 5) max_step(db / 3);
      NHA_FENCE();
    }
    if (is_edge(u + 1)) {
      mask_unit(Sn, u + 1);
      m0 = max8(Sn);
    }
    // The reference of the window stays where the prologue put it: moving it would mean rescaling 64
    // accumulator registers inside this loop, which costs the loop its registers whether or not the branch
    // is ever taken.  fp32 sums and bf16 probabilities hold 2^BIG above it; a score beyond that sends the
    // wave's 16 rows to the exact pass (mfma_repair_kernel recomputes flagged sub-blocks) and is clamped.
    if (__any(m0 > BIG)) {
      if (lane == 0) atomicOr(p.flags + (cg + (int64_t)ch * H) * 4, 1 << Q);
#pragma unroll
      for (int kk = 0; kk < 2; ++kk)
#pragma unroll
        for (int r = 0; r < 4; ++r) Sn[kk][r] = fminf(Sn[kk][r], BIG);
    }
    Sc[0] = Sn[0];
    Sc[1] = Sn[1];
    const uint32_t t0 = s0;
    s0 = s1;
    s1 = s2;
    s2 = t0;
  }
  // ---- the last unit: no further scores; the slot-branch queries are requested meanwhile ----
  {
    const int u = nunits - 1;
    const uint32_t v_c = C::RING_V + (u % NR) * UB;
    bf16x8 vf[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db) vf[db] = vfrag(v_c, db);
    load_qg();
#pragma unroll
    for (int kk = 0; kk < 2; ++kk)
#pragma unroll
      for (int r = 0; r < 4; ++r) Sc[kk][r] = fexp2(Sc[kk][r]);
    const bf16x8 Pq = pack_p();
    Lw = mfma16(ones, Pq, Lw);
#pragma unroll
    for (int db = 0; db < DB; ++db) O[db] = mfma16(vf[db], Pq, O[db]);
  }

  // ================= slot branch, folded into the running softmax =================================
  // One chunk at a time: the tables and tiles in LDS are one chunk's.  Every wave requests its share of the loads,
  // helps with the tables and keeps the barriers; the products are those of the waves whose rows the chunk holds.
  // every request of this wave has landed, every wave is done with the rings
  wait_vm<0>();
  lds_barrier();
  // the window's own log-sum-exp, before the slots join the running softmax
  if (p.lse_swa && kb == 0 && irow < rows) p.lse_swa[(int64_t)(c0 + yrow) * HQ + hq] = (__builtin_amdgcn_logf(Lw[0]) - nm) * LN2;
  float psum = 0.f;
#pragma unroll 1
  for (cc = 0; cc < NCH; ++cc) {
    if (cc == 0) {
      if (!early) {
        issue_ta(oA0, 0);
        issue_ta(oA1, 1);
        issue_tb(oB0, 0);
        issue_tb(oB1, 1);
      } else {   // the V buffers of the last two units (s0, s2 after the loop's last rotation) are the free ones
        oC0 = C::RING_V + s2;
        oC1 = C::RING_V + s0;
      }
      issue_tc(oC0, 0);
      issue_tc(oC1, 1);
    } else {
      // the second chunk: its tiles are requested once the first chunk is done with the buffers, and its decay tables
      // built, from the gate blocks that came in during the window loop, once the first chunk is done with the tables
      if (!second) break;
      lds_barrier();
      vlo = (p.shift - (it + 1) * BT) < 0 ? 0 : (p.shift - (it + 1) * BT);
      rows_c = rows_wg - BT;
      grow_s = c0 + BT - p.shift;
      gco = C::GC2;
      // the tiles go where the first chunk's were; the k_gsa rows are already on their way (requested when the first
      // chunk had read its own)
      issue_ta(oA0, 0);
      issue_ta(oA1, 1);
      issue_tc(oC0, 0);
      issue_tc(oC1, 1);
      build_decay_tables();
    }
    const bool mine = ch == cc;

    // k-state and k_gsa rows have landed (the two v-state halves may still fly)
    wait_vm<2 * LPB>();
    __syncthreads();

    const int etu = Q < 2 ? Q : 2 * Q - 2;   // first table unit of this wave's sub-block
    // E_Q transposed: rows = slots 16 mb + l16, contraction over the tokens 32 pr + {4 kb + e, 16 + 4 kb + e - 4}
    auto etab_tr = [&](int pr, int mb) -> bf16x8 {
      const lbyte* pa = lds + C::ETAB + (etu + pr) * 4096 + (mb >> 1) * 1024 + (mb & 1) * 512 + vaddr;
      struct { s16x4 a, b; } t;
      t.a = __builtin_amdgcn_ds_read_tr16_b64_v4i16((NHA_LDS s16x4*)pa);
      t.b = __builtin_amdgcn_ds_read_tr16_b64_v4i16((NHA_LDS s16x4*)(pa + 2048));
      return __builtin_bit_cast(bf16x8, t);
    };
    // E_Q by rows: row = token 16 jb + l16, contraction over the slots 32 pr + {4 kb + e, 16 + 4 kb + e - 4}
    auto etab_row = [&](int jb, int pr) -> bf16x8 {
      const lbyte* pa = lds + C::ETAB + (etu + (jb >> 1)) * 4096 + (jb & 1) * 2048 + pr * 1024 + l16 * 32 + 8 * kb;
      struct { bf16x4 a, b; } t;
      t.a = *reinterpret_cast<const NHA_LDS bf16x4*>(pa);
      t.b = *reinterpret_cast<const NHA_LDS bf16x4*>(pa + 512);
      return __builtin_bit_cast(bf16x8, t);
    };

    // inter-chunk slot logits: okT[m][i] = sum_d hkT[m][d] q[i][d]
    f32x4 ok[4];
    if (mine) {
#pragma unroll
      for (int mb = 0; mb < 4; ++mb) ok[mb] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
#pragma unroll
        for (int mb = 0; mb < 4; ++mb) ok[mb] = mfma16(kfrag(((mb >> 1) ? oA1 : oA0), mb & 1, ks), qg[ks], ok[mb]);
    }
    // every wave is done with the k-state tile: the v rows take its buffers and land during what follows
    lds_barrier();
#pragma unroll
    for (int half = 0; half < 2; ++half)
      issue_buffer(half ? oA1 : oA0, true, vbase, (uint32_t)(H * D), [&](int r) { return tok(32 * half + r); });
    bf16x8 bp[2], bpr[2];   // slot probabilities x exp(gc_i) and x exp(gc_i - gr), B operands
    if (mine) {
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
            if (jb <= Q) at[jb] = mfma16(kfrag(((jb >> 1) ? oB1 : oB0), jb & 1, ks), qg[ks], at[jb]);
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
      // okT_intra[m][i] = sum_j s_j[m] exp(gr[m] - gc_j[m]) AT[j][i]
      f32x4 oki[4];
#pragma unroll
      for (int mb = 0; mb < 4; ++mb) {
        oki[mb] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int pr = 0; pr < 2; ++pr)
          if (2 * pr <= Q) oki[mb] = mfma16(etab_tr(pr, mb), bA[pr], oki[mb]);
      }
      // combine; the slot logits join the running softmax as one more set of keys
      const int rref = 16 * Q - 1;
      f32x4 egi[4], egr[4];   // exp(gc_i[m]) and exp(gc_i[m] - gr[m]) in accumulator layout
      float xmax = -INFINITY;
#pragma unroll
      for (int mb = 0; mb < 4; ++mb) {
        const f32x4 gi = *reinterpret_cast<const NHA_LDS f32x4*>(gc_at(irow, 16 * mb + 4 * kb));
        f32x4 gr4 = (f32x4){0.f, 0.f, 0.f, 0.f};
        if (Q > 0) gr4 = *reinterpret_cast<const NHA_LDS f32x4*>(gc_at(rref, 16 * mb + 4 * kb));
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          egi[mb][r] = fexp(gi[r]);
          egr[mb][r] = fexp(gi[r] - gr4[r]);
          ok[mb][r] = (ok[mb][r] * egi[mb][r] + oki[mb][r] * egr[mb][r]) * cs;   // slot logit, log2 units
          xmax = fmaxf(xmax, ok[mb][r]);
        }
      }
      const float ms = max_over_rows(xmax);   // the slots' own maximum
      if (__any(ms + nm > THR)) rescale_acc(fmaxf(ms + nm, 0.f));
      if (p.lse_gsa) {
        float pown = 0.f;
#pragma unroll
        for (int mb = 0; mb < 4; ++mb)
#pragma unroll
          for (int r = 0; r < 4; ++r) pown += fexp2(ok[mb][r] - ms);
        pown += __shfl_xor(pown, 16, 64);
        pown += __shfl_xor(pown, 32, 64);
        if (kb == 0 && irow < rows) p.lse_gsa[(int64_t)(c0 + yrow) * HQ + hq] = (__builtin_amdgcn_logf(pown) + ms) * LN2;
      }
#pragma unroll
      for (int mb = 0; mb < 4; ++mb)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          ok[mb][r] = fexp2(ok[mb][r] + nm);   // unnormalised slot probabilities
          psum += ok[mb][r];
        }
      psum += __shfl_xor(psum, 16, 64);
      psum += __shfl_xor(psum, 32, 64);
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
    }
    // the v-state halves have landed (this wave's part, then everybody's); the v rows behind them may fly
    wait_vm<2 * LPB>();
    lds_barrier();
    // every wave has read the chunk's k_gsa rows: the second chunk's take their buffers now
    const bool ahead = NCH == 2 && cc == 0 && second;
    if (ahead) {
#pragma unroll
      for (int half = 0; half < 2; ++half)
        issue_buffer(half ? oB1 : oB0, false, t_kg, (uint32_t)(H * D), [&](int r) { return tok_from(c0 + BT - p.shift, 32 * half + r); });
    }
    bf16x8 bAv[2];
    if (mine) {
      // slot read, inter-chunk part: O^T[d][i] += sum_m hv[m][d] (p[i][m] exp(gc_i[m]))
#pragma unroll
      for (int pr = 0; pr < 2; ++pr)
#pragma unroll
        for (int db = 0; db < DB; ++db) O[db] = mfma16(vfrag((pr ? oC1 : oC0), db), bp[pr], O[db]);
      // intra-chunk part: AvT[j][i] = sum_m s_j[m] exp(gr[m]-gc_j[m]) (p[i][m] exp(gc_i[m]-gr[m])), j <= i
      f32x4 av[4];
#pragma unroll
      for (int jb = 0; jb < 4; ++jb) {
        av[jb] = (f32x4){0.f, 0.f, 0.f, 0.f};
        if (jb <= Q) {
#pragma unroll
          for (int pr = 0; pr < 2; ++pr) av[jb] = mfma16(etab_row(jb, pr), bpr[pr], av[jb]);
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
    // the v rows have landed (this wave's part, then everybody's); the second chunk's k_gsa rows behind them may fly
    if (ahead) wait_vm<2 * LPB>();
    else wait_vm<0>();
    lds_barrier();
    if (mine) {
#pragma unroll
      for (int pr = 0; pr < 2; ++pr)
        if (2 * pr <= Q) {
#pragma unroll
          for (int db = 0; db < DB; ++db) O[db] = mfma16(vfrag((pr ? oA1 : oA0), db), bAv[pr], O[db]);
        }
    }
  }

  // ---- epilogue: 16-byte stores (the lanes of an even 16-lane row keep block db, those of the odd
  //      row block db + 1, and the two trade their halves) -------------------------------------------
  {
    const float inv = 1.f / (Lw[0] + psum);
    bf16_t* op = p.o + ((int64_t)(c0 + yrow) * HQ + hq) * D;
#pragma unroll
    for (int db = 0; db < DB; db += 2) {
      unsigned a[2], b[2];
      a[0] = cvt2(O[db][0] * inv, O[db][1] * inv);
      a[1] = cvt2(O[db][2] * inv, O[db][3] * inv);
      b[0] = cvt2(O[db + 1][0] * inv, O[db + 1][1] * inv);
      b[1] = cvt2(O[db + 1][2] * inv, O[db + 1][3] * inv);
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

}  // namespace

// Served: K == V == 256 with any grouping of query heads (each head walks its kv-head's window on its
// own).  The per-lane byte offsets of the LDS-direct loads are 32 bits: the tensors of one call must
// stay below 4 GiB.
bool prefill_ring256_supported(const mf::MP& p, int D) {
  if (D != 256) return false;
  return (int64_t)p.T_tot * p.H * D * 2 < ((int64_t)1 << 32) && (int64_t)p.T_tot * p.H * MS * 2 < ((int64_t)1 << 32);
}

int prefill_ring256_launch(const mf::MP& p, hipStream_t st) {
  static std::once_flag once;
  static hipError_t attr_err = hipSuccess;
  std::call_once(once, [&] {
    attr_err = hipFuncSetAttribute((const void*)ring256_out_kernel<2>, hipFuncAttributeMaxDynamicSharedMemorySize, Cfg<2>::BYTES);
    if (attr_err == hipSuccess)
      attr_err = hipFuncSetAttribute((const void*)ring256_out_kernel<1>, hipFuncAttributeMaxDynamicSharedMemorySize, Cfg<1>::BYTES);
  });
  if (attr_err != hipSuccess) {
    set_error("nha_prefill_fwd(mfma): cannot reserve %d bytes of LDS: %s", Cfg<2>::BYTES, hipGetErrorString(attr_err));
    return NHA_ERR_LAUNCH;
  }
  // two chunks per workgroup unless most sequences have a single chunk (fewer than three chunks per two sequences):
  // there the second half of a two-chunk workgroup would mostly idle
  if (2 * (int64_t)p.NT < 3 * (int64_t)p.N)
    hipLaunchKernelGGL(ring256_out_kernel<1>, dim3(p.HQ, p.NT), dim3(256), Cfg<1>::BYTES, st, p);
  else
    hipLaunchKernelGGL(ring256_out_kernel<2>, dim3(p.HQ, p.NT), dim3(512), Cfg<2>::BYTES, st, p);
  NHA_CHECK_LAUNCH("nha_prefill_fwd(mfma output pass, ring, head size 256)");
  return NHA_OK;
}

}  // namespace nha
