// Shared by the matrix-core prefill kernels (prefill_mfma.hip, prefill_ring.hip): vector types,
// LDS helpers, the kernel parameter block and the constants of the chunk algebra.
#pragma once
#include "common.h"

namespace nha {
namespace mf {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef short s16x4 __attribute__((ext_vector_type(4)));

// explicit LDS address space: keeps every tile access a ds_* instruction (never a flat access)
#define NHA_LDS __attribute__((address_space(3)))
typedef NHA_LDS bf16_t lbf16;
typedef NHA_LDS float lfloat;
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ void lds_st16(lbf16* p, uint4 v) { *reinterpret_cast<NHA_LDS u32x4*>(p) = (u32x4){v.x, v.y, v.z, v.w}; }
__device__ __forceinline__ float4 lds_ld_f4(const lfloat* p) {
  const f32x4 v = *reinterpret_cast<const NHA_LDS f32x4*>(p);
  return make_float4(v[0], v[1], v[2], v[3]);
}

constexpr int BT = 64;        // chunk rows == window tile keys
constexpr int MS = 64;        // slots
constexpr int GLD = 68;       // LDS row stride (floats) of the gate-cumsum tables
constexpr int SLD = 72;       // LDS row stride (bf16) of the s tables
constexpr float LOG2E = 1.4426950408889634f;
constexpr float LN2 = 0.6931471805599453f;
// Largest positive decay exponent formed on the MFMA path.  A factor s exp(60) = 1.1e26 still multiplies
// unscaled intra-chunk scores (the layer's default scale is 1) summed over 16 rows with e^28 of fp32
// range to spare; sub-blocks that decay faster are flagged and recomputed exactly.
constexpr float DECAY_CLAMP = 60.f;
// The backward's factored products use one reference per 32-row half of a chunk; the large factor
// s exp(ref - gc_j) <= e^70 = 2.5e30 meets gradient-sized weights there (p (dp - delta), not raw scores), so
// e^18 of fp32 range is enough, and gates drawn as logsigmoid(N(-1, 1)) (32 rows decay by e^-42 +- e^-4.5)
// stay on the matrix-core path; chunks beyond it take the fp32 kernels.
constexpr float BWD_DECAY_CLAMP = 70.f;

struct MP {
  const bf16_t *q_swa, *k_swa, *q_gsa, *k_gsa, *v, *s, *g;
  bf16_t* o;
  float *lse_swa, *lse_gsa;
  const float *h0k, *h0v;
  float *hkt, *hvt;
  const int32_t *cu, *cidx, *coff;
  bf16_t* hkT;   // [NT][H][MS][D]   segment-local chunk-start k-state, transposed ([m][d])
  bf16_t* hvc;   // [NT][H][MS][D]   segment-local chunk-start v-state ([m][d])
  float* gc;     // [NT][H][BT][MS]  chunk-local inclusive gate cumsum
  float* dcum;   // [NT][H][MS]      decay from the segment start to the chunk start
  float *hend_k, *hend_v;   // [NSLOT][H][MS][D]  segment-local end states
  float *hseg_k, *hseg_v;   // [NSLOT][H][MS][D]  true segment-start states
  float* dtot;   // [NSLOT][H][MS]   total decay of a segment
  int* flags;    // [NT][H][4]       per 16-slot block: bit q = sub-block q decays past DECAY_CLAMP
  int T_tot, N, NT, HQ, H, NG, wl, shift;
  int sinks;     // window-only launches (prefill_ring.hip, SINK): zero-logit keys in front of every sequence
  float scale;
};

__device__ __forceinline__ f32x4 mfma16(bf16x8 a, bf16x8 b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ bf16x8 as_bf16x8(uint4 u) { return __builtin_bit_cast(bf16x8, u); }
__device__ __forceinline__ float fexp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fexp(float x) { return __builtin_amdgcn_exp2f(x * LOG2E); }

__device__ __forceinline__ bf16x8 pack8(f32x4 a, f32x4 b) {
  bf16x8 r;
  r[0] = (__bf16)a[0]; r[1] = (__bf16)a[1]; r[2] = (__bf16)a[2]; r[3] = (__bf16)a[3];
  r[4] = (__bf16)b[0]; r[5] = (__bf16)b[1]; r[6] = (__bf16)b[2]; r[7] = (__bf16)b[3];
  return r;
}

// workgroup barrier that orders LDS traffic only: outstanding global loads (tile prefetches) stay
// in flight across it
// Tile of a workgroup in a launch of (kv-heads x groups-per-kv-head, chunks) tiles.  Workgroups are dispatched
// in the order L = y * gridDim.x + x and workgroup L runs on XCD L % 8, each XCD with its own L2: XCD k takes
// the k-th eighth of the tile sequence (kv-head, chunk, group of the kv-head), fastest last, so that what an
// XCD works on at one time is a run of neighbouring chunks of one kv-head, whose windows overlap.  Returns the
// tile's x (kv-head * ngrp + group) and y (chunk slot).
__device__ __forceinline__ void xcd_tile(int ngrp, int nchunks, int& vx, int& vy) {
  const int total = gridDim.x * gridDim.y, per = total >> 3;
  const int L = blockIdx.y * gridDim.x + blockIdx.x;
  // the up to seven workgroups beyond a multiple of 8 take the last tiles of the sequence
  const int v = L < 8 * per ? (L & 7) * per + (L >> 3) : L;
  const int g = v % ngrp, rest = v / ngrp;
  vy = rest % nchunks;
  vx = (rest / nchunks) * ngrp + g;
}

__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// max over the four 16-lane rows of a wave (lanes l, l^16, l^32, l^48), VALU only
__device__ __forceinline__ float max_over_rows(float x) {
  const unsigned u = __float_as_uint(x);
  const auto a = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  x = fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1]));
  const unsigned v = __float_as_uint(x);
  const auto b = __builtin_amdgcn_permlane16_swap(v, v, false, false);
  return fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));
}

// A/B fragment of a row-major LDS tile: 8 consecutive elements of row `row` starting at `col`.
__device__ __forceinline__ bf16x8 lds_frag(const lbf16* tile, int ld, int row, int col) {
  return *reinterpret_cast<const NHA_LDS bf16x8*>(tile + row * ld + col);
}

// Transposed fragment of a row-major [rows][ld] bf16 LDS tile: the lane (c = l%16, kb = l/16)
// receives X[r0a + 4*kb + e][col0 + c] for e = 0..3 and X[r0b + 4*kb + e][col0 + c] for e = 4..7.
__device__ __forceinline__ bf16x8 lds_frag_tr(const lbf16* tile, int ld, int r0a, int r0b, int col0, int lane) {
  const int l16 = lane & 15, kb = lane >> 4;
  const lbf16* pa = tile + (r0a + 4 * kb + (l16 >> 2)) * ld + col0 + 4 * (l16 & 3);
  const lbf16* pb = tile + (r0b + 4 * kb + (l16 >> 2)) * ld + col0 + 4 * (l16 & 3);
  struct { s16x4 a, b; } t;
  t.a = __builtin_amdgcn_ds_read_tr16_b64_v4i16((NHA_LDS s16x4*)pa);
  t.b = __builtin_amdgcn_ds_read_tr16_b64_v4i16((NHA_LDS s16x4*)pb);
  return __builtin_bit_cast(bf16x8, t);
}

// the slot recurrence is cut into segments of SEG chunks (two-level state pass)
constexpr int SEG = 8;

__device__ __forceinline__ int seg_slot(const int32_t* coff, int n, int it) { return coff[n] / SEG + it / SEG + n; }

// decay-factor fragments of the slot branch, built once per workgroup in MFMA operand order
constexpr int NSEA = 24;   // fragments s*decay with rows = slots  (A operand of the logit update)
constexpr int NSEB = 20;   // fragments s*decay with rows = tokens (A operand of the slot-read weights)
__device__ __forceinline__ int sea_base(int Q) { return Q == 0 ? 0 : Q == 1 ? 4 : Q == 2 ? 8 : 16; }
__device__ __forceinline__ int seb_base(int Q) { return Q == 0 ? 0 : Q == 1 ? 2 : Q == 2 ? 6 : 12; }

}  // namespace mf

// output pass with LDS-direct window loads (prefill_ring.hip); false when the shape is not served
bool prefill_ring_supported(const mf::MP& p, int D);
int prefill_ring_launch(const mf::MP& p, int D, hipStream_t st);
// the same for head size 256, one query head per workgroup (prefill_ring256.hip)
bool prefill_ring256_supported(const mf::MP& p, int D);
int prefill_ring256_launch(const mf::MP& p, hipStream_t st);

}  // namespace nha
