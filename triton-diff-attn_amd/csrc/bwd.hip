// Differential-attention backward for gfx950.  Same mathematics as the reference's fused backward
// (src/kernel.py:221-458) but split into stream-ordered kernels, which removes the reference's
// in-launch dependency between the row preprocess and the main loops:
//
//   bwd_prep_kernel   per row: RMSNorm backward (src/kernel.py:283-290), the two row dots
//                     delta1/delta2 (:295-296), d(lambda) partials (:293); writes dX in fp16 and
//                     the four row statistics the main kernels need.
//   bwd_dkdv_kernel   one workgroup per 128 keys, loops over all query tiles:
//                     dV += (P1 - lambda P2)^T dX, dK_t += s dS_t^T Q_t      (:410-424)
//   bwd_dq_kernel     one workgroup per 128 queries, loops over all key tiles:
//                     dQ_t += s dS_t K_t                                      (:426-436)
//   d(lambda)         fixed-order sum of the partials into one fp16 value (one per head with per-head
//                     lambda) (:573): one extra workgroup per value at the end of the first dK/dV or dQ
//                     grid of the call, or bwd_dlambda_kernel when neither of them is launched
//
// The pre-norm row X is rebuilt as Y / ((1 - lambda_init) * rinv); only U2 = softmax(S2) V is
// needed besides it, because U1 = X + lambda U2.
#include <type_traits>

#include "params.hpp"

namespace DA_NS {

constexpr int kPrepRows = 64;   // rows per workgroup of the preprocess kernel = one d(lambda) partial

int bwd_num_partials(int BH, int N, int D) { (void)D; return (int)(((long long)BH * N) / kPrepRows); }

// ------------------------------------------------------------------------------------------------
template <int D, bool RMS>
__global__ __launch_bounds__(256) void bwd_prep_kernel(BwdParams p) {
  constexpr int DV = 2 * D, LPR = DV / 8, RPP = 256 / LPR;
  __shared__ float red[256];
  const int tid = threadIdx.x, sub = tid % LPR, rloc = tid / LPR;
  // the 64 rows of a workgroup belong to one (batch, head) unit: N is a multiple of 128
  const int bh = (int)(((size_t)blockIdx.x * kPrepRows) / p.N);
  const int n0 = (int)(((size_t)blockIdx.x * kPrepRows) % p.N);
  const float lam = da_abi::lambda_of_unit(p, bh);
  const half_t* gy = p.y + da_abi::unit_base(p, p.sy, bh) + 8 * sub;
  const half_t* gdy = p.dy + da_abi::unit_base(p, p.sdy, bh) + 8 * sub;
  const float c = 1.0f - p.lambda_init;
  const size_t rows = (size_t)p.BH * p.N;
  float part = 0.f;
#pragma unroll 1
  for (int pass = 0; pass < kPrepRows / RPP; ++pass) {
    const size_t row = (size_t)blockIdx.x * kPrepRows + pass * RPP + rloc;
    const size_t off = row * DV + 8 * sub;
    const size_t n = (size_t)(n0 + pass * RPP + rloc);
    // a padding row (past the sequence's real length) has no y and dy rows: it gets dX = 0 and zero statistics,
    // so it adds nothing to dK, dV and d(lambda)
    const bool real = n < (size_t)p.n_keys;
    h8 y8, g8;
#pragma unroll
    for (int e = 0; e < 8; ++e) { y8[e] = (half_t)0.f; g8[e] = (half_t)0.f; }
    if (real) {
      y8 = *reinterpret_cast<const h8*>(gy + n * (size_t)p.sy.n);
      g8 = *reinterpret_cast<const h8*>(gdy + n * (size_t)p.sdy.n);
    }
    const h8 u8 = *reinterpret_cast<const h8*>(p.u2 + off);
    // dX of the row, and ix with X = ix * Y (the pre-norm row rebuilt from the saved output)
    float dx[8], ix = 1.0f;
    if (RMS) {
      float gy = 0.f;
#pragma unroll
      for (int e = 0; e < 8; e += 2) gy = dot_pair(h2{g8[e], g8[e + 1]}, h2{y8[e], y8[e + 1]}, gy);
#pragma unroll
      for (int msk = LPR / 2; msk >= 1; msk >>= 1) gy += __shfl_xor(gy, msk, 64);
      const float r = p.rinv[row];
      if (c != 0.f) {
        const float a = c * r, b = r * gy / (c * DV);
        ix = 1.0f / (c * r);
#pragma unroll
        for (int e = 0; e < 8; ++e) dx[e] = a * (float)g8[e] - b * (float)y8[e];
      } else {
        ix = 0.f;
#pragma unroll
        for (int e = 0; e < 8; ++e) dx[e] = 0.f;
      }
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) dx[e] = (float)g8[e];
    }
    // The row sums are formed from dX as the other kernels will read it, rounded to 16 bits: dS = A (dP - delta)
    // with dP = dX V^T cancels almost completely where a row attends to a single key, and a delta from the
    // unrounded dX would leave the rounding error of dX times V behind, scaled by a norm factor that is large
    // exactly in the rows where the two streams nearly cancel.  (The reference takes delta from the unrounded
    // gradient, src/kernel.py:290-296, and dP from the rounded one, :374-375 and :419.)  The products of the
    // 16-bit values are exact and summed in fp32.
    float t2 = 0.f, ty = 0.f;
    h8 d8;
#pragma unroll
    for (int e = 0; e < 8; ++e) d8[e] = (half_t)dx[e];
#pragma unroll
    for (int e = 0; e < 8; e += 2) {
      t2 = dot_pair(h2{d8[e], d8[e + 1]}, h2{u8[e], u8[e + 1]}, t2);
      ty = dot_pair(h2{d8[e], d8[e + 1]}, h2{y8[e], y8[e + 1]}, ty);
    }
#pragma unroll
    for (int msk = LPR / 2; msk >= 1; msk >>= 1) {
      t2 += __shfl_xor(t2, msk, 64);
      ty += __shfl_xor(ty, msk, 64);
    }
    const float tx = ty * ix;      // rowsum(dX * X)
    *reinterpret_cast<h8*>(p.dx + off) = d8;
    if (sub == 0) {
      const float delta2 = -lam * t2;
      p.stat[0 * rows + row] = -p.lse1[row] * kLog2e;
      p.stat[1 * rows + row] = -p.lse2[row] * kLog2e;
      const float delta1 = tx - delta2;
      p.stat[2 * rows + row] = -delta1;
      p.stat[3 * rows + row] = -(lam * delta1 + delta2);
      part -= t2;
    }
  }
  red[tid] = part;
  __syncthreads();
#pragma unroll
  for (int s = 128; s >= 1; s >>= 1) {
    if (tid < s) red[tid] += red[tid + s];
    __syncthreads();
  }
  if (tid == 0) p.dlam_part[blockIdx.x] = red[0];
}

// Output o of n_out is the sum of the partials of the units o, o + n_out, o + 2 n_out, ...: with n_out = 1
// every unit (one lambda), with n_out = H the units of head o (one lambda per head).  `per_unit`
// consecutive partials belong to a unit.  One workgroup per output.  The sum is formed over 256 slots and a
// binary tree in a fixed order; a workgroup of fewer threads lets each thread play several slots, so the
// result does not depend on the kernel that hosts the reduction.
__device__ __forceinline__ void dlambda_reduce(const float* __restrict__ part, int per_unit, int n_units, half_t* out,
                                               int o, int n_out, float* red, int out_fp32) {
  const int tid = threadIdx.x, nt = blockDim.x;
  const int n = (n_units / n_out) * per_unit;        // partials this workgroup sums
  for (int slot = tid; slot < 256; slot += nt) {
    float acc = 0.f;
    if (n_out == 1) {
      for (int i = slot; i < n; i += 256) acc += part[i];
    } else {
      for (int i = slot; i < n; i += 256) acc += part[(size_t)(o + (i / per_unit) * n_out) * per_unit + i % per_unit];
    }
    red[slot] = acc;
  }
  __syncthreads();
#pragma unroll
  for (int s = 128; s >= 1; s >>= 1) {
    for (int slot = tid; slot < s; slot += nt) red[slot] += red[slot + s];
    __syncthreads();
  }
  if (tid == 0) {
    // the sum leaves the library in the 16-bit type of the tensors, like the reference's (src/kernel.py:573),
    // or unrounded in fp32 when the caller keeps lambda in fp32
    if (out_fp32) reinterpret_cast<float*>(out)[o] = red[0];
    else out[o] = (half_t)red[0];
  }
}

__global__ __launch_bounds__(256) void bwd_dlambda_kernel(const float* __restrict__ part, int per_unit, int n_units,
                                                          half_t* out, int out_fp32) {
  __shared__ float red[256];
  dlambda_reduce(part, per_unit, n_units, out, blockIdx.x, gridDim.x, red, out_fp32);
}

// The dK/dV and dQ kernels can host that reduction in p.dlam_fold extra workgroups at the end of their grid
// (one launch less per backward): such a workgroup does nothing else.
#define DA_HOST_DLAMBDA(smem_)                                                                                  \
  if (p.dlam_fold && (int)blockIdx.x >= (int)gridDim.x - p.dlam_fold) {                                         \
    dlambda_reduce(p.dlam_part, p.n_part / p.BH, p.BH, p.dlambda, (int)blockIdx.x - ((int)gridDim.x - p.dlam_fold), \
                   p.dlam_fold, reinterpret_cast<float*>(smem_), p.lambda_fp32);                                \
    return;                                                                                                     \
  }

// ------------------------------------------------------------------------------------------------
template <int D, int NWAVES = 4>
struct DkvCfg {
  static constexpr int DV = 2 * D;
  static constexpr int NW = NWAVES;            // waves per workgroup, 32 keys each (2: half-size key blocks for small grids)
  static constexpr int NT = NW * 64;
  static constexpr int BK = NW * 32;           // keys per workgroup
  static constexpr int BQ = (D <= 64) ? 64 : 32;  // query rows per staged tile
  static constexpr int Q_TILE = BQ * D;        // halfs (swizzled, unpadded)
  static constexpr int X_TILE = BQ * DV;
  static constexpr int STAT = 4 * BQ * 2;      // 4 float arrays, counted in halfs
  static constexpr int STAGE = 2 * Q_TILE + X_TILE + STAT;
  // LDS map in bytes: the ring buffers of each kind of tile are contiguous, so that any buffer of a kind
  // is within the 64 KiB reach of an LDS instruction's immediate offset from one per-lane address
  static constexpr int QBUF = 2 * Q_TILE * 2, XBUF = X_TILE * 2, SBUF = STAT * 2;   // one ring buffer of Q1|Q2, dX, statistics
  // A staged tile is read until half a step after its last sub-tile was scored while the tile after
  // the next is already being fetched, which takes three buffers; there are four so that the ring
  // position of every step is known at compile time (the loop is unrolled over one turn of the ring,
  // and the number of steps is a multiple of four): every LDS address is then a per-lane register
  // plus an immediate offset, with no address arithmetic inside the loop.
  static constexpr int NBUF = 4;
  static constexpr int XBASE = NBUF * QBUF, SBASE = XBASE + NBUF * XBUF;
  static_assert(NBUF * QBUF <= 65536 && NBUF * XBUF <= 65536, "immediate offsets reach every buffer");
};

// dK_t and dV for one block of keys.  Products are formed as [queries x keys] so that a lane owns
// one key column; P and dS in accumulator layout are then directly the A operands (rows = keys,
// contraction over queries) of dV = P^T dX and dK_t = dS_t^T Q_t.
// MODE 0 computes dV, dK1 and dK2 in one pass.  At D = 128 their accumulators plus the resident
// K1, K2, V rows exceed the 512 registers of a lane, so the work is split in two launches:
// MODE 1 computes dV only (scores S1, S2; no dP), MODE 2 computes dK1 and dK2 only.
// CAUSAL: queries before the key block are skipped and the four sub-tiles on the diagonal are masked.
// DROP: dropout on both softmax maps, masks regenerated from the hash the forward used.  With the
// keep mask m_t and c = 1/(1-p):  dS1 = A1 (c m1 dP - delta1),  dS2 = A2 (-lambda c m2 dP - delta2),
// dV = c (m1 A1 - lambda m2 A2)^T dX; delta1, delta2 are the row dots with the dropped-out U1, U2.
// PADDED: rows n_keys..N-1 are padding.  As queries they read the last real row of Q1 and Q2 (the row the
// forward used for their logsumexp) and carry dX = 0; as keys they read the last real row of K1, K2, V and
// their results are not stored.
template <int D, int MODE, bool CAUSAL, bool DROP, bool PADDED, int NWAVES = 4>
__global__ __launch_bounds__((DkvCfg<D, NWAVES>::NT)) __attribute__((amdgpu_waves_per_eu(1, 1))) void bwd_dkdv_kernel(BwdParams p) {
  using C = DkvCfg<D, NWAVES>;
  constexpr int DV = C::DV, NW = C::NW, BK = C::BK, BQ = C::BQ;
  constexpr int NKS = D / 16, NKV = DV / 16, NDT = D / 32, NVT = DV / 32;
  constexpr bool DO_V = (MODE != 2), DO_K = (MODE != 1);

  __shared__ __attribute__((aligned(16))) half_t smem[C::NBUF * C::STAGE];
  static_assert(sizeof(smem) >= 256 * sizeof(float), "the hosted reduction uses the tile memory");
  DA_HOST_DLAMBDA(smem)

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int j = lane & 31, g = lane >> 5;

  const int n_kt = p.N / BK;
  int bh, kt;
  if constexpr (CAUSAL) {   // the first key block of a unit is seen by the most queries
    const UnitBlock ub = longest_first(blockIdx.x, p.BH);
    bh = ub.unit; kt = ub.rank;
  } else {
    const int tile = xcd_remap(blockIdx.x, gridDim.x - p.dlam_fold);
    bh = tile / n_kt; kt = tile % n_kt;
  }
  const size_t rows = (size_t)p.BH * p.N;
  const size_t row0 = (size_t)bh * p.N;
  const int key = kt * BK + wave * 32 + j;
  const int key_row = (PADDED && key >= p.n_keys) ? p.n_keys - 1 : key;    // the row this lane's key is read from
  // element offsets of the unit's first row and the row strides of the strided tensors
  const size_t qk_base = da_abi::unit_base(p, p.sqk, bh), v_base = da_abi::unit_base(p, p.sv, bh);
  const int qk_n = (int)p.sqk.n, v_n = (int)p.sv.n;

  const float c = p.sm_scale * kLog2e;
  const float lam = da_abi::lambda_of_unit(p, bh);
  // hash keys of this unit's two softmax streams (used with dropout only)
  const DropoutKey dkey1 = dropout_key(p.drop, 2u * bh), dkey2 = dropout_key(p.drop, 2u * bh + 1);

  // persistent B operands: this lane's key row of K1, K2, V
  h8 kf1[NKS], kf2[NKS], vf[NKV];
  {
    const half_t* r1 = p.k1 + qk_base + (size_t)key_row * qk_n + 8 * g;
    const half_t* r2 = p.k2 + qk_base + (size_t)key_row * qk_n + 8 * g;
    const half_t* rv = p.v + v_base + (size_t)key_row * v_n + 8 * g;
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) {
      // pre-multiplied by sm_scale*log2(e): the score products come out in log2 units
      h8 x1 = *reinterpret_cast<const h8*>(r1 + 16 * ks);
      h8 x2 = *reinterpret_cast<const h8*>(r2 + 16 * ks);
#pragma unroll
      for (int e = 0; e < 8; ++e) { x1[e] = (half_t)((float)x1[e] * c); x2[e] = (half_t)((float)x2[e] * c); }
      kf1[ks] = x1; kf2[ks] = x2;
    }
    if constexpr (DO_K) {
#pragma unroll
      for (int kv = 0; kv < NKV; ++kv) vf[kv] = *reinterpret_cast<const h8*>(rv + 16 * kv);
    }
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) { keep_in_agpr(kf1[ks]); keep_in_agpr(kf2[ks]); }
    if constexpr (DO_K) {
#pragma unroll
      for (int kv = 0; kv < NKV; ++kv) keep_in_agpr(vf[kv]);
    }
  }

  f16v dv[NVT], dk1[NDT], dk2[NDT];
#pragma unroll
  for (int t = 0; t < NVT; ++t)
#pragma unroll
    for (int r = 0; r < 16; ++r) dv[t][r] = 0.f;
#pragma unroll
  for (int t = 0; t < NDT; ++t)
#pragma unroll
    for (int r = 0; r < 16; ++r) { dk1[t][r] = 0.f; dk2[t][r] = 0.f; }

  using QTile = AsyncTile<BQ, D, NW>;
  using XTile = AsyncTile<BQ, DV, NW>;
  const half_t* gq1 = p.q1 + qk_base;
  const half_t* gq2 = p.q2 + qk_base;
  const half_t* gx = p.dx + row0 * DV;
  const unsigned q_off = QTile::lane_off(wave, lane, qk_n);
  // the 4 x BQ statistics of a query tile are one piece of 16*BQ bytes: lane l < BQ fetches
  // stat[l / (BQ/4)][4 * (l % (BQ/4)) .. +3]
  const float* gstat = p.stat + row0;
  const unsigned stat_off = (unsigned)(((size_t)(lane / (BQ / 4)) * rows + 4 * (lane % (BQ / 4))) * sizeof(float));
  constexpr int XH = (XTile::PER + 1) / 2;

  auto stage = [&](int qt, int buf, int part) {
    half_t* bq = smem + buf * (C::QBUF / 2);
    half_t* bx = smem + (C::XBASE + buf * C::XBUF) / 2;
    // dX and the statistics come from the workspace, which has all N rows; Q1 and Q2 have n_keys
    const bool past_end = PADDED && (qt + 1) * BQ > p.n_keys;
    if (part == 0) {
      if (past_end) QTile::issue_clamped(gq1 + (size_t)qt * BQ * qk_n, bq, wave, lane, q_off, qk_n, p.n_keys - 1 - qt * BQ);
      else QTile::issue_at(gq1 + (size_t)qt * BQ * qk_n, bq, wave, lane, q_off, qk_n);
      if (wave == 0 && lane < BQ) async_copy16(reinterpret_cast<const half_t*>(gstat + (size_t)qt * BQ), stat_off, smem + (C::SBASE + buf * C::SBUF) / 2);
    } else if (part == 1) {
      if (past_end) QTile::issue_clamped(gq2 + (size_t)qt * BQ * qk_n, bq + C::Q_TILE, wave, lane, q_off, qk_n, p.n_keys - 1 - qt * BQ);
      else QTile::issue_at(gq2 + (size_t)qt * BQ * qk_n, bq + C::Q_TILE, wave, lane, q_off, qk_n);
    } else if (part == 2) {
      XTile::template issue<0, XH>(gx + (size_t)qt * BQ * DV, bx, wave, lane);
    } else {
      XTile::template issue<XH, XTile::PER>(gx + (size_t)qt * BQ * DV, bx, wave, lane);
    }
  };

  const int tr_row = 4 * g + ((lane & 15) >> 2);  // transposing reads: row inside a 16-row k-step
  const int tr_col = 16 * ((lane >> 4) & 1) + 4 * (lane & 3);

  // Per-lane LDS byte addresses, computed once.  The XOR swizzle makes the address of a fragment a
  // different function of the lane for every 16-byte chunk column, so there is one register per chunk
  // column a lane ever reads; everything else (ring buffer, Q1 or Q2, sub-tile, k-step of 16 rows) is a
  // multiple of 16 rows, which the swizzle does not see, and travels in the instruction's immediate offset.
  const unsigned lds0 = (unsigned)(unsigned long)((DA_LDS char*)smem);
  unsigned qb[NKS], xb[NKV], qtr[NDT][2], xtr[NVT][2], stb;
#pragma unroll
  for (int ks = 0; ks < NKS; ++ks) qb[ks] = lds0 + 2u * (unsigned)swz_off<D>(j, 16 * ks + 8 * g);
#pragma unroll
  for (int kv = 0; kv < NKV; ++kv) xb[kv] = lds0 + C::XBASE + 2u * (unsigned)swz_off<DV>(j, 16 * kv + 8 * g);
#pragma unroll
  for (int tt = 0; tt < NDT; ++tt)
#pragma unroll
    for (int e = 0; e < 2; ++e) qtr[tt][e] = lds0 + 2u * (unsigned)swz_off<D>(tr_row + 8 * e, 32 * tt + tr_col);
#pragma unroll
  for (int tt = 0; tt < NVT; ++tt)
#pragma unroll
    for (int e = 0; e < 2; ++e) xtr[tt][e] = lds0 + C::XBASE + 2u * (unsigned)swz_off<DV>(tr_row + 8 * e, 32 * tt + tr_col);
  stb = lds0 + C::SBASE + 16u * (unsigned)g;
  // kept as they are: the compiler neither folds constants into them nor recomputes them in the loop
#pragma unroll
  for (int ks = 0; ks < NKS; ++ks) asm volatile("" : "+v"(qb[ks]));
#pragma unroll
  for (int kv = 0; kv < NKV; ++kv) asm volatile("" : "+v"(xb[kv]));
#pragma unroll
  for (int tt = 0; tt < NDT; ++tt) asm volatile("" : "+v"(qtr[tt][0]), "+v"(qtr[tt][1]));
#pragma unroll
  for (int tt = 0; tt < NVT; ++tt) asm volatile("" : "+v"(xtr[tt][0]), "+v"(xtr[tt][1]));
  asm volatile("" : "+v"(stb));
  auto lds_h8 = [](unsigned addr, int off) -> h8 { return lds_read_at<h8>(addr, off); };
  auto lds_tr = [](unsigned addr, int off) -> h4 { return lds_read_tr_at(addr, off); };

  // The loop runs over 32-query sub-tiles i (SPT per staged tile), software-pipelined inside the
  // wave.  Step i interleaves, instruction group by instruction group,
  //   the matrix products S1, S2, dP of sub-tile i+1          (matrix unit, A fragments from LDS)
  //   the element-wise work of sub-tile i, one register row at a time          (VALU)
  //   the products dV, dK1, dK2 over queries 16..31 of sub-tile i-1 during the first half of the
  //   step and over queries 0..15 of sub-tile i during the second half, as soon as the
  //   element-wise work has packed their operands              (matrix unit, B fragments from LDS)
  // The interleaving is written out in source order and pinned with scheduling barriers, because
  // the matrix products with AGPR-resident B fragments are opaque to the instruction scheduler.
  constexpr int SPT = BQ / 32;
  struct Scores { f16v s1, s2, dp; };
  struct Packed { h8 pc[2], d1[2], d2[2]; };   // A operands of the dV / dK1 / dK2 products
  constexpr int NPROD = 2 * NKS + (DO_K ? NKV : 0);   // score products per sub-tile (dP is needed for dK only)
  // the D = 128 instantiations with dropout are short of registers: they request one fragment ahead
  constexpr bool kShort = DROP && D == 128;
  // A fragments requested ahead of their product (measured in one GPU call: 4 is 1 % faster than 3 at D = 64 and
  // D = 128 and the same at D = 32; 5 and 6 spill in some instantiations and are not faster)
  constexpr int DEPTH = kShort ? 1 : 4;

  // Product k of a sub-tile: even k is k-step k/2 of dP, odd k alternates k-steps of S1 and S2, so
  // the three accumulation chains advance together; without dP (MODE 1) S1 and S2 alternate.
  static_assert(NKV == 2 * NKS, "every second product belongs to dP");
  auto prod_frag = [&](int buf, int qs, int k) -> h8 {
    if (!DO_K || (k & 1)) {
      const int t = DO_K ? (k >> 1) : k;
      return lds_h8(qb[t >> 1], buf * C::QBUF + (t & 1) * C::Q_TILE * 2 + qs * 32 * D * 2);
    }
    return lds_h8(xb[k >> 1], buf * C::XBUF + qs * 32 * DV * 2);
  };
  // The products read their resident operand from AGPRs through the inline-assembly form, for which the
  // compiler places no wait states: nothing may be spilled (a reloaded operand directly in front of such a
  // product would be read too early; the build checks that no backward kernel uses scratch memory) and no
  // VALU instruction may write an operand right in front of one (an assembly scan in the tests checks that).
  // The dropout instantiations, whose mask arithmetic makes the compiler shuffle operands, issue ordinary
  // (compiler-visible) matrix instructions instead: the compiler then places every wait state itself.
  auto prod_mfma = [&](int k, h8 a, Scores& out) {
    if (!DO_K || (k & 1)) {
      const int t = DO_K ? (k >> 1) : k, ks = t >> 1;
      if (t & 1) out.s2 = DROP ? mfma32(a, kf2[ks], out.s2) : mfma32_bagpr(a, kf2[ks], out.s2);
      else       out.s1 = DROP ? mfma32(a, kf1[ks], out.s1) : mfma32_bagpr(a, kf1[ks], out.s1);
    } else {
      out.dp = DROP ? mfma32(a, vf[k >> 1], out.dp) : mfma32_bagpr(a, vf[k >> 1], out.dp);
    }
  };
  // Row statistics written by the preprocess kernel: 0: -lse1*log2e, 1: -lse2*log2e, 2: -delta1,
  // 3: -(lambda*delta1 + delta2).  Statistics 0..2 are the initial accumulator values of the three
  // product chains, so the matrix unit delivers s1 - lse1, s2 - lse2 (log2 units) and dP - delta1.
  auto stat4 = [&](int buf, int qs, int which, int r4) -> f4v {
    return lds_read_at<f4v>(stb, buf * C::SBUF + (which * BQ + qs * 32 + 8 * r4) * 4);
  };
  auto results_ready = [&](Scores& s) {
    if constexpr (DO_K) mfma_results_ready(s.s1, s.s2, s.dp);
    else mfma_results_ready(s.s1, s.s2);
  };
  auto init_scores = [&](int buf, int qs, Scores& out) {
#pragma unroll
    for (int r4 = 0; r4 < 4; ++r4) {
      const f4v a = stat4(buf, qs, 0, r4), bq = stat4(buf, qs, 1, r4);
#pragma unroll
      for (int e = 0; e < 4; ++e) { out.s1[4 * r4 + e] = a[e]; out.s2[4 * r4 + e] = bq[e]; }
      if constexpr (DO_K) {
        // with dropout the mask applies to dP alone, so -delta1 cannot ride in the accumulator
        const f4v cq = DROP ? f4v{0.f, 0.f, 0.f, 0.f} : stat4(buf, qs, 2, r4);
#pragma unroll
        for (int e = 0; e < 4; ++e) out.dp[4 * r4 + e] = cq[e];
      }
    }
  };
  // Element-wise work of accumulator register r (query row 8*(r/4) + 4g + (r%4)), split in three
  // stages that are issued one product apart, so that no VALU instruction waits on the one
  // before it: (1) exponentials, (2) products, (3) fp16 packing of a pair of rows.
  struct RowTmp { float p1[16], p2[16], u[16], ds1[16], ds2[16], pc[16], a1[16], k1[16], k2[16]; unsigned w1, w2, w1b, w2b; };
  // `rel` (masked steps only) = key index minus the query index of register 0 of the sub-tile:
  // register r holds query 8*(r/4) + (r%4) relative to that, and a query before its key sees nothing
  auto ew1 = [&](int r, const f4v& st3, const f4v& st2, const Scores& in, RowTmp& t, auto masked_tag, int rel, int qbase) {
    t.p1[r] = fast_exp2(in.s1[r]);
    t.p2[r] = fast_exp2(in.s2[r]);
    if constexpr (decltype(masked_tag)::value) {
      if (8 * (r / 4) + (r % 4) < rel) { t.p1[r] = 0.f; t.p2[r] = 0.f; }
    }
    if constexpr (DROP) {
      // register r holds query qbase + 8*(r/4) + (r%4) of this lane's key; registers r, r+1 (r even)
      // share the hash words of their 2x2 block, one word per softmax stream
      const unsigned query = (unsigned)(qbase + 8 * (r / 4) + (r % 4));
      // the blocks of registers r..r+1 and r+2..r+3 (r a multiple of 4) are neighbours, hashed one by each
      // lane of a key pair
      if ((r & 3) == 0) {
        const unsigned odd = (unsigned)key & 1u;
        dropout_words_shared(dropout_word(dkey1, (unsigned)p.N / 2, (query >> 1) + odd, (unsigned)key >> 1), odd, t.w1, t.w1b);
        dropout_words_shared(dropout_word(dkey2, (unsigned)p.N / 2, (query >> 1) + odd, (unsigned)key >> 1), odd, t.w2, t.w2b);
      }
      const bool keep1 = dropout_keep((r & 2) ? t.w1b : t.w1, query, (unsigned)key, p.drop.threshold);
      const bool keep2 = dropout_keep((r & 2) ? t.w2b : t.w2, query, (unsigned)key, p.drop.threshold);
      t.k1[r] = keep1 ? t.p1[r] : 0.f;
      t.k2[r] = keep2 ? t.p2[r] : 0.f;
      if constexpr (DO_K) {
        const float dpc = p.drop.keep_scale * in.dp[r];
        t.a1[r] = (keep1 ? dpc : 0.f) + st2[r % 4];                       // c m1 dP - delta1
        // -delta2 = statistic 3 - lambda * statistic 2
        t.u[r] = __builtin_fmaf(-lam, keep2 ? dpc : 0.f, __builtin_fmaf(-lam, st2[r % 4], st3[r % 4]));
      }
      return;
    }
    if constexpr (DO_K) {
      t.u[r] = __builtin_fmaf(-lam, in.dp[r], st3[r % 4]);
      asm volatile("" : "+v"(t.p1[r]), "+v"(t.p2[r]), "+v"(t.u[r]));   // computed here, not moved to its use
    } else {
      asm volatile("" : "+v"(t.p1[r]), "+v"(t.p2[r]));
    }
  };
  auto ew2 = [&](int r, const Scores& in, RowTmp& t) {
    if constexpr (DROP) {
      if constexpr (DO_K) {
        t.ds1[r] = t.p1[r] * t.a1[r];
        t.ds2[r] = t.p2[r] * t.u[r];
      }
      if constexpr (DO_V) t.pc[r] = p.drop.keep_scale * __builtin_fmaf(-lam, t.k2[r], t.k1[r]);
      return;
    }
    if constexpr (DO_K) {
      t.ds1[r] = t.p1[r] * in.dp[r];
      t.ds2[r] = t.p2[r] * t.u[r];
    }
    if constexpr (DO_V) t.pc[r] = __builtin_fmaf(-lam, t.p2[r], t.p1[r]);
    if constexpr (DO_K && DO_V) asm volatile("" : "+v"(t.ds1[r]), "+v"(t.ds2[r]), "+v"(t.pc[r]));
    else if constexpr (DO_K) asm volatile("" : "+v"(t.ds1[r]), "+v"(t.ds2[r]));
    else asm volatile("" : "+v"(t.pc[r]));
  };
  auto ew3 = [&](int r, const RowTmp& t, Packed& out) {   // r odd: packs rows r-1 and r
    if constexpr (DO_V) { out.pc[r / 8][r % 8 - 1] = (half_t)t.pc[r - 1]; out.pc[r / 8][r % 8] = (half_t)t.pc[r]; }
    if constexpr (DO_K) {
      out.d1[r / 8][r % 8 - 1] = (half_t)t.ds1[r - 1]; out.d1[r / 8][r % 8] = (half_t)t.ds1[r];
      out.d2[r / 8][r % 8 - 1] = (half_t)t.ds2[r - 1]; out.d2[r / 8][r % 8] = (half_t)t.ds2[r];
    }
  };
  // slot s of the skewed schedule: stage 1 of row s, stage 2 of row s-1, stage 3 of the pair ending at row s-2
  auto ew_slot = [&](int s, const f4v (&st)[4], const f4v (&st2)[4], const Scores& in, RowTmp& t, Packed& out, auto masked_tag,
                     int rel, int qbase) {
    if (s < 16) ew1(s, st[s / 4], st2[s / 4], in, t, masked_tag, rel, qbase);
    if (s >= 1 && s - 1 < 16) ew2(s - 1, in, t);
    if (s >= 2 && s - 2 < 16 && ((s - 2) & 1)) ew3(s - 2, t, out);
  };
  // B fragment (transposing read) of accumulate product m of sub-tile qs: m = kk*NACC1 + slot, where
  // the slots of a 16-query k-step are the dV feature tiles followed by the dK1/dK2 feature tiles
  constexpr int NSV = DO_V ? NVT : 0;          // dV slots
  constexpr int NACC1 = NSV + (DO_K ? 2 * NDT : 0);
  constexpr int NACC = 2 * NACC1;
  static_assert(NPROD % NACC == 0, "a whole number of score products per accumulate product");
  constexpr int RATIO = NPROD / NACC;
  auto acc_frag = [&](int buf, int qs, int m) -> h8 {
    const int kk = m / NACC1, slot = m % NACC1;
    const int row0 = qs * 32 + 16 * kk;
    if (slot < NSV) {
      const int off = buf * C::XBUF + row0 * DV * 2;
      return join(lds_tr(xtr[slot][0], off), lds_tr(xtr[slot][1], off));
    }
    const int t2 = slot - NSV;
    const int off = buf * C::QBUF + (t2 & 1) * C::Q_TILE * 2 + row0 * D * 2;
    return join(lds_tr(qtr[t2 >> 1][0], off), lds_tr(qtr[t2 >> 1][1], off));
  };
  auto acc_mfma = [&](int m, h8 bfrag, const Packed& in) {
    const int kk = m / NACC1, slot = m % NACC1;
    if (slot < NSV) { dv[slot] = mfma32(in.pc[kk], bfrag, dv[slot]); return; }
    const int t2 = slot - NSV;
    if (t2 & 1) dk2[t2 >> 1] = mfma32(in.d2[kk], bfrag, dk2[t2 >> 1]);
    else        dk1[t2 >> 1] = mfma32(in.d1[kk], bfrag, dk1[t2 >> 1]);
  };

  const int n_qt = p.N / BQ;
  const int n_sub = p.N / 32;
  // first sub-tile and tile of the loop: with the causal mask no query before the key block matters
  const int i0 = CAUSAL ? kt * (BK / 32) : 0;
  const int t0 = i0 / SPT;
  // Tile t0 + k lives in buffer k % NBUF.  Step number s of the loop (sub-tile i0 + s) is at ring
  // position s % RING; the positions of its three sub-tiles follow from that at compile time.
  constexpr int NBUF = C::NBUF, RING = SPT * NBUF, HALF = RING / 2;
  static_assert(HALF % 2 == 0 && 4 % HALF == 0, "half a turn is an even number of steps and divides the step count");

  // One step.  Chunk k holds score product k of sub-tile (bufn, qsn), every RATIO-th chunk also
  // accumulate product (k/RATIO + NACC/2) % NACC -- the upper query half of sub-tile (bufp, qsp)
  // during the first half of the step, then the lower query half of sub-tile (bufc, qsc) -- and
  // every chunk its share of the element-wise rows of sub-tile (bufc, qsc).  `pk` holds the packed operands: its lower half is written during the first half
  // of the step and read during the second, its upper half is written during the second half and
  // read during the first half of the next step.
  static_assert(NPROD % 16 == 0 || 16 % NPROD == 0, "rows are spread evenly over the products");
  constexpr int AHEAD = kShort ? 1 : 3;        // B fragments requested ahead of their product (4: no faster)
  auto fused = [&](int bufn, int qsn, Scores& s_nxt, int bufc, int qsc, const Scores& s_cur, Packed& pk,
                   int bufp, int qsp, int tile_next, auto buf_next_tag, auto fetch_tag, auto masked_tag, int rel, int qbase) {
    constexpr int buf_next = decltype(buf_next_tag)::value;
    constexpr bool fetch = decltype(fetch_tag)::value;
    constexpr int NSLOT = 18;                  // 16 rows + 2 slots of pipeline drain
    constexpr int LEAD = 2;                    // slots run before the first product
    // rows 0..7 are packed by slot 9, which must precede the first product that reads them
    static_assert(LEAD + (NSLOT - LEAD) * (NPROD / 2) / NPROD > 9, "lower half packed before it is read");
    auto bfrag = [&](int ja) -> h8 {
      const int m = (ja + NACC / 2) % NACC;
      return (ja < NACC / 2) ? acc_frag(bufp, qsp, m) : acc_frag(bufc, qsc, m);
    };
    h8 a[NPROD], bf[NACC];
    f4v st[4], st2[4];
    RowTmp tmp;
    init_scores(bufn, qsn, s_nxt);
#pragma unroll
    for (int k = 0; k < DEPTH; ++k) a[k] = prod_frag(bufn, qsn, k);
    if constexpr (DO_K) st[0] = stat4(bufc, qsc, 3, 0);
    if constexpr (DO_K && DROP) {
#pragma unroll
      for (int r4 = 0; r4 < 4; ++r4) st2[r4] = stat4(bufc, qsc, 2, r4);
    }
#pragma unroll
    for (int k = 0; k < AHEAD; ++k) bf[k] = bfrag(k);
    // the first slots run while the initial accumulator values and the first fragments arrive
#pragma unroll
    for (int s = 0; s < LEAD; ++s) ew_slot(s, st, st2, s_cur, tmp, pk, masked_tag, rel, qbase);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int k = 0; k < NPROD; ++k) {
      if (k + DEPTH < NPROD) a[k + DEPTH] = prod_frag(bufn, qsn, k + DEPTH);
      if (k % RATIO == 0 && k / RATIO + AHEAD < NACC) bf[k / RATIO + AHEAD] = bfrag(k / RATIO + AHEAD);
      // statistics of the next row group, requested a quarter of a step ahead of their use
      if (DO_K && k % (NPROD / 4) == 0 && k / (NPROD / 4) < 3) st[k / (NPROD / 4) + 1] = stat4(bufc, qsc, 3, k / (NPROD / 4) + 1);
      // the next tile's fetch is spread over the products so that the waves do not queue up at the memory pipeline
      if (fetch && k % (NPROD / 4) == 1) stage(tile_next, buf_next, k / (NPROD / 4));
      prod_mfma(k, a[k], s_nxt);
      if (k % RATIO == 0) acc_mfma((k / RATIO + NACC / 2) % NACC, bf[k / RATIO], pk);
      // slots LEAD .. NSLOT-1 spread over the products
      const int s0 = LEAD + (NSLOT - LEAD) * k / NPROD, s1 = LEAD + (NSLOT - LEAD) * (k + 1) / NPROD;
#pragma unroll
      for (int s = s0; s < s1; ++s) ew_slot(s, st, st2, s_cur, tmp, pk, masked_tag, rel, qbase);
      __builtin_amdgcn_sched_barrier(0);
    }
    // the next step's VALU reads these results right away
    results_ready(s_nxt);
  };

  // step i at ring position POS: sub-tile i+1 is scored, sub-tile i gets its element-wise work, and the
  // accumulate products run over the upper half of sub-tile i-1 and the lower half of sub-tile i
  auto step = [&](int i, auto pos_tag, const Scores& s_cur, Scores& s_nxt, Packed& pk, auto masked_tag) {
    constexpr int POS = decltype(pos_tag)::value;
    constexpr int SUBN = (POS + 1) % SPT, SUBC = POS % SPT, SUBP = (POS + RING - 1) % SPT;
    constexpr int BUFN = ((POS + 1) / SPT) % NBUF, BUFC = POS / SPT, BUFP = ((POS + RING - 1) / SPT) % NBUF;
    constexpr bool opens = (SUBN == 0);
    const int tn = (i + 1) / SPT;
    if constexpr (opens) {
      // sub-tile i+1 opens tile tn: its data must have landed; tile tn+1 is fetched during this step
      wait_async_tiles();
      __syncthreads();
    }
    // Past the end the last tile is fetched and scored again and the result is never used.  In front of
    // the first sub-tile the all-zero upper operand half is accumulated against the zero-filled last buffer.
    const int tl = (tn + 1 < n_qt) ? tn + 1 : n_qt - 1;
    fused(BUFN, SUBN, s_nxt, BUFC, SUBC, s_cur, pk, BUFP, SUBP, tl, std::integral_constant<int, (BUFN + 1) % NBUF>{},
          std::integral_constant<bool, opens>{}, masked_tag, key - 32 * i - 4 * g, 32 * i + 4 * g);
  };

  // prologue: the last buffer, which the first step reads as "the sub-tile before the first", is cleared
  // (uninitialised LDS could hold NaN patterns, and 0 * NaN would poison the sums); the first tile is
  // fetched, then the second starts; scores of the first sub-tile
  const bool head_half = (HALF == 4) && (((n_sub - i0) / HALF) & 1);   // with HALF == 2 the steps are whole turns
  const int b0 = head_half ? NBUF / 2 : 0;          // buffer of the first tile
  {
    const int bz = (b0 + NBUF - 1) % NBUF;          // the buffer in front of the first tile's
    u32x4* zq = reinterpret_cast<u32x4*>(smem + bz * (C::QBUF / 2));
    u32x4* zx = reinterpret_cast<u32x4*>(smem + (C::XBASE + bz * C::XBUF) / 2);
    for (int k = tid; k < C::QBUF / 16; k += C::NT) zq[k] = u32x4{0u, 0u, 0u, 0u};
    for (int k = tid; k < C::XBUF / 16; k += C::NT) zx[k] = u32x4{0u, 0u, 0u, 0u};
  }
  stage(t0, b0, 0); stage(t0, b0, 1); stage(t0, b0, 2); stage(t0, b0, 3);
  wait_async_tiles();
  __syncthreads();
  {
    const int t1 = (t0 + 1 < n_qt) ? t0 + 1 : t0;
    stage(t1, b0 + 1, 0); stage(t1, b0 + 1, 1); stage(t1, b0 + 1, 2); stage(t1, b0 + 1, 3);
  }
  Scores sa, sb;
  Packed pk;
#pragma unroll
  for (int kk = 0; kk < 2; ++kk)
#pragma unroll
    for (int e = 0; e < 8; ++e) { pk.pc[kk][e] = (half_t)0.f; pk.d1[kk][e] = (half_t)0.f; pk.d2[kk][e] = (half_t)0.f; }
  if (head_half) {
    init_scores(NBUF / 2, 0, sa);
#pragma unroll
    for (int k = 0; k < NPROD; ++k) prod_mfma(k, prod_frag(NBUF / 2, 0, k), sa);
  } else {
    init_scores(0, 0, sa);
#pragma unroll
    for (int k = 0; k < NPROD; ++k) prod_mfma(k, prod_frag(0, 0, k), sa);
  }
  results_ready(sa);

  // two steps, starting at the even ring position P0 with the scores of sub-tile i in sa
  auto two_steps = [&](int i, auto p0_tag, auto masked_tag) {
    constexpr int P0 = decltype(p0_tag)::value;
    step(i, std::integral_constant<int, P0>{}, sa, sb, pk, masked_tag);
    step(i + 1, std::integral_constant<int, P0 + 1>{}, sb, sa, pk, masked_tag);
  };
  auto half_turn = [&](int i, auto h0_tag, auto masked_tag) {
    constexpr int H0 = decltype(h0_tag)::value;
    two_steps(i, std::integral_constant<int, H0>{}, masked_tag);
    if constexpr (HALF == 4) two_steps(i + 2, std::integral_constant<int, H0 + 2>{}, masked_tag);
  };
  // The steps, a multiple of four, are an odd or even number of half turns; the loop below runs whole
  // turns, so an odd half turn comes first, at the ring's second half (the prologue has put the first
  // tile into the buffer that goes with it).  With the causal mask the key block's own four sub-tiles
  // come first and straddle the diagonal: wave w masks sub-tiles i0 .. i0+w.
  static_assert(!CAUSAL || BK == 128, "four diagonal sub-tiles per key block");
  constexpr std::integral_constant<int, 0> first_half{};
  constexpr std::integral_constant<int, HALF> second_half{};
  constexpr std::integral_constant<bool, CAUSAL> head_masked{};
  int i = i0;
  if (head_half) {
    half_turn(i, second_half, head_masked);
    i += HALF;
  } else if constexpr (CAUSAL) {
    half_turn(i, first_half, std::true_type{});
    half_turn(i + HALF, second_half, std::integral_constant<bool, HALF == 2>{});
    i += RING;
  }
#pragma nounroll
  while (i < n_sub) {
    half_turn(i, first_half, std::false_type{});
    half_turn(i + HALF, second_half, std::false_type{});
    i += RING;
  }
  // upper query half of the last sub-tile, at the last ring position
#pragma unroll
  for (int m = NACC / 2; m < NACC; ++m) acc_mfma(m, acc_frag((RING - 1) / SPT, (RING - 1) % SPT, m), pk);

  wait_async_tiles();   // the re-fetch issued by the last step has nothing left to land in after the kernel
  // accumulator tile tt: column = 32*tt + j (feature), register r = key row 8*(r/4) + 4g + (r%4)
  const int kloc0 = kt * BK + wave * 32;               // first key of this wave inside the unit
  if constexpr (DO_V) {
    half_t* const o = p.dv + da_abi::unit_base(p, p.sdv, bh) + (size_t)kloc0 * (size_t)p.sdv.n;
#pragma unroll
    for (int tt = 0; tt < NVT; ++tt)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int kr = 8 * (r / 4) + 4 * g + (r % 4);
        if (!PADDED || kloc0 + kr < p.n_keys) o[(size_t)kr * (size_t)p.sdv.n + 32 * tt + j] = (half_t)dv[tt][r];
      }
  }
  if constexpr (DO_K) {
    const size_t ob = da_abi::unit_base(p, p.sdqk, bh) + (size_t)kloc0 * (size_t)p.sdqk.n;
#pragma unroll
    for (int tt = 0; tt < NDT; ++tt)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int kr = 8 * (r / 4) + 4 * g + (r % 4);
        if (!PADDED || kloc0 + kr < p.n_keys) {
          p.dk1[ob + (size_t)kr * (size_t)p.sdqk.n + 32 * tt + j] = (half_t)(dk1[tt][r] * p.sm_scale);
          p.dk2[ob + (size_t)kr * (size_t)p.sdqk.n + 32 * tt + j] = (half_t)(dk2[tt][r] * p.sm_scale);
        }
      }
  }
}

// ------------------------------------------------------------------------------------------------
template <int D, int NWAVES>
struct DqCfg {
  static constexpr int DV = 2 * D;
  static constexpr int NW = NWAVES;            // waves per workgroup, 32 query rows each
  // waves per SIMD the register budget is sized for: the resident Q1, Q2, dX rows and the two dQ
  // accumulators of a D = 128 wave do not fit 256 registers
  static constexpr int OCC = (D == 128) ? 1 : 2;
  static constexpr int NT = NW * 64;
  // thread count the register budget is derived from: with fewer than 4 * OCC waves in a workgroup
  // the occupancy attribute alone does not hold the allocator to 512 / OCC registers
  static constexpr int REG_NT = (OCC * 256 > NT) ? OCC * 256 : NT;
  static constexpr int BM = NW * 32;           // query rows per workgroup
  static constexpr int BN = (D <= 64) ? 64 : 32;  // keys per staged tile
  static constexpr int K_TILE = BN * D;        // halfs (swizzled, unpadded)
  static constexpr int V_TILE = BN * DV;
  static constexpr int STAGE = 2 * K_TILE + V_TILE;
  // A ring of four buffers whose position is a compile-time constant in every iteration (the loop body is one
  // turn of the ring), laid out by tile kind so that an instruction's immediate offset reaches every buffer.
  // Tiles are fetched two iterations ahead.  With a barrier per tile three buffers would do; four let the
  // workgroup meet every second tile only (a tile's buffer is refilled two tiles after it was read, which is
  // always past one barrier), so the two waves of a SIMD, which leave a barrier in step, have twice as long to
  // drift apart and overlap one's matrix products with the other's element-wise work.  Measured in one GPU call
  // against a barrier per tile: 3.6 % faster at D = 128, 0.8 % at D = 32, 2 % slower at D = 64.
  static constexpr bool PAIR = (D != 64);      // a barrier every second tile
  static constexpr int NBUF = 4;
  static constexpr int KBUF_BYTES = 2 * K_TILE * 2, VBUF_BYTES = V_TILE * 2, VBASE_BYTES = NBUF * KBUF_BYTES;
  static_assert(NBUF * KBUF_BYTES <= 65536 && NBUF * VBUF_BYTES <= 65536, "immediate offsets reach every buffer");
};

// dQ_t = s * dS_t K_t for one block of query rows.  Every product is formed transposed,
// [keys x queries], so that a lane owns one query column: the row statistics are per-lane
// scalars and dS^T in accumulator layout is directly the B operand of dQ^T = K^T dS^T.
// MASK: 0 none; 1 causal (key <= query); 2 the last keys of the sequence are padding (key < n_keys).
// A padded key has a zero K row, but its recomputed "probability" exp(0 - lse) is not small when a
// row's logsumexp is negative, and its dS can overflow fp16: it must be masked, not multiplied by 0.
// DROP: dropout on both softmax maps, as in bwd_dkdv_kernel.
template <int D, int NWAVES, int MASK, bool DROP>
__global__ __launch_bounds__((DqCfg<D, NWAVES>::REG_NT)) __attribute__((amdgpu_waves_per_eu(DqCfg<D, NWAVES>::OCC, DqCfg<D, NWAVES>::OCC))) void bwd_dq_kernel(BwdParams p) {
  using C = DqCfg<D, NWAVES>;
  constexpr bool CAUSAL = (MASK == 1), PADDED = (MASK == 2);
  // rows past the real length are neither read from the caller's tensors nor written to the gradients: checked
  // in both masked variants (the causal one serves padded sequences too), compiled out of the plain one
  constexpr bool TAIL = (MASK != 0);
  constexpr int DV = C::DV, NW = C::NW, BM = C::BM, BN = C::BN;
  constexpr int NKS = D / 16, NKV = DV / 16, NDT = D / 32;
#ifndef DQ_ASM_SCORES
#define DQ_ASM_SCORES (D == 128 && !DROP)
#endif
#ifndef DQ_PIPE
#define DQ_PIPE (D == 128 && !DROP)
#endif
  constexpr bool kPipe = DQ_PIPE;     // the software-pipelined loop of the one-wave-per-SIMD kernel, below

  __shared__ __attribute__((aligned(16))) half_t smem[C::NBUF * C::STAGE];
  static_assert(sizeof(smem) >= 256 * sizeof(float), "the hosted reduction uses the tile memory");
  DA_HOST_DLAMBDA(smem)

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int j = lane & 31, g = lane >> 5;

  const int n_qt = p.N / BM;
  int bh, qt;
  if constexpr (CAUSAL) {   // the last query block of a unit sees the most keys
    const UnitBlock ub = longest_first(blockIdx.x, p.BH);
    bh = ub.unit; qt = n_qt - 1 - ub.rank;
  } else {
    const int tile = xcd_remap(blockIdx.x, gridDim.x - p.dlam_fold);
    bh = tile / n_qt; qt = tile % n_qt;
  }
  const size_t rows = (size_t)p.BH * p.N;
  const size_t row0 = (size_t)bh * p.N;
  const size_t qrow = row0 + qt * BM + wave * 32 + j;
  // element offsets of the unit's first row and the row strides of the strided tensors
  const size_t qk_base = da_abi::unit_base(p, p.sqk, bh), v_base = da_abi::unit_base(p, p.sv, bh);
  const int qk_n = (int)p.sqk.n, v_n = (int)p.sv.n;

  const float lam = da_abi::lambda_of_unit(p, bh);
  // hash keys of this unit's two softmax streams (used with dropout only)
  const DropoutKey dkey1 = dropout_key(p.drop, 2u * bh), dkey2 = dropout_key(p.drop, 2u * bh + 1);

  // persistent B operands: this lane's query row of Q1, Q2 (pre-multiplied by sm_scale*log2(e)
  // exactly as in the forward kernel, so the recomputed probabilities match it), dX, and its row
  // statistics
  h8 qf1[NKS], qf2[NKS], xf[NKV];
  {
    const float c = p.sm_scale * kLog2e;
    // a padding row stands in with the last real row, as in the forward; its results are not stored
    int qr = qt * BM + wave * 32 + j;
    if (TAIL && qr >= p.n_keys) qr = p.n_keys - 1;
    const half_t* r1 = p.q1 + qk_base + (size_t)qr * qk_n + 8 * g;
    const half_t* r2 = p.q2 + qk_base + (size_t)qr * qk_n + 8 * g;
    const half_t* rx = p.dx + qrow * DV + 8 * g;
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) {
      h8 a = *reinterpret_cast<const h8*>(r1 + 16 * ks);
      h8 b = *reinterpret_cast<const h8*>(r2 + 16 * ks);
#pragma unroll
      for (int e = 0; e < 8; ++e) { a[e] = (half_t)((float)a[e] * c); b[e] = (half_t)((float)b[e] * c); }
      qf1[ks] = a; qf2[ks] = b;
    }
#pragma unroll
    for (int kv = 0; kv < NKV; ++kv) xf[kv] = *reinterpret_cast<const h8*>(rx + 16 * kv);
  }
  const float nl1_ld = p.stat[0 * rows + qrow], nl2_ld = p.stat[1 * rows + qrow];
  const float de1_ld = p.stat[2 * rows + qrow], de2_ld = p.stat[3 * rows + qrow];

  f16v dq1[NDT], dq2[NDT];
#pragma unroll
  for (int t = 0; t < NDT; ++t)
#pragma unroll
    for (int r = 0; r < 16; ++r) { dq1[t][r] = 0.f; dq2[t][r] = 0.f; }

  using KTile = AsyncTile<BN, D, NW>;
  using VTile = AsyncTile<BN, DV, NW>;
  const half_t* gk1 = p.k1 + qk_base;
  const half_t* gk2 = p.k2 + qk_base;
  const half_t* gv = p.v + v_base;
  const unsigned k_off = KTile::lane_off(wave, lane, qk_n), v_off = VTile::lane_off(wave, lane, v_n);
  // causal: keys beyond the last row of the workgroup are never visited
  // padding: tiles that hold no real key are not visited either
  // (an even count in every variant: with padding, a last tile without a real key may be visited; its keys are masked)
  const int n_tiles = CAUSAL ? (qt + 1) * (BM / BN) : PADDED ? (((p.n_keys + BN - 1) / BN + 1) & ~1) : p.N / BN;
  constexpr int VH = (VTile::PER + 1) / 2;

  // loads a wave issues per iteration (one K1, one K2 and one V tile)
  const int loads_per_iter = 2 * KTile::count(wave) + VTile::count(wave);
  // with padding, the tiles that reach past the last real key are copied with their row index clamped to it
  auto copy_k = [&](const half_t* gk, int t, half_t* dst) {
    if (TAIL && (t + 1) * BN > p.n_keys) KTile::issue_clamped(gk + (size_t)t * BN * qk_n, dst, wave, lane, k_off, qk_n, p.n_keys - 1 - t * BN);
    else KTile::issue_at(gk + (size_t)t * BN * qk_n, dst, wave, lane, k_off, qk_n);
  };
  auto copy_v = [&](int t, half_t* dst, auto k0_tag, auto k1_tag) {
    constexpr int K0 = decltype(k0_tag)::value, K1 = decltype(k1_tag)::value;
    if (TAIL && (t + 1) * BN > p.n_keys) VTile::template issue_clamped<K0, K1>(gv + (size_t)t * BN * v_n, dst, wave, lane, v_off, v_n, p.n_keys - 1 - t * BN);
    else VTile::template issue_at<K0, K1>(gv + (size_t)t * BN * v_n, dst, wave, lane, v_off, v_n);
  };
  constexpr std::integral_constant<int, 0> v_begin{};
  constexpr std::integral_constant<int, VH> v_mid{};
  constexpr std::integral_constant<int, VTile::PER> v_end{};
  // tile memory by kind: K1 and K2 of buffer b, then the V tiles
  auto k_buf = [&](int b) { return smem + b * (C::KBUF_BYTES / 2); };
  auto v_buf = [&](int b) { return smem + C::VBASE_BYTES / 2 + b * C::V_TILE; };
  auto fetch_all = [&](int t, int buf) {
    copy_k(gk1, t, k_buf(buf));
    copy_k(gk2, t, k_buf(buf) + C::K_TILE);
    copy_v(t, v_buf(buf), v_begin, v_end);
  };
  // The loop runs whole turns of the ring (NBUF iterations); the tile count is even, so when it is not a
  // multiple of four, half a turn comes first and tile 0 goes into buffer 2: tile t is in buffer (t + b0) % NBUF.
  static_assert(C::NBUF == 4, "the loop is unrolled over a ring of four");
  const bool head_half = (n_tiles & 2) != 0;
  const int b0 = head_half ? 2 : 0;
  fetch_all(0, b0);
  fetch_all((n_tiles > 1) ? 1 : 0, b0 + 1);
  if constexpr (kPipe) fetch_all((n_tiles > 2) ? 2 : n_tiles - 1, (b0 + 2) % C::NBUF);   // it fetches three tiles ahead
  // dX and the row statistics are first used inside the loop, and the compiler waits for a load where it is first
  // used.  It does not see the asynchronous tile copies, so its wait for "the newest loads" would in fact be a
  // wait for every tile copy in flight, in every iteration.  Touching the registers here puts that wait in front
  // of the loop, where the first tiles are waited for anyway.
  // At D = 128 the kernel runs one wave per SIMD, and for a kernel with that register budget the compiler selects
  // every MFMA with its C and D operands in AGPRs: right for the dQ accumulators, but each recomputed score
  // and dP value then costs a copy back for the element-wise work (a quarter of the loop's VALU instructions).
  // There the three score products are issued as assembly with their results in VGPRs and the resident
  // Q1, Q2 and dX rows, which are only ever B operands, in AGPRs.  (Not in the dropout instantiations, whose
  // mask arithmetic makes the compiler move operands about: see bwd_dkdv_kernel.)
  constexpr bool kAsmScores = DQ_ASM_SCORES;
  if constexpr (kAsmScores) {
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) { keep_in_agpr(qf1[ks]); keep_in_agpr(qf2[ks]); }
#pragma unroll
    for (int kv = 0; kv < NKV; ++kv) keep_in_agpr(xf[kv]);
  } else {
#pragma unroll
    for (int kv = 0; kv < NKV; ++kv) asm volatile("" : "+v"(xf[kv]));
  }
  float nl1 = nl1_ld, nl2 = nl2_ld, de1 = de1_ld, de2 = de2_ld;
  asm volatile("" : "+v"(nl1), "+v"(nl2), "+v"(de1), "+v"(de2));
  if (C::PAIR || kPipe) wait_async_tiles();         // tiles 0 and 1 are read before the next barrier
  else wait_async_tiles_except(loads_per_iter);     // tile 0 has landed, tile 1 may still be in flight
  __syncthreads();

  // Per-lane LDS byte addresses, computed once.  The XOR swizzle makes the address of a fragment a different
  // function of the lane for every 16-byte chunk column, so there is one register per chunk column a lane
  // reads; the ring buffer, K1 or K2, the 32-key sub-tile and the k-step of 16 keys are multiples of 16 rows,
  // which the swizzle does not see, and travel in the instructions' immediate offsets.
  const int tr_row = 4 * g + ((lane & 15) >> 2);
  const int tr_col = 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
  const unsigned lds0 = (unsigned)(unsigned long)((DA_LDS char*)smem);
  unsigned kfr[NKS], vfr[NKV], ktr[NDT][2];
#pragma unroll
  for (int ks = 0; ks < NKS; ++ks) kfr[ks] = lds0 + 2u * (unsigned)swz_off<D>(j, 16 * ks + 8 * g);
#pragma unroll
  for (int kv = 0; kv < NKV; ++kv) vfr[kv] = lds0 + C::VBASE_BYTES + 2u * (unsigned)swz_off<DV>(j, 16 * kv + 8 * g);
#pragma unroll
  for (int tt = 0; tt < NDT; ++tt)
#pragma unroll
    for (int e = 0; e < 2; ++e) ktr[tt][e] = lds0 + 2u * (unsigned)swz_off<D>(tr_row + 8 * e, 32 * tt + tr_col);
  // kept as they are: the compiler neither folds constants into them nor recomputes them in the loop
#pragma unroll
  for (int ks = 0; ks < NKS; ++ks) asm volatile("" : "+v"(kfr[ks]));
#pragma unroll
  for (int kv = 0; kv < NKV; ++kv) asm volatile("" : "+v"(vfr[kv]));
#pragma unroll
  for (int tt = 0; tt < NDT; ++tt) asm volatile("" : "+v"(ktr[tt][0]), "+v"(ktr[tt][1]));

  // Where registers allow, a row statistic that is added to every element of a product is the product's
  // initial accumulator value instead: sixteen registers that hold it, for sixteen additions less per sub-tile.
#ifndef DQ_FOLD_DP
#define DQ_FOLD_DP (!DROP && (D == 32 || (D == 64 && MASK == 0)))
#endif
#ifndef DQ_FOLD_S
#define DQ_FOLD_S (D == 32)
#endif
  constexpr bool kFoldDP = DQ_FOLD_DP;     // dP starts from -delta1 (not with dropout, which masks dP first)
  constexpr bool kFoldS = DQ_FOLD_S;       // S1, S2 start from the negated logsumexp
  f16v de1v, nl1v, nl2v;
#pragma unroll
  for (int r = 0; r < 16; ++r) { de1v[r] = kFoldDP ? de1 : 0.f; nl1v[r] = kFoldS ? nl1 : 0.f; nl2v[r] = kFoldS ? nl2 : 0.f; }
  if constexpr (kFoldDP) asm volatile("" : "+v"(de1v));
  if constexpr (kFoldS) asm volatile("" : "+v"(nl1v), "+v"(nl2v));

  if constexpr (kPipe) {
    // One wave per SIMD has nobody to run its element-wise work under, so the loop is pipelined inside the wave,
    // as in the dK/dV kernel: while the element-wise work of tile t runs on the VALU, row by row, the score
    // products of tile t+1 (assembly, results in VGPRs) run on the matrix unit, two per row; the dQ products
    // of tile t follow.  Tiles are 32 keys (one sub-tile) and are fetched three iterations ahead; the workgroup
    // meets once per tile.
    static_assert(kAsmScores && BN == 32 && !kFoldDP && !kFoldS, "the pipelined loop");
    struct Scores { f16v s1, s2, dp; };
    constexpr int NPROD = 2 * NKS + NKV;              // score products per tile: S1 and S2 alternating, then dP
    // A fragment of product k of the tile in the buffer at byte offsets (KOFF, VOFF)
    auto prod_frag = [&](auto koff_tag, auto voff_tag, int k) -> h8 {
      constexpr int KOFF = decltype(koff_tag)::value, VOFF = decltype(voff_tag)::value;
      if (k < 2 * NKS) return lds_read_at<h8>(kfr[k / 2], KOFF + (k & 1) * C::K_TILE * 2);
      return lds_read_at<h8>(vfr[k - 2 * NKS], VOFF);
    };
    auto prod_mfma = [&](int k, h8 a, Scores& s) {
      if (k < 2 * NKS) {
        const int ks = k / 2;
        if (k & 1) s.s2 = ks ? mfma32_bagpr(a, qf2[ks], s.s2) : mfma32_bagpr_first(a, qf2[0]);
        else       s.s1 = ks ? mfma32_bagpr(a, qf1[ks], s.s1) : mfma32_bagpr_first(a, qf1[0]);
      } else {
        const int kv = k - 2 * NKS;
        s.dp = kv ? mfma32_bagpr(a, xf[kv], s.dp) : mfma32_bagpr_first(a, xf[0]);
      }
    };
    constexpr int DEPTH = 4;                          // A fragments requested ahead of their product
    Scores sa, sb;
    {
      // scores of tile 0, nothing to run them under
      h8 a[NPROD];
      if (head_half) {
#pragma unroll
        for (int k = 0; k < NPROD; ++k)
          a[k] = prod_frag(std::integral_constant<int, 2 * C::KBUF_BYTES>{}, std::integral_constant<int, 2 * C::VBUF_BYTES>{}, k);
      } else {
#pragma unroll
        for (int k = 0; k < NPROD; ++k) a[k] = prod_frag(std::integral_constant<int, 0>{}, std::integral_constant<int, 0>{}, k);
      }
#pragma unroll
      for (int k = 0; k < NPROD; ++k) prod_mfma(k, a[k], sa);
      mfma_results_ready(sa.s1, sa.s2, sa.dp);
    }

    auto iteration = [&](int t, auto pos_tag, Scores& cur, Scores& nxt) {
      constexpr int POS = decltype(pos_tag)::value;
      constexpr int KCUR = POS * C::KBUF_BYTES;
      constexpr int PNXT = (POS + 1) % C::NBUF, BFAR = (POS + 3) % C::NBUF;
      constexpr std::integral_constant<int, PNXT * C::KBUF_BYTES> knext{};
      constexpr std::integral_constant<int, PNXT * C::VBUF_BYTES> vnext{};
      const int tf = (t + 3 < n_tiles) ? t + 3 : n_tiles - 1;   // past the end: harmless re-reads
      copy_k(gk1, tf, k_buf(BFAR));
      if constexpr (CAUSAL) {
        // only the last tiles of a wave's loop reach past its first row: mask key > query there
        const int wrow0 = qt * BM + wave * 32;
        const int kbase = t * BN;
        if (kbase + 31 > wrow0) {
          const int rel = wrow0 + j - kbase - 4 * g;     // query index minus the key index of register 0
#pragma unroll
          for (int r = 0; r < 16; ++r)
            if (8 * (r / 4) + (r % 4) > rel) { cur.s1[r] = -INFINITY; cur.s2[r] = -INFINITY; }
        }
      }
      if constexpr (PADDED) {
        const int kbase = t * BN;
        if (kbase + 32 > p.n_keys) {
          const int rel = p.n_keys - 1 - kbase - 4 * g;   // last real key minus the key index of register 0
#pragma unroll
          for (int r = 0; r < 16; ++r)
            if (8 * (r / 4) + (r % 4) > rel) { cur.s1[r] = -INFINITY; cur.s2[r] = -INFINITY; }
        }
      }
      // the transposed K fragments of this tile's dQ products are requested here and arrive under the loop below
      h8 tk1[2][NDT], tk2[2][NDT];
#pragma unroll
      for (int kk = 0; kk < 2; ++kk)
#pragma unroll
        for (int tt = 0; tt < NDT; ++tt) {
          const int off = KCUR + 16 * kk * D * 2;
          tk1[kk][tt] = join(lds_read_tr_at(ktr[tt][0], off), lds_read_tr_at(ktr[tt][1], off));
          tk2[kk][tt] = join(lds_read_tr_at(ktr[tt][0], off + C::K_TILE * 2), lds_read_tr_at(ktr[tt][1], off + C::K_TILE * 2));
        }
      h8 a[NPROD];
#pragma unroll
      for (int k = 0; k < DEPTH; ++k) a[k] = prod_frag(knext, vnext, k);
      h8 b1[2], b2[2];
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int k = 0; k < NPROD; ++k) {
        if (k + DEPTH < NPROD) a[k + DEPTH] = prod_frag(knext, vnext, k + DEPTH);
        // the far tile's copies are spread over the products
        if (k == NPROD / 4) copy_k(gk2, tf, k_buf(BFAR) + C::K_TILE);
        if (k == NPROD / 2) copy_v(tf, v_buf(BFAR), v_begin, v_mid);
        if (k == 3 * NPROD / 4) copy_v(tf, v_buf(BFAR), v_mid, v_end);
        prod_mfma(k, a[k], nxt);
        // element-wise rows of this tile, spread evenly over the products
        const int r0 = 16 * k / NPROD, r1 = 16 * (k + 1) / NPROD;
#pragma unroll
        for (int r = r0; r < r1; ++r) {
          const float p1 = fast_exp2(cur.s1[r] + nl1);
          const float p2 = fast_exp2(cur.s2[r] + nl2);
          // in fp32 up to the rounding of dS itself (see the loop of the other head dims)
          const float dpc = cur.dp[r] + de1;
          b1[r / 8][r % 8] = (half_t)(p1 * dpc);
          b2[r / 8][r % 8] = (half_t)(p2 * __builtin_fmaf(-lam, dpc, de2));
        }
        __builtin_amdgcn_sched_barrier(0);
      }
      mfma_results_ready(nxt.s1, nxt.s2, nxt.dp);     // the next iteration's VALU reads them
#pragma unroll
      for (int kk = 0; kk < 2; ++kk)
#pragma unroll
        for (int tt = 0; tt < NDT; ++tt) {
          dq1[tt] = mfma32(tk1[kk][tt], b1[kk], dq1[tt]);
          dq2[tt] = mfma32(tk2[kk][tt], b2[kk], dq2[tt]);
        }
      // the next iteration reads tiles t+1 and t+2: only this iteration's loads (tile t+3) may remain in flight
      wait_async_tiles_except(loads_per_iter);
      __syncthreads();
    };

    int t = 0;
    if (head_half) {
      iteration(0, std::integral_constant<int, 2>{}, sa, sb);
      iteration(1, std::integral_constant<int, 3>{}, sb, sa);
      t = 2;
    }
#pragma nounroll
    for (; t < n_tiles; t += 4) {
      iteration(t, std::integral_constant<int, 0>{}, sa, sb);
      iteration(t + 1, std::integral_constant<int, 1>{}, sb, sa);
      iteration(t + 2, std::integral_constant<int, 2>{}, sa, sb);
      iteration(t + 3, std::integral_constant<int, 3>{}, sb, sa);
    }
  } else {
  // One iteration: tile t, in the buffer at ring position POS; tile t+2 is requested into the buffer two
  // positions on, which held a tile that every wave has finished reading.
  auto iteration = [&](int t, auto pos_tag) {
    constexpr int POS = decltype(pos_tag)::value;
    constexpr int KCUR = POS * C::KBUF_BYTES, VCUR = POS * C::VBUF_BYTES, BNXT = (POS + 2) % C::NBUF;
    const int tn = (t + 2 < n_tiles) ? t + 2 : n_tiles - 1;   // past the end: harmless re-reads
    copy_k(gk1, tn, k_buf(BNXT));

#pragma unroll
    for (int ksub = 0; ksub < BN / 32; ++ksub) {
      if (ksub == 0) copy_k(gk2, tn, k_buf(BNXT) + C::K_TILE);
      // transposed tiles [32 keys x 32 queries]: this lane's column is its query
      f16v s1 = nl1v, s2 = nl2v, dp = de1v;       // zero, or the folded statistic
      // all fragments of the three score products are requested before the first product is issued
      h8 ak1[NKS], ak2[NKS], av[NKV];
#pragma unroll
      for (int ks = 0; ks < NKS; ++ks) {
        ak1[ks] = lds_read_at<h8>(kfr[ks], KCUR + ksub * 32 * D * 2);
        ak2[ks] = lds_read_at<h8>(kfr[ks], KCUR + C::K_TILE * 2 + ksub * 32 * D * 2);
      }
#pragma unroll
      for (int kv = 0; kv < NKV; ++kv) av[kv] = lds_read_at<h8>(vfr[kv], VCUR + ksub * 32 * DV * 2);
      __builtin_amdgcn_sched_barrier(0);
      if constexpr (kAsmScores) {
        if constexpr (kFoldS) {
          s1 = mfma32_bagpr_from(ak1[0], qf1[0], nl1v);
          s2 = mfma32_bagpr_from(ak2[0], qf2[0], nl2v);
        } else {
          s1 = mfma32_bagpr_first(ak1[0], qf1[0]);
          s2 = mfma32_bagpr_first(ak2[0], qf2[0]);
        }
#pragma unroll
        for (int ks = 1; ks < NKS; ++ks) {
          s1 = mfma32_bagpr(ak1[ks], qf1[ks], s1);
          s2 = mfma32_bagpr(ak2[ks], qf2[ks], s2);
        }
        dp = kFoldDP ? mfma32_bagpr_from(av[0], xf[0], de1v) : mfma32_bagpr_first(av[0], xf[0]);
#pragma unroll
        for (int kv = 1; kv < NKV; ++kv) dp = mfma32_bagpr(av[kv], xf[kv], dp);
        mfma_results_ready(s1, s2, dp);      // the compiler does not know these are matrix instructions
      } else {
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks) {
          s1 = mfma32(ak1[ks], qf1[ks], s1);
          s2 = mfma32(ak2[ks], qf2[ks], s2);
        }
#pragma unroll
        for (int kv = 0; kv < NKV; ++kv) dp = mfma32(av[kv], xf[kv], dp);
      }
      if (ksub == 0) copy_v(tn, v_buf(BNXT), v_begin, v_mid);
      // with a barrier every second tile all of a tile's copies go out early: they have to land by the next barrier
      if (ksub == (C::PAIR ? 0 : BN / 32 - 1)) copy_v(tn, v_buf(BNXT), v_mid, v_end);
      if constexpr (CAUSAL) {
        // only the last sub-tiles of a wave's loop reach past its first row: mask key > query there
        const int wrow0 = qt * BM + wave * 32;
        const int kbase = t * BN + ksub * 32;
        if (kbase + 31 > wrow0) {
          const int rel = wrow0 + j - kbase - 4 * g;     // query index minus the key index of register 0
#pragma unroll
          for (int r = 0; r < 16; ++r)
            if (8 * (r / 4) + (r % 4) > rel) { s1[r] = -INFINITY; s2[r] = -INFINITY; }
        }
      }
      if constexpr (PADDED) {
        // only the last sub-tiles hold padding keys
        const int kbase = t * BN + ksub * 32;
        if (kbase + 32 > p.n_keys) {
          const int rel = p.n_keys - 1 - kbase - 4 * g;   // last real key minus the key index of register 0
#pragma unroll
          for (int r = 0; r < 16; ++r)
            if (8 * (r / 4) + (r % 4) > rel) { s1[r] = -INFINITY; s2[r] = -INFINITY; }
        }
      }
      // The transposed K fragments of the dQ products do not depend on the element-wise work: they
      // are requested before it and arrive while it runs.  (Left to itself the compiler requests
      // each one right in front of its product and waits out the LDS latency eight times.)
      // (The dropout instantiations need the registers for the mask arithmetic and read each
      // fragment in front of its product instead.)
      h8 tk1[2][NDT], tk2[2][NDT];
      auto read_tk = [&](int kk, int tt) {
        const int off = KCUR + (ksub * 32 + 16 * kk) * D * 2;
        tk1[kk][tt] = join(lds_read_tr_at(ktr[tt][0], off), lds_read_tr_at(ktr[tt][1], off));
        tk2[kk][tt] = join(lds_read_tr_at(ktr[tt][0], off + C::K_TILE * 2), lds_read_tr_at(ktr[tt][1], off + C::K_TILE * 2));
      };
      // (At D = 128 the masked variants, which also carry the row clamping of padded sequences, are short of
      // registers in the same way.)
      constexpr bool kFragmentsAhead = !DROP && !(D == 128 && TAIL);
      if constexpr (kFragmentsAhead) {
#pragma unroll
        for (int kk = 0; kk < 2; ++kk)
#pragma unroll
          for (int tt = 0; tt < NDT; ++tt) read_tk(kk, tt);
      }
      __builtin_amdgcn_sched_barrier(0);
      h8 b1[2], b2[2];
      unsigned w1 = 0, w2 = 0, w1b = 0, w2b = 0;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const float p1 = fast_exp2(kFoldS ? s1[r] : s1[r] + nl1);
        const float p2 = fast_exp2(kFoldS ? s2[r] : s2[r] + nl2);
        if constexpr (DROP) {
          // register r holds key kq + 8*(r/4) + (r%4) of this lane's query; registers r, r+1 (r even)
          // share the hash words of their 2x2 block
          const unsigned query = (unsigned)(qt * BM + wave * 32 + j);
          const unsigned kq = (unsigned)(t * BN + ksub * 32 + 4 * g + 8 * (r / 4) + (r % 4));
          // the blocks of registers r..r+1 and r+2..r+3 (r a multiple of 4) are neighbours, hashed one by each
          // lane of a query pair
          if ((r & 3) == 0) {
            dropout_words_shared(dropout_word(dkey1, (unsigned)p.N / 2, query >> 1, (kq >> 1) + (query & 1)), query & 1, w1, w1b);
            dropout_words_shared(dropout_word(dkey2, (unsigned)p.N / 2, query >> 1, (kq >> 1) + (query & 1)), query & 1, w2, w2b);
          }
          const float dpk = p.drop.keep_scale * dp[r];
          const float d1 = dropout_keep((r & 2) ? w1b : w1, query, kq, p.drop.threshold) ? dpk : 0.f;
          const float d2 = dropout_keep((r & 2) ? w2b : w2, query, kq, p.drop.threshold) ? dpk : 0.f;
          b1[r / 8][r % 8] = (half_t)(p1 * (d1 + de1));                                             // c m1 dP - delta1
          b2[r / 8][r % 8] = (half_t)(p2 * __builtin_fmaf(-lam, d2, __builtin_fmaf(-lam, de1, de2)));   // -lambda c m2 dP - delta2
        } else {
          // in fp32 up to the rounding of dS itself: dP - delta alone may exceed the 16-bit range when the
          // upstream gradient carries a loss scale, while its product with the probability does not
          const float dpc = kFoldDP ? dp[r] : dp[r] + de1;                  // statistic 2 is -delta1
          b1[r / 8][r % 8] = (half_t)(p1 * dpc);
          b2[r / 8][r % 8] = (half_t)(p2 * __builtin_fmaf(-lam, dpc, de2));   // statistic 3 is -(lambda*delta1 + delta2)
        }
      }
#pragma unroll
      for (int kk = 0; kk < 2; ++kk)
#pragma unroll
        for (int tt = 0; tt < NDT; ++tt) {
          if constexpr (!kFragmentsAhead) read_tk(kk, tt);
          dq1[tt] = mfma32(tk1[kk][tt], b1[kk], dq1[tt]);
          dq2[tt] = mfma32(tk2[kk][tt], b2[kk], dq2[tt]);
        }
    }

    if constexpr (C::PAIR) {
      // Every second tile the workgroup meets: the copies of the next two tiles (requested during the last
      // two) have landed for everybody, and the buffers of the last two tiles may be refilled.
      if constexpr (POS & 1) {
        wait_async_tiles();
        __syncthreads();
      }
    } else {
      // tile t+1 was requested one iteration ago: only this iteration's loads may remain in flight
      wait_async_tiles_except(loads_per_iter);
      __syncthreads();
    }
  };

  int t = 0;
  if (head_half) {
    iteration(0, std::integral_constant<int, 2>{});
    iteration(1, std::integral_constant<int, 3>{});
    t = 2;
  }
#pragma nounroll
  for (; t < n_tiles; t += 4) {
    iteration(t, std::integral_constant<int, 0>{});
    iteration(t + 1, std::integral_constant<int, 1>{});
    iteration(t + 2, std::integral_constant<int, 2>{});
    iteration(t + 3, std::integral_constant<int, 3>{});
  }
  }
  wait_async_tiles();
  __syncthreads();      // the tile memory is reused below; other waves may still have been reading it

  // dQ^T tile tt: this lane's column is its query; register r = feature 32*tt + 8*(r/4) + 4g + (r%4).
  // The accumulated sums carry log2(e) from the pre-scaled Q only inside the probabilities, so the
  // remaining factor is the plain softmax scale.  Each wave stages its 32 rows of dQ1 and dQ2 in the
  // now idle tile memory (8 bytes per lane, row stride D+8 halfs) and reads them back row by row, so
  // that the global stores are whole 16-byte chunks of consecutive rows.
  constexpr int SROW = D + 8;
  static_assert(NW * 2 * 32 * SROW <= C::NBUF * C::STAGE, "staging blocks fit the tile memory");
  half_t* const stg = smem + (size_t)wave * 2 * 32 * SROW;
#pragma unroll
  for (int tt = 0; tt < NDT; ++tt)
#pragma unroll
    for (int r4 = 0; r4 < 4; ++r4) {
      h4 v1, v2;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        v1[e] = (half_t)(dq1[tt][4 * r4 + e] * p.sm_scale);
        v2[e] = (half_t)(dq2[tt][4 * r4 + e] * p.sm_scale);
      }
      *reinterpret_cast<h4*>(stg + j * SROW + 32 * tt + 8 * r4 + 4 * g) = v1;
      *reinterpret_cast<h4*>(stg + (32 + j) * SROW + 32 * tt + 8 * r4 + 4 * g) = v2;
    }
  __builtin_amdgcn_wave_barrier();   // the rows are read back by other lanes of this wave only
  constexpr int LPR = D / 8;         // lanes per row
  constexpr int RPI = 64 / LPR;      // rows per instruction
  const int qloc0 = qt * BM + wave * 32;             // first query of this wave inside the unit
  const size_t ob = da_abi::unit_base(p, p.sdqk, bh) + (size_t)qloc0 * (size_t)p.sdqk.n;
  half_t* const o1 = p.dq1 + ob;
  half_t* const o2 = p.dq2 + ob;
#pragma unroll
  for (int k = 0; k < 32 / RPI; ++k) {
    const int row = k * RPI + lane / LPR, ch = lane % LPR;
    const u32x4 v1 = *reinterpret_cast<const u32x4*>(stg + row * SROW + 8 * ch);
    const u32x4 v2 = *reinterpret_cast<const u32x4*>(stg + (32 + row) * SROW + 8 * ch);
    if (!TAIL || qloc0 + row < p.n_keys) {    // the gradient tensors have no rows past the real length
      *reinterpret_cast<u32x4*>(o1 + (size_t)row * (size_t)p.sdqk.n + 8 * ch) = v1;
      *reinterpret_cast<u32x4*>(o2 + (size_t)row * (size_t)p.sdqk.n + 8 * ch) = v2;
    }
  }
}

// ------------------------------------------------------------------------------------------------
template <int D>
static hipError_t launch_bwd_t(const BwdParams& p_in, hipStream_t stream) {
  BwdParams p = p_in;
  const int n_prep = bwd_num_partials(p.BH, p.N, D);
  hipError_t e = hipSuccess;
  // Shape-aware launch geometry (the reference autotunes its tiles per (N, D, Dv), src/kernel.py:12-19): a problem
  // whose 128-row blocks do not fill the chip once runs in twice as many 64-row workgroups.  A pure function of
  // (B*H, N, D) and the options: no tuning state.  Only the plain dK/dV instantiation has the small variant
  // (the dQ kernel was measured with 64-row workgroups too: 15-20 % slower on such grids, so it keeps 128).
  constexpr int kNumCU = 256;
  const bool small_grid = D != 128 && !p.causal && !p.drop.threshold && p.n_keys == p.N &&
                          (long long)p.BH * (p.N / 128) < kNumCU;
  // the d(lambda) reduce rides in the first dK/dV or dQ launch when there is one, else it is a launch of its own
  const int n_lambda = p.lambda_stride ? p.H : 1;
  bool fold = (p.stages & 2u) && (p.stages & 12u);
  p.dlam_fold = 0;
  if (p.stages & 1u) {
    if (p.rms_norm)
      hipLaunchKernelGGL((bwd_prep_kernel<D, true>), dim3(n_prep), dim3(256), 0, stream, p);
    else
      hipLaunchKernelGGL((bwd_prep_kernel<D, false>), dim3(n_prep), dim3(256), 0, stream, p);
    if ((e = hipGetLastError()) != hipSuccess) return e;
  }
  if ((p.stages & 2u) && !fold) {
    hipLaunchKernelGGL(bwd_dlambda_kernel, dim3(n_lambda), dim3(256), 0, stream,
                       p.dlam_part, n_prep / p.BH, p.BH, p.dlambda, p.lambda_fp32);
    if ((e = hipGetLastError()) != hipSuccess) return e;
  }
  if ((p.stages & 4u) && small_grid) {
    if constexpr (D != 128) {
      p.dlam_fold = fold ? n_lambda : 0;
      fold = false;
      const dim3 grid(p.BH * (p.N / DkvCfg<D, 2>::BK) + p.dlam_fold), block(DkvCfg<D, 2>::NT);
      hipLaunchKernelGGL((bwd_dkdv_kernel<D, 0, false, false, false, 2>), grid, block, 0, stream, p);
      if ((e = hipGetLastError()) != hipSuccess) return e;
    }
  } else if (p.stages & 4u) {
    const dim3 block(DkvCfg<D>::NT);
    auto launch_mode = [&](auto mode_tag) {
      constexpr int M = decltype(mode_tag)::value;
      p.dlam_fold = fold ? n_lambda : 0;
      fold = false;
      const dim3 grid(p.BH * (p.N / DkvCfg<D>::BK) + p.dlam_fold);
      auto launch_padded = [&](auto padded_tag) {
        constexpr bool PAD = decltype(padded_tag)::value;
        if (p.drop.threshold) {
          if (p.causal) hipLaunchKernelGGL((bwd_dkdv_kernel<D, M, true, true, PAD>), grid, block, 0, stream, p);
          else          hipLaunchKernelGGL((bwd_dkdv_kernel<D, M, false, true, PAD>), grid, block, 0, stream, p);
        } else {
          if (p.causal) hipLaunchKernelGGL((bwd_dkdv_kernel<D, M, true, false, PAD>), grid, block, 0, stream, p);
          else          hipLaunchKernelGGL((bwd_dkdv_kernel<D, M, false, false, PAD>), grid, block, 0, stream, p);
        }
      };
      if (p.n_keys < p.N) launch_padded(std::true_type{});
      else                launch_padded(std::false_type{});
    };
    if constexpr (D == 128) {
      launch_mode(std::integral_constant<int, 1>{});
      if ((e = hipGetLastError()) != hipSuccess) return e;
      launch_mode(std::integral_constant<int, 2>{});
    } else {
      launch_mode(std::integral_constant<int, 0>{});
    }
    if ((e = hipGetLastError()) != hipSuccess) return e;
  }
  if (p.stages & 8u) {
    // 256 query rows per workgroup when the sequence allows it, otherwise 128 (a D = 128 workgroup
    // runs one wave per SIMD and therefore always has four waves).  A grid so small that even its
    // 128-row workgroups all fit on the chip at once is launched that way too: it finishes sooner
    // in twice as many, half as long workgroups.
    bool wide = false;
    auto launch_dq = [&](auto nw_tag, dim3 grid, dim3 block) {
      constexpr int NWV = decltype(nw_tag)::value;
      p.dlam_fold = fold ? n_lambda : 0;
      fold = false;
      grid.x += p.dlam_fold;
      if (p.drop.threshold) {
        if (p.causal)            hipLaunchKernelGGL((bwd_dq_kernel<D, NWV, 1, true>), grid, block, 0, stream, p);
        else if (p.n_keys < p.N) hipLaunchKernelGGL((bwd_dq_kernel<D, NWV, 2, true>), grid, block, 0, stream, p);
        else                     hipLaunchKernelGGL((bwd_dq_kernel<D, NWV, 0, true>), grid, block, 0, stream, p);
      } else {
        if (p.causal)            hipLaunchKernelGGL((bwd_dq_kernel<D, NWV, 1, false>), grid, block, 0, stream, p);
        else if (p.n_keys < p.N) hipLaunchKernelGGL((bwd_dq_kernel<D, NWV, 2, false>), grid, block, 0, stream, p);
        else                     hipLaunchKernelGGL((bwd_dq_kernel<D, NWV, 0, false>), grid, block, 0, stream, p);
      }
    };
    if constexpr (D != 128) {
      if (p.N % 256 == 0 && (long long)p.BH * (p.N / 128) > kNumCU) {
        wide = true;
        const dim3 grid(p.BH * (p.N / 256)), block(512);
        launch_dq(std::integral_constant<int, 8>{}, grid, block);
      }
    }
    if (!wide) {
      const dim3 grid(p.BH * (p.N / 128)), block(256);
      launch_dq(std::integral_constant<int, 4>{}, grid, block);
    }
    if ((e = hipGetLastError()) != hipSuccess) return e;
  }
  return e;
}

hipError_t launch_bwd(const BwdParams& p, int D, hipStream_t stream) {
  switch (D) {
    case 32:  return launch_bwd_t<32>(p, stream);
    case 64:  return launch_bwd_t<64>(p, stream);
    case 128: return launch_bwd_t<128>(p, stream);
    default:  return hipErrorInvalidValue;
  }
}

}  // namespace DA_NS
