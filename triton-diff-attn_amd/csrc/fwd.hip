// Differential-attention forward for gfx950: two online-softmax streams per query row, fused
// lambda-combine and RMSNorm epilogue.  Computes what the reference's forward kernel computes
// (src/kernel.py:20-207) with a different decomposition:
//
//   * a workgroup of 8 waves owns 128 query rows; waves 0-3 run softmax stream 1 (Q1,K1) and
//     waves 4-7 run stream 2 (Q2,K2) for the same rows, 32 rows per wave.  All 8 waves share
//     the K1/K2/V tiles, double-buffered in LDS, and the two streams meet only in the epilogue;
//   * scores are computed transposed, S^T = K * Q^T (K fragments from LDS as the MFMA A operand,
//     Q fragments resident in registers as B), so each lane owns one query column: the row
//     max / row sum are in-lane reductions plus one exchange with lane^32, and the rescale
//     factor, 1/l, lambda-combine and RMSNorm are per-lane scalars;
//   * the P^T accumulator registers are reused directly (after fp16 packing) as the B operand of
//     O^T = V^T * P^T; the V^T A-fragments come from the row-major V tile through the
//     transposing LDS read, using the same key permutation as the accumulator layout.
#include "params.hpp"

namespace da {

template <int D>
struct FwdCfg {
  static constexpr int DV = 2 * D;
  static constexpr int BN = (D <= 64) ? 64 : 32;   // keys per tile
  static constexpr int BM = 128;                   // query rows per workgroup
  static constexpr int NT = 512;                   // threads per workgroup
  static constexpr int KS = D + 8;                 // K row stride in LDS (halfs), 16 B pad
  static constexpr int VS = DV + 32;               // V row stride in LDS (halfs), 64 B pad
  static constexpr int K_TILE = BN * KS;           // halfs
  static constexpr int V_TILE = BN * VS;
  static constexpr int STAGE = 2 * K_TILE + V_TILE;
  static constexpr int XCHG = 4 * (DV / 32) * 16 * 64 * 2;   // halfs needed by the epilogue exchange
  static constexpr int SMEM = (2 * STAGE > XCHG) ? 2 * STAGE : XCHG;
};

template <int D, bool RMS>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2))) void fwd_kernel(FwdParams p) {
  using C = FwdCfg<D>;
  constexpr int DV = C::DV, BN = C::BN, KS = C::KS, VS = C::VS, NT = C::NT, BM = C::BM;
  constexpr int NKS = D / 16;                // k-steps of the score product
  constexpr int NKT = BN / 32;               // 32-key tiles of S^T
  constexpr int NKK = BN / 16;               // k-steps of the P*V product
  constexpr int NOT = DV / 32;               // 32-row tiles of O^T

  __shared__ __attribute__((aligned(16))) half_t smem[C::SMEM];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int st = wave >> 2, qw = wave & 3;   // stream, 32-row block inside the workgroup
  const int j = lane & 31, g = lane >> 5;

  const int n_qt = p.N / BM;
  const int tile = xcd_remap(blockIdx.x, gridDim.x);
  const int bh = tile / n_qt, qt = tile % n_qt;
  const size_t qk_base = (size_t)bh * p.N * D;
  const size_t v_base = (size_t)bh * p.N * DV;
  const int qrow = qt * BM + qw * 32 + j;

  const float c = p.sm_scale * kLog2e;       // scores are handled in log2 units

  // Q fragments (B operand): column j = this lane's query, k = 8g..8g+7 of each 16-wide k-step.
  h8 qf[NKS];
  {
    const half_t* r = (st ? p.q2 : p.q1) + qk_base + (size_t)qrow * D + 8 * g;
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) qf[ks] = *reinterpret_cast<const h8*>(r + 16 * ks);
  }

  f16v o[NOT];
#pragma unroll
  for (int t = 0; t < NOT; ++t)
#pragma unroll
    for (int r = 0; r < 16; ++r) o[t][r] = 0.f;
  float m = -INFINITY, l = 0.f;

  TileStage<BN, D, KS, NT> stK1, stK2;
  TileStage<BN, DV, VS, NT> stV;
  const half_t* gk1 = p.k1 + qk_base;
  const half_t* gk2 = p.k2 + qk_base;
  const half_t* gv = p.v + v_base;

  stK1.load(gk1, tid); stK2.load(gk2, tid); stV.load(gv, tid);
  stK1.store(smem, tid); stK2.store(smem + C::K_TILE, tid); stV.store(smem + 2 * C::K_TILE, tid);
  __syncthreads();

  // per-lane LDS offsets (halfs)
  const int k_off = st * C::K_TILE + j * KS + 8 * g;                        // K A-fragment
  const int v_off = 2 * C::K_TILE + (4 * g + ((lane & 15) >> 2)) * VS + 16 * ((lane >> 4) & 1) + 4 * (lane & 3);

  const int n_tiles = p.N / BN;
  for (int t = 0; t < n_tiles; ++t) {
    const half_t* sK = smem + (t & 1) * C::STAGE + k_off;
    const half_t* sV = smem + (t & 1) * C::STAGE + v_off;
    // prefetch the next tile into registers (the last iteration re-reads its own tile: harmless)
    const int tn = (t + 1 < n_tiles) ? t + 1 : t;
    stK1.load(gk1 + (size_t)tn * BN * D, tid);
    stK2.load(gk2 + (size_t)tn * BN * D, tid);
    stV.load(gv + (size_t)tn * BN * DV, tid);

    f16v s[NKT];
#pragma unroll
    for (int kt = 0; kt < NKT; ++kt) {
#pragma unroll
      for (int r = 0; r < 16; ++r) s[kt][r] = 0.f;
#pragma unroll
      for (int ks = 0; ks < NKS; ++ks) {
        h8 a = *reinterpret_cast<const h8*>(sK + kt * 32 * KS + 16 * ks);
        s[kt] = mfma32(a, qf[ks], s[kt]);
      }
    }
    float mx = s[0][0];
#pragma unroll
    for (int kt = 0; kt < NKT; ++kt)
#pragma unroll
      for (int r = 0; r < 16; ++r) mx = fmaxf(mx, s[kt][r]);
    mx = pair_max(mx);
    const float mnew = fmaxf(m, mx * c);
    const float alpha = fast_exp2(m - mnew);
    m = mnew;
    float rs = 0.f;
    h8 pb[NKK];          // P^T as B operands: pb[kk] covers keys 16kk..16kk+15 (accumulator order)
#pragma unroll
    for (int kt = 0; kt < NKT; ++kt)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        float e = fast_exp2(__builtin_fmaf(s[kt][r], c, -mnew));
        rs += e;
        pb[kt * 2 + r / 8][r % 8] = (half_t)e;
      }
    l = l * alpha + rs;
    if (__any(alpha != 1.0f)) {
#pragma unroll
      for (int tt = 0; tt < NOT; ++tt)
#pragma unroll
        for (int r = 0; r < 16; ++r) o[tt][r] *= alpha;
    }

#pragma unroll
    for (int kk = 0; kk < NKK; ++kk) {
#pragma unroll
      for (int tt = 0; tt < NOT; ++tt) {
        const half_t* vp = sV + (16 * kk) * VS + 32 * tt;
        h8 a = join(lds_read_tr(vp), lds_read_tr(vp + 8 * VS));
        o[tt] = mfma32(a, pb[kk], o[tt]);
      }
    }

    {
      half_t* nb = smem + ((t + 1) & 1) * C::STAGE;
      stK1.store(nb, tid); stK2.store(nb + C::K_TILE, tid); stV.store(nb + 2 * C::K_TILE, tid);
    }
    __syncthreads();
  }

  // ---- epilogue: every quantity below is per query = per lane pair (l, l^32) ----
  l = pair_sum(l);
  const float inv = 1.0f / l;
  const size_t row = (size_t)bh * p.N + qrow;
  {
    float* lse = st ? p.lse2 : p.lse1;
    if (g == 0 && lse) lse[row] = (m + __builtin_log2f(l)) * kLn2;
  }
  // stream-2 waves hand softmax(S2)V to the stream-1 wave that owns the same rows (same lane,
  // same register index), through the now idle tile memory
  float* xchg = reinterpret_cast<float*>(smem) + (size_t)qw * NOT * 16 * 64 + lane;
  if (st == 1) {
    half_t* urow = p.u2 ? p.u2 + row * DV : nullptr;
#pragma unroll
    for (int tt = 0; tt < NOT; ++tt)
#pragma unroll
      for (int r4 = 0; r4 < 4; ++r4) {
        h4 uv;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          float u = o[tt][4 * r4 + e] * inv;
          xchg[(tt * 16 + 4 * r4 + e) * 64] = u;
          uv[e] = (half_t)u;
        }
        if (urow) *reinterpret_cast<h4*>(urow + 32 * tt + 8 * r4 + 4 * g) = uv;
      }
  }
  __syncthreads();
  if (st == 0) {
    const float lam = (float)p.lambda_scale[0];
    float ss = 0.f;
#pragma unroll
    for (int tt = 0; tt < NOT; ++tt)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        float x = o[tt][r] * inv - lam * xchg[(tt * 16 + r) * 64];
        o[tt][r] = x;
        ss += x * x;
      }
    float scale = 1.0f;
    if (RMS) {
      ss = pair_sum(ss);
      const float rr = __builtin_amdgcn_rsqf(ss * (1.0f / DV) + kEps);
      scale = (1.0f - p.lambda_init) * rr;
      if (g == 0 && p.rinv) p.rinv[row] = rr;
    }
    half_t* yrow = p.y + row * DV;
#pragma unroll
    for (int tt = 0; tt < NOT; ++tt)
#pragma unroll
      for (int r4 = 0; r4 < 4; ++r4) {
        h4 yv;
#pragma unroll
        for (int e = 0; e < 4; ++e) yv[e] = (half_t)(o[tt][4 * r4 + e] * scale);
        *reinterpret_cast<h4*>(yrow + 32 * tt + 8 * r4 + 4 * g) = yv;
      }
  }
}

template <int D>
static hipError_t launch_fwd_t(const FwdParams& p, hipStream_t stream) {
  dim3 grid(p.BH * (p.N / FwdCfg<D>::BM)), block(FwdCfg<D>::NT);
  if (p.rms_norm)
    hipLaunchKernelGGL((fwd_kernel<D, true>), grid, block, 0, stream, p);
  else
    hipLaunchKernelGGL((fwd_kernel<D, false>), grid, block, 0, stream, p);
  return hipGetLastError();
}

// Tile-size choice per head dimension (replaces the reference's run-time autotuner,
// src/kernel.py:12-19): 128 query rows per workgroup; 64 keys per step for D <= 64, 32 for D = 128.
hipError_t launch_fwd(const FwdParams& p, int D, hipStream_t stream) {
  switch (D) {
    case 32:  return launch_fwd_t<32>(p, stream);
    case 64:  return launch_fwd_t<64>(p, stream);
    case 128: return launch_fwd_t<128>(p, stream);
    default:  return hipErrorInvalidValue;
  }
}

}  // namespace da
