// Differential-attention forward for gfx950: two online-softmax streams per query row, fused
// lambda-combine and RMSNorm epilogue.  Computes what the reference's forward kernel computes
// (src/kernel.py:20-207) with a different decomposition:
//
//   * a workgroup of 8 waves owns 128 query rows (4 waves and 64 rows for D = 128); waves 0-3 run softmax stream 1 (Q1,K1) and
//     waves 4-7 run stream 2 (Q2,K2) for the same rows, 32 rows per wave.  All 8 waves share
//     the K1/K2/V tiles, double-buffered in LDS, and the two streams meet only in the epilogue;
//   * scores are computed transposed, S^T = K * Q^T (K fragments from LDS as the MFMA A operand,
//     Q fragments resident in registers as B), so each lane owns one query column: the row
//     max / row sum are in-lane reductions plus one exchange with lane^32, and the rescale
//     factor, 1/l, lambda-combine and RMSNorm are per-lane scalars;
//   * the P^T accumulator registers are reused directly (after fp16 packing) as the B operand of
//     O^T = V^T * P^T; the V^T A-fragments come from the row-major V tile through the
//     transposing LDS read, using the same key permutation as the accumulator layout.
#include <type_traits>

#include "params.hpp"

namespace DA_NS {

// SMALL: 64 query rows per workgroup (four waves), for problems whose 128-row blocks do not fill the chip and
// for the D = 128 instantiations that do not fit the register budget of two waves per SIMD.
template <int D, bool SMALL = false>
struct FwdCfg {
  static constexpr int DV = 2 * D;
  static constexpr int BN = (D <= 64) ? 64 : 32;   // keys per tile
  static constexpr int QS = 1;                     // 32-row query blocks per wave
  // query rows per workgroup
  static constexpr int BM = SMALL ? 64 : 128;
  static constexpr int NW = 2 * BM / (32 * QS);    // waves per workgroup: half of them per softmax stream
  static constexpr int NT = NW * 64;
  // waves per SIMD the register budget is sized for: two, except in the four-wave D = 128 workgroups, whose
  // masked and dropout instantiations need more than 256 registers
  static constexpr int OCC = (D == 128 && SMALL) ? 1 : 2;
  // thread count the register budget is derived from: with fewer than 4 * OCC waves in a workgroup the
  // occupancy attribute alone does not hold the allocator to 512 / OCC registers (the four-wave variant at
  // D = 64 then took 336 and shuffled values between the two halves of the register file all through its loop)
  static constexpr int REG_NT = (OCC * 256 > NT) ? OCC * 256 : NT;
  static constexpr int K_TILE = BN * D;            // halfs, one stream (swizzled, unpadded)
  static constexpr int V_TILE = BN * DV;
  static constexpr int K_BUF = 2 * K_TILE;         // K1 and K2 of one tile
  // Ring depth.  Tiles are fetched two iterations ahead, which takes three buffers; there are four so that
  // the loop can be unrolled over one turn of the ring with every buffer known at compile time: an LDS
  // address is then a per-lane register plus an immediate offset, with no arithmetic inside the loop.
  static constexpr int NBUF = 4;
  // A barrier every second tile instead of every tile (the ring allows it): measured in one GPU call,
  // 3.3 % faster at D = 32, 3 % slower at D = 64 and 5 % slower at D = 128.
  static constexpr bool PAIR = (D == 32);
  static constexpr int KBUF_BYTES = K_BUF * 2, VBUF_BYTES = V_TILE * 2, VBASE_BYTES = NBUF * KBUF_BYTES;
  static_assert(NBUF * KBUF_BYTES <= 65536 && NBUF * VBUF_BYTES <= 65536, "immediate offsets reach every buffer");
  static constexpr int TILES = NBUF * (K_BUF + V_TILE);
  // halfs needed by the epilogue: per pair of waves (stream 1, stream 2 of the same 32 rows) an fp32 exchange
  // block of 32 x DV values, which the stream-1 wave reuses for its staged rows, and the staging block
  // (32 rows of DV + 8 halfs) of the stream-2 wave
  // (a block holds the exchange, and after it has been read the staged rows of both waves of the pair)
  static constexpr int XCH_BLOCK = (64 * DV > 2 * 32 * (DV + 8)) ? 64 * DV : 2 * 32 * (DV + 8);
  static constexpr int XCHG = (NW / 2) * XCH_BLOCK;
  static constexpr int SMEM = (TILES > XCHG) ? TILES : XCHG;
};

constexpr float kRescaleThreshold = 8.0f;   // log2 units: probabilities stay below 2^8 between updates of the row max

// MASK: 0 none; 1 causal (key <= query); 2 the last keys of the sequence are padding (key < n_keys).
// With the causal mask the padding needs no extra test: a padded key lies after every real query.
// DROP: dropout on both softmax maps (not in the reference, which lists it as missing,
// src/kernel.py:4): a dropped probability still counts in its row's sum but not in P*V, and the
// kept ones are scaled by 1/(1-p) -- in the epilogue, together with 1/l.
template <int D, bool RMS, int MASK, bool DROP, bool SMALL = false>
__global__ __launch_bounds__((FwdCfg<D, SMALL>::REG_NT)) __attribute__((amdgpu_waves_per_eu(FwdCfg<D, SMALL>::OCC, FwdCfg<D, SMALL>::OCC)))
void fwd_kernel(FwdParams p) {
  using C = FwdCfg<D, SMALL>;
  constexpr int DV = C::DV, BN = C::BN, NW = C::NW, BM = C::BM, QS = C::QS;
  constexpr int NKS = D / 16;                // k-steps of the score product
  constexpr int NKT = BN / 32;               // 32-key tiles of S^T
  constexpr int NKK = BN / 16;               // k-steps of the P*V product
  constexpr int NOT = DV / 32;               // 32-row tiles of O^T

  __shared__ __attribute__((aligned(16))) half_t smem[C::SMEM];
  half_t* const sKbuf = smem;                              // [NBUF][K1 tile, K2 tile]
  half_t* const sVbuf = smem + C::NBUF * C::K_BUF;         // [NBUF][V tile]

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int st = wave / (NW / 2), qw = wave % (NW / 2);   // stream, block of 32*QS rows inside the workgroup
  const int j = lane & 31, g = lane >> 5;

  const int n_qt = p.N / BM;
  constexpr bool CAUSAL = (MASK == 1), PADDED = (MASK == 2);
  // rows past the real length are neither read from the caller's tensors nor written to y: checked in both
  // masked variants (the causal one serves padded sequences too), compiled out of the plain one
  constexpr bool TAIL = (MASK != 0);
  int bh, qt;
  if constexpr (CAUSAL) {   // the last query block of a unit sees the most keys
    const UnitBlock ub = longest_first(blockIdx.x, p.BH);
    bh = ub.unit; qt = n_qt - 1 - ub.rank;
  } else {
    const int tile = xcd_remap(blockIdx.x, gridDim.x);
    bh = tile / n_qt; qt = tile % n_qt;
  }
  // element offsets of the unit's first row and the row strides of its tensors
  const size_t qk_base = da_abi::unit_base(p, p.sqk, bh);
  const size_t v_base = da_abi::unit_base(p, p.sv, bh);
  const int qk_n = (int)p.sqk.n, v_n = (int)p.sv.n;
  const int qrow0 = qt * BM + qw * 32 * QS + j;   // this lane's query row of block qs is qrow0 + 32*qs
  const DropoutKey dkey = dropout_key(p.drop, 2u * bh + st);   // hash key of this wave's softmax stream (used with dropout only)

  // Q fragments (B operand): column j = this lane's query, k = 8g..8g+7 of each 16-wide k-step.
  // They are pre-multiplied by sm_scale*log2(e), so the MFMA result is the score in log2 units.
  h8 qf[QS][NKS];
  {
    const float c = p.sm_scale * kLog2e;
#pragma unroll
    for (int qs = 0; qs < QS; ++qs) {
      // a padding row (past the sequence's real length) stands in with the last real row: finite scores,
      // results that are never stored
      int qr = qrow0 + 32 * qs;
      if (TAIL && qr >= p.n_keys) qr = p.n_keys - 1;
      const half_t* r = (st ? p.q2 : p.q1) + qk_base + (size_t)qr * qk_n + 8 * g;
#pragma unroll
      for (int ks = 0; ks < NKS; ++ks) {
        h8 q = *reinterpret_cast<const h8*>(r + 16 * ks);
#pragma unroll
        for (int e = 0; e < 8; ++e) q[e] = (half_t)((float)q[e] * c);
        qf[qs][ks] = q;
      }
    }
  }

  f16v o[QS][NOT];
#pragma unroll
  for (int qs = 0; qs < QS; ++qs)
#pragma unroll
    for (int t = 0; t < NOT; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r) o[qs][t][r] = 0.f;
  // The running reference m of the online softmax is folded into the score product as the
  // initial accumulator value -m, so the MFMA result is already s - m.
  float m[QS], l[QS];
  f16v negm[QS];
#pragma unroll
  for (int qs = 0; qs < QS; ++qs) {
    m[qs] = 0.f; l[qs] = 0.f;
#pragma unroll
    for (int r = 0; r < 16; ++r) negm[qs][r] = 0.f;
    asm volatile("" : "+v"(negm[qs]));   // sixteen registers of its own: the score products take it as their C operand as it is
  }

  using KTile = AsyncTile<BN, D, NW>;
  using VTile = AsyncTile<BN, DV, NW>;
  const half_t* gk1 = p.k1 + qk_base;
  const half_t* gk2 = p.k2 + qk_base;
  const half_t* gv = p.v + v_base;
  // causal: keys beyond the last row of the workgroup are never visited (BM is a multiple of 2*BN,
  // so the tile count stays even)
  const int n_tiles = CAUSAL ? (qt + 1) * (BM / BN) : p.N / BN;
  static_assert(!CAUSAL || BM % (2 * BN) == 0, "an even number of key tiles per query block");
  constexpr int VH = (VTile::PER + 1) / 2;   // V instructions are issued in two groups
  const unsigned k_off = KTile::lane_off(wave, lane, qk_n), v_off = VTile::lane_off(wave, lane, v_n);
  // With padding, the tiles that reach past the last real row are copied with their row index clamped to it.
  // `tail` (a compile-time tag) says whether the call site can meet such a tile at all.
  auto load_k1 = [&](int tk, int buf, auto tail) {
    if (TAIL && decltype(tail)::value && (tk + 1) * BN > p.n_keys)
      KTile::issue_clamped(gk1 + (size_t)tk * BN * qk_n, sKbuf + buf * C::K_BUF, wave, lane, k_off, qk_n, p.n_keys - 1 - tk * BN);
    else
      KTile::issue_at(gk1 + (size_t)tk * BN * qk_n, sKbuf + buf * C::K_BUF, wave, lane, k_off, qk_n);
  };
  auto load_k2 = [&](int tk, int buf, auto tail) {
    if (TAIL && decltype(tail)::value && (tk + 1) * BN > p.n_keys)
      KTile::issue_clamped(gk2 + (size_t)tk * BN * qk_n, sKbuf + buf * C::K_BUF + C::K_TILE, wave, lane, k_off, qk_n, p.n_keys - 1 - tk * BN);
    else
      KTile::issue_at(gk2 + (size_t)tk * BN * qk_n, sKbuf + buf * C::K_BUF + C::K_TILE, wave, lane, k_off, qk_n);
  };
  auto load_va = [&](int tv, int buf, auto tail) {
    if (TAIL && decltype(tail)::value && (tv + 1) * BN > p.n_keys)
      VTile::template issue_clamped<0, VH>(gv + (size_t)tv * BN * v_n, sVbuf + buf * C::V_TILE, wave, lane, v_off, v_n, p.n_keys - 1 - tv * BN);
    else
      VTile::template issue_at<0, VH>(gv + (size_t)tv * BN * v_n, sVbuf + buf * C::V_TILE, wave, lane, v_off, v_n);
  };
  auto load_vb = [&](int tv, int buf, auto tail) {
    if (TAIL && decltype(tail)::value && (tv + 1) * BN > p.n_keys)
      VTile::template issue_clamped<VH, VTile::PER>(gv + (size_t)tv * BN * v_n, sVbuf + buf * C::V_TILE, wave, lane, v_off, v_n, p.n_keys - 1 - tv * BN);
    else
      VTile::template issue_at<VH, VTile::PER>(gv + (size_t)tv * BN * v_n, sVbuf + buf * C::V_TILE, wave, lane, v_off, v_n);
  };
  constexpr std::true_type with_tail{};
  constexpr std::false_type no_tail{};

  // Per-lane LDS byte addresses, computed once.  The XOR swizzle makes the address of a fragment a
  // different function of the lane for every 16-byte chunk column, so there is one register per chunk
  // column a lane reads; the ring buffer, the 32-key block and the k-step of 16 keys are multiples of 16
  // rows, which the swizzle does not see, and travel in the instructions' immediate offsets.
  // transposing-read coordinates of this lane inside a 16-key k-step: key row and feature column
  const int tr_row = 4 * g + ((lane & 15) >> 2);
  const int tr_col = 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
  const unsigned lds0 = (unsigned)(unsigned long)((DA_LDS char*)smem);
  unsigned kb[NKS], vtr[NOT][2];
#pragma unroll
  for (int ks = 0; ks < NKS; ++ks) kb[ks] = lds0 + 2u * (unsigned)(st * C::K_TILE + swz_off<D>(j, 16 * ks + 8 * g));
#pragma unroll
  for (int tt = 0; tt < NOT; ++tt)
#pragma unroll
    for (int e = 0; e < 2; ++e) vtr[tt][e] = lds0 + C::VBASE_BYTES + 2u * (unsigned)swz_off<DV>(tr_row + 8 * e, 32 * tt + tr_col);
  // kept as they are: the compiler neither folds constants into them nor recomputes them in the loop
#pragma unroll
  for (int ks = 0; ks < NKS; ++ks) asm volatile("" : "+v"(kb[ks]));
#pragma unroll
  for (int tt = 0; tt < NOT; ++tt) asm volatile("" : "+v"(vtr[tt][0]), "+v"(vtr[tt][1]));

  // A-fragments of K for all k-steps of all 32-key tiles: row kt*32 + j, halfs 16ks + 8g .. +7
  auto read_k = [&](int byte_off, h8 (&ka)[NKT][NKS]) {
#pragma unroll
    for (int kt = 0; kt < NKT; ++kt)
#pragma unroll
      for (int ks = 0; ks < NKS; ++ks) ka[kt][ks] = lds_read_at<h8>(kb[ks], byte_off + kt * 32 * D * 2);
  };
  // Score products number I0 .. I1-1 of a tile, counted in issue order: 32-key tile kt, k-step ks is number
  // kt * NKS + ks.  The first product of a 32-key tile starts from the running reference.
  auto scores_of = [&](const h8 (&ka)[NKT][NKS], f16v (&s)[QS][NKT], auto i0, auto i1) {
#pragma unroll
    for (int i = decltype(i0)::value; i < decltype(i1)::value; ++i) {
      const int kt = i / NKS, ks = i % NKS;
#pragma unroll
      for (int qs = 0; qs < QS; ++qs) {
        if (ks == 0) s[qs][kt] = negm[qs];
        s[qs][kt] = mfma32(ka[kt][ks], qf[qs][ks], s[qs][kt]);
      }
    }
  };
  constexpr int NSC = NKT * NKS;      // score products per tile and 32-row block
  auto scores = [&](const h8 (&ka)[NKT][NKS], f16v (&s)[QS][NKT]) {
    scores_of(ka, s, std::integral_constant<int, 0>{}, std::integral_constant<int, NSC>{});
  };
  // How many of the next tile's score products are issued ahead of the row maxima of this one; the rest follow
  // the reference update and run under the first exponentials, which have no other matrix work beside them.
  // The split is between 32-key tiles.  Measured against all of them ahead, inside one GPU call each: the
  // first of two tiles ahead -2.5 % at D = 64 (0.442 -> 0.432 ms) and -1 % at D = 32; none ahead the same at
  // D = 64 and +0.7 % at D = 128; a D = 128 tile is a single 32-key tile, and splitting it in the middle
  // of its k-steps cost 1.5 %, so it stays whole and ahead.
  constexpr int SC_EARLY = DROP ? NSC : ((NKT + 1) / 2) * NKS;
  constexpr int KT_EARLY = (SC_EARLY + NKS - 1) / NKS;     // 32-key tiles whose first product is among them
  constexpr std::integral_constant<int, 0> sc_first{};
  constexpr std::integral_constant<int, SC_EARLY> sc_split{};
  constexpr std::integral_constant<int, NSC> sc_end{};

  // loads this wave issues per iteration (one K1, one K2 and one V tile)
  const int loads_per_iter = 2 * KTile::count(wave) + VTile::count(wave);
  auto clampt = [&](int t) { return t < n_tiles ? t : n_tiles - 1; };   // past the end: harmless re-reads

  // The loop below runs whole turns of the ring (NBUF iterations); the tile count is even, so when it is
  // not a multiple of four, half a turn comes first and tile 0 goes into buffer 2: tile t is in buffer
  // (t + b0) % NBUF, b0 = 0 or 2.
  static_assert(C::NBUF == 4, "the loop is unrolled over a ring of four");
  const bool head_half = (n_tiles & 2) != 0;
  const int b0 = head_half ? 2 : 0;
  // prologue: K tiles 0..2 and V tiles 0..1; scores of tile 0
  load_k1(0, b0, with_tail); load_k2(0, b0, with_tail); load_va(0, b0, with_tail); load_vb(0, b0, with_tail);
  load_k1(clampt(1), b0 + 1, with_tail); load_k2(clampt(1), b0 + 1, with_tail);
  load_va(clampt(1), b0 + 1, with_tail); load_vb(clampt(1), b0 + 1, with_tail);
  load_k1(clampt(2), (b0 + 2) % 4, with_tail); load_k2(clampt(2), (b0 + 2) % 4, with_tail);
  wait_async_tiles();
  __syncthreads();
  f16v s_a[QS][NKT], s_b[QS][NKT];
  {
    h8 ka[NKT][NKS];
    if (head_half) read_k(2 * C::KBUF_BYTES, ka);
    else read_k(0, ka);
    scores(ka, s_a);
  }

  // One iteration: softmax of tile t (scores in s_cur) and its P*V product, overlapped with the score
  // product of tile t+1 (into s_nxt).
  // POS = (t + b0) % NBUF is the ring position: K tile t+1 is read from buffer POS+1 and V tile t from
  // buffer POS; K tile t+3 goes to buffer POS+3 (tile t-1, consumed two iterations ago) and V tile t+2 to
  // buffer POS+2 (tile t-2, likewise), all modulo NBUF.
  // `tail`: the iteration can meet tiles that reach past the last real key (their copies are clamped and, in
  // the padded variant, their keys masked); iterations that cannot are compiled without those tests.
  auto iteration = [&](int t, auto pos_tag, auto tail, f16v (&s_cur)[QS][NKT], f16v (&s_nxt)[QS][NKT]) {
    constexpr int POS = decltype(pos_tag)::value;
    constexpr int KR = (POS + 1) % 4, KP = (POS + 3) % 4, VR = POS, VP = (POS + 2) % 4;
    // Asynchronous prefetch straight into LDS, two iterations ahead: K tile t+3 and V tile t+2.
    // The groups of load instructions are spread over the iteration so that the waves do not
    // queue up behind each other at the memory pipeline.
    const int tk = clampt(t + 3);
    const int tv = clampt(t + 2);
    load_k1(tk, KP, tail);

    // K fragments of the next tile are requested first; the row maxima of this tile are reduced
    // while they arrive.
    h8 ka[NKT][NKS];
    read_k(KR * C::KBUF_BYTES, ka);

    if constexpr (CAUSAL) {
      // only the last tiles of a wave's loop reach past its first row: mask key > query there
      static_assert(QS == 1, "one 32-row block per wave");
      const int wrow0 = qt * BM + qw * 32;
      if ((t + 1) * BN - 1 > wrow0) {
        const int rel = wrow0 + j - t * BN - 4 * g;      // query index minus the key index of register 0, tile 0
#pragma unroll
        for (int kt = 0; kt < NKT; ++kt)
#pragma unroll
          for (int r = 0; r < 16; ++r)
            if (kt * 32 + 8 * (r / 4) + (r % 4) > rel) s_cur[0][kt][r] = -INFINITY;
      }
    }

    if constexpr (PADDED && decltype(tail)::value) {
      // only the last tiles hold padding keys
      if ((t + 1) * BN > p.n_keys) {
        const int rel = p.n_keys - 1 - t * BN - 4 * g;   // last real key minus the key index of register 0, tile 0
#pragma unroll
        for (int kt = 0; kt < NKT; ++kt)
#pragma unroll
          for (int r = 0; r < 16; ++r)
            if (kt * 32 + 8 * (r / 4) + (r % 4) > rel) s_cur[0][kt][r] = -INFINITY;
      }
    }

    // The score product of the next tile goes to the matrix unit first and runs under the row maxima and
    // the exponentials of this tile.  It starts from the running reference as it stands before this
    // tile's update; when the update moves the reference, the few results are corrected with it.
    load_k2(tk, KP, tail);
    scores_of(ka, s_nxt, sc_first, sc_split);

    float mx[QS];
#pragma unroll
    for (int qs = 0; qs < QS; ++qs) {
      float mx0 = fmaxf(s_cur[qs][0][0], s_cur[qs][0][1]), mx1 = fmaxf(s_cur[qs][0][2], s_cur[qs][0][3]);
      float mx2 = fmaxf(s_cur[qs][0][4], s_cur[qs][0][5]), mx3 = fmaxf(s_cur[qs][0][6], s_cur[qs][0][7]);
#pragma unroll
      for (int kt = 0; kt < NKT; ++kt)
#pragma unroll
        for (int r = (kt == 0 ? 8 : 0); r < 16; r += 8) {
          mx0 = fmaxf(mx0, fmaxf(s_cur[qs][kt][r + 0], s_cur[qs][kt][r + 1]));
          mx1 = fmaxf(mx1, fmaxf(s_cur[qs][kt][r + 2], s_cur[qs][kt][r + 3]));
          mx2 = fmaxf(mx2, fmaxf(s_cur[qs][kt][r + 4], s_cur[qs][kt][r + 5]));
          mx3 = fmaxf(mx3, fmaxf(s_cur[qs][kt][r + 6], s_cur[qs][kt][r + 7]));
        }
      mx[qs] = fmaxf(fmaxf(mx0, mx1), fmaxf(mx2, mx3));
    }
    float mxall = mx[0];
#pragma unroll
    for (int qs = 1; qs < QS; ++qs) mxall = fmaxf(mxall, mx[qs]);
    // The reference only moves when some row of the wave outgrew it by more than the threshold
    // (always on the first tile, where it starts at 0 with nothing accumulated yet).
    if (__any(mxall > kRescaleThreshold) || t == 0) {
#pragma unroll
      for (int qs = 0; qs < QS; ++qs) {
        const float pm = pair_max(mx[qs]);
        const float d = (t == 0) ? pm : fmaxf(pm, 0.f);
        const float alpha = fast_exp2(-d);
        m[qs] += d;
        l[qs] *= alpha;
#pragma unroll
        for (int tt = 0; tt < NOT; ++tt)
#pragma unroll
          for (int r = 0; r < 16; ++r) o[qs][tt][r] *= alpha;
#pragma unroll
        for (int kt = 0; kt < NKT; ++kt)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            s_cur[qs][kt][r] -= d;
            if (kt < KT_EARLY) s_nxt[qs][kt][r] -= d;     // the later ones start from the new reference
          }
#pragma unroll
        for (int r = 0; r < 16; ++r) negm[qs][r] = -m[qs];
        asm volatile("" : "+v"(negm[qs]));
      }
    }

    // From here on one basic block: the P*V product of this tile runs on the matrix unit while the
    // exponentials run on the VALU.
    // dropout: the mask arithmetic needs the registers of the K fragments, so the score product is
    // issued in full before the exponentials instead of between them
    if constexpr (DROP) __builtin_amdgcn_sched_barrier(0);

    // V^T fragments are requested PD products ahead of the product that uses them (measured: 2 and
    // 3 are 1.3 % faster than the single product the compiler picks by itself, 5 and 7 are not); the
    // first ones here, so that they arrive under the exponentials
    constexpr int NPV = NKK * NOT;
    constexpr int PD = DROP ? 1 : 3;           // dropout: registers are short
    auto vt_frag = [&](int i) {
      const int kk = i / NOT, tt = i % NOT;
      const int off = VR * C::VBUF_BYTES + 16 * kk * DV * 2;
      return join(lds_read_tr_at(vtr[tt][0], off), lds_read_tr_at(vtr[tt][1], off));
    };
    h8 vfr[NPV];
    if constexpr (!DROP) {
#pragma unroll
      for (int i = 0; i < PD && i < NPV; ++i) vfr[i] = vt_frag(i);
    }
    scores_of(ka, s_nxt, sc_split, sc_end);

    // P^T as B operands: pb[kk] covers keys 16kk..16kk+15 (accumulator order).  Built from the packed
    // pairs as 32-bit words, so that each pair is converted once, for the row sum and the operand alike.
    u32x4 pw[QS][NKK];
#pragma unroll
    for (int qs = 0; qs < QS; ++qs) {
      float rs = 0.f;
      unsigned word_a = 0, word_b = 0;     // dropout: hash words of two neighbouring 2x2 blocks
#pragma unroll
      for (int kt = 0; kt < NKT; ++kt)
#pragma unroll
        for (int r = 0; r < 16; r += 2) {
          h2 e2;
          e2[0] = (half_t)fast_exp2(s_cur[qs][kt][r]);
          e2[1] = (half_t)fast_exp2(s_cur[qs][kt][r + 1]);
          rs = add_pair(e2, rs);   // row sum of the rounded probabilities
          unsigned w2 = __builtin_bit_cast(unsigned, e2);
          if constexpr (DROP) {
            // registers r, r+1 hold the keys key, key+1 (key even) of this lane's query; the blocks of registers
            // r..r+1 and r+2..r+3 (r a multiple of 4) are neighbours, hashed one by each lane of a query pair
            const unsigned query = (unsigned)(qrow0 + 32 * qs);
            const unsigned key = (unsigned)(t * BN + kt * 32 + 8 * (r / 4) + 4 * g + (r % 4));
            if (r % 4 == 0)
              dropout_words_shared(dropout_word(dkey, (unsigned)p.N / 2, query >> 1, (key >> 1) + (query & 1)), query & 1,
                                   word_a, word_b);
            const unsigned word = (r % 4 == 0) ? word_a : word_b;
            w2 &= (dropout_keep(word, query, key, p.drop.threshold) ? 0x0000ffffu : 0u) |
                  (dropout_keep(word, query, key + 1, p.drop.threshold) ? 0xffff0000u : 0u);
          }
          pw[qs][kt * 2 + r / 8][(r % 8) / 2] = w2;
        }
      l[qs] += rs;
    }

    if constexpr (DROP) {
#pragma unroll
      for (int i = 0; i < PD && i < NPV; ++i) vfr[i] = vt_frag(i);
    }
#pragma unroll
    for (int i = 0; i < NPV; ++i) {
      const int kk = i / NOT, tt = i % NOT;
      if (i == 0) load_va(tv, VP, tail);
      if (i == NPV / 2) load_vb(tv, VP, tail);
      if (i + PD < NPV) vfr[i + PD] = vt_frag(i + PD);
#pragma unroll
      for (int qs = 0; qs < QS; ++qs) o[qs][tt] = mfma32(vfr[i], __builtin_bit_cast(h8, pw[qs][kk]), o[qs][tt]);
    }

    // the tiles needed next were requested one iteration ago: only this iteration's loads may remain
    if constexpr (C::PAIR) {
      // the ring of four lets the workgroup meet every second tile only: the copies for the next two tiles
      // (requested during the last two) have landed for everybody, and the last two buffers may be refilled
      if constexpr (POS & 1) { wait_async_tiles(); __syncthreads(); }
    } else {
      wait_async_tiles_except(loads_per_iter);
      __syncthreads();
    }
  };

  // the tile count is even (N is a multiple of 128, tiles are at most 64 keys)
  int t = 0;
  if (head_half) {
    iteration(0, std::integral_constant<int, 2>{}, with_tail, s_a, s_b);
    iteration(1, std::integral_constant<int, 3>{}, with_tail, s_b, s_a);
    t = 2;
  }
  auto turn = [&](int t, auto tail) {
    iteration(t, std::integral_constant<int, 0>{}, tail, s_a, s_b);
    iteration(t + 1, std::integral_constant<int, 1>{}, tail, s_b, s_a);
    iteration(t + 2, std::integral_constant<int, 2>{}, tail, s_a, s_b);
    iteration(t + 3, std::integral_constant<int, 3>{}, tail, s_b, s_a);
  };
  if constexpr (PADDED) {
    // Padding concerns the last tiles only: an iteration copies K tile t+3, so the first one that can touch a
    // tile with padding rows is number n_keys / BN - 3.  Whole turns in front of it run without the tests.
    const int t_tail = p.n_keys / BN - 3;
#pragma nounroll
    for (; t + 4 <= t_tail; t += 4) turn(t, no_tail);
  }
#pragma nounroll
  for (; t < n_tiles; t += 4) turn(t, with_tail);

  wait_async_tiles();   // the staging blocks below reuse the tile memory the last prefetches write to
  __syncthreads();
  // ---- epilogue ----------------------------------------------------------------------------
  // Every row quantity is per query = per lane pair (l, l^32).  Each wave has a staging block of
  // 32 rows x DV halfs in the now idle tile memory (row stride DV+8 halfs).  Results are written
  // there in accumulator layout (8 bytes per lane) and read back row by row, so that the global
  // stores are whole 16-byte chunks of consecutive rows.  The stream-2 waves stage softmax(S2)V
  // rounded to 16 bits -- the tensor saved for backward -- and also hand it, unrounded, to the stream-1
  // wave that owns the same rows: the lambda-combine is formed in fp32, as in the reference
  // (src/kernel.py:191-194), so that rows in which the two streams nearly cancel (lambda near 1, similar
  // attention maps) do not see the rounding error of one stream amplified by the norm.  The two waves
  // hold a row's values in the same lanes and registers, so the exchange is lane to lane.
  // Each pair of waves has one block of tile memory: first it carries the fp32 exchange, then, once the
  // workgroup has met behind the combine, the staged rows of the two waves side by side.
  constexpr int SROW = DV + 8;
  float* const xch = reinterpret_cast<float*>(smem + (size_t)qw * C::XCH_BLOCK);
  half_t* const stg_own = smem + (size_t)qw * C::XCH_BLOCK + (st ? 32 * SROW : 0);
  auto stage_rows = [&](int qs, const f16v (&val)[NOT], float scale) {
#pragma unroll
    for (int tt = 0; tt < NOT; ++tt)
#pragma unroll
      for (int r4 = 0; r4 < 4; ++r4) {
        h4 v;
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = (half_t)(val[tt][4 * r4 + e] * scale);
        *reinterpret_cast<h4*>(stg_own + j * SROW + 32 * tt + 8 * r4 + 4 * g) = v;
      }
    (void)qs;
  };
  // `rows`: how many of the wave's 32 rows exist in the destination (32 unless the sequence is padded and
  // the destination is the caller's tensor, which has no rows past the real length)
  auto store_rows = [&](half_t* gbase /* first of this wave's 32 rows */, size_t row_stride, int rows) {
    constexpr int LPR = DV / 8;            // lanes per row
    constexpr int RPI = 64 / LPR;          // rows per instruction
#pragma unroll
    for (int k = 0; k < 32 / RPI; ++k) {
      const int row = k * RPI + lane / LPR, ch = lane % LPR;
      const u32x4 v = *reinterpret_cast<const u32x4*>(stg_own + row * SROW + 8 * ch);
      if (!TAIL || row < rows) *reinterpret_cast<u32x4*>(gbase + (size_t)row * row_stride + 8 * ch) = v;
    }
  };

  static_assert(QS == 1, "the epilogue stages one 32-row block per wave");
  const float lsum = pair_sum(l[0]);
  const float inv = (DROP ? p.drop.keep_scale : 1.0f) / lsum;
  const size_t row = (size_t)bh * p.N + qrow0;
  const size_t wave_row0 = (size_t)bh * p.N + qt * BM + qw * 32;
  {
    float* lse = st ? p.lse2 : p.lse1;
    if (g == 0 && lse) lse[row] = (m[0] + __builtin_log2f(lsum)) * kLn2;
  }
  if (st == 1) {
#pragma unroll
    for (int tt = 0; tt < NOT; ++tt)
#pragma unroll
      for (int r4 = 0; r4 < 4; ++r4) {
        f4v u;
#pragma unroll
        for (int e = 0; e < 4; ++e) u[e] = o[0][tt][4 * r4 + e] * inv;
        *reinterpret_cast<f4v*>(xch + ((tt * 4 + r4) * 64 + lane) * 4) = u;
      }
  }
  __syncthreads();
  const float lam = da_abi::lambda_of_unit(p, bh);
  float ss = 0.f;
  if (st == 0) {
#pragma unroll
    for (int tt = 0; tt < NOT; ++tt)
#pragma unroll
      for (int r4 = 0; r4 < 4; ++r4) {
        const f4v u = *reinterpret_cast<const f4v*>(xch + ((tt * 4 + r4) * 64 + lane) * 4);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const float x = o[0][tt][4 * r4 + e] * inv - lam * u[e];
          o[0][tt][4 * r4 + e] = x;
          ss += x * x;
        }
      }
  }
  __syncthreads();      // the exchange has been read: the blocks may take the staged rows
  if (st == 1) {
    stage_rows(0, o[0], inv);
    __builtin_amdgcn_wave_barrier();   // the rows are read back by other lanes of this wave only
    if (p.u2) store_rows(p.u2 + wave_row0 * DV, DV, 32);
  } else {
    float scale = 1.0f;
    if (RMS) {
      ss = pair_sum(ss);
      const float rr = __builtin_amdgcn_rsqf(ss * (1.0f / DV) + kEps);
      scale = (1.0f - p.lambda_init) * rr;
      if (g == 0 && p.rinv) p.rinv[row] = rr;
    }
    stage_rows(0, o[0], scale);
    __builtin_amdgcn_wave_barrier();   // the rows are read back by other lanes of this wave only
    store_rows(p.y + da_abi::unit_base(p, p.sy, bh) + (size_t)(qt * BM + qw * 32) * (size_t)p.sy.n, (size_t)p.sy.n,
               p.n_keys - (qt * BM + qw * 32));
  }
}

template <int D, bool RMS, bool DROP, bool SMALL>
static void launch_fwd_c(const FwdParams& p, hipStream_t stream) {
  using C = FwdCfg<D, SMALL>;
  const dim3 grid(p.BH * (p.N / C::BM)), block(C::NT);
  if (p.causal)
    hipLaunchKernelGGL((fwd_kernel<D, RMS, 1, DROP, SMALL>), grid, block, 0, stream, p);
  else if (p.n_keys < p.N)
    hipLaunchKernelGGL((fwd_kernel<D, RMS, 2, DROP, SMALL>), grid, block, 0, stream, p);
  else
    hipLaunchKernelGGL((fwd_kernel<D, RMS, 0, DROP, SMALL>), grid, block, 0, stream, p);
}

template <int D>
static hipError_t launch_fwd_t(const FwdParams& p, hipStream_t stream) {
  const bool drop = p.drop.threshold != 0;
  const bool plain = !p.causal && !drop && p.n_keys == p.N;
  // Shape-aware launch geometry (the reference autotunes its tiles per (N, D, Dv), src/kernel.py:12-19): a problem
  // whose 128-row blocks do not fill the chip once runs in twice as many 64-row, four-wave workgroups.  A pure
  // function of (B*H, N, D) and the options: no tuning state.  At D <= 64 only the plain instantiation has the
  // small variant.  At D = 128 it is the other way round: only the plain instantiation fits the 256 registers of
  // the 128-row workgroup (two waves per SIMD); with a mask or dropout the kernel runs in 64-row workgroups at one
  // wave per SIMD.
  constexpr int kNumCU = 256;
  const bool small_grid = (long long)p.BH * (p.N / 128) < kNumCU;
  if constexpr (D == 128) {
    if (!plain || small_grid) {
      if (p.rms_norm) { if (drop) launch_fwd_c<D, true, true, true>(p, stream); else launch_fwd_c<D, true, false, true>(p, stream); }
      else            { if (drop) launch_fwd_c<D, false, true, true>(p, stream); else launch_fwd_c<D, false, false, true>(p, stream); }
    } else {
      const dim3 grid(p.BH * (p.N / FwdCfg<D>::BM)), block(FwdCfg<D>::NT);
      if (p.rms_norm) hipLaunchKernelGGL((fwd_kernel<D, true, 0, false, false>), grid, block, 0, stream, p);
      else            hipLaunchKernelGGL((fwd_kernel<D, false, 0, false, false>), grid, block, 0, stream, p);
    }
    return hipGetLastError();
  } else {
    if (plain && small_grid) {
      const dim3 sgrid(p.BH * (p.N / FwdCfg<D, true>::BM)), sblock(FwdCfg<D, true>::NT);
      if (p.rms_norm) hipLaunchKernelGGL((fwd_kernel<D, true, 0, false, true>), sgrid, sblock, 0, stream, p);
      else            hipLaunchKernelGGL((fwd_kernel<D, false, 0, false, true>), sgrid, sblock, 0, stream, p);
      return hipGetLastError();
    }
    if (p.rms_norm) { if (drop) launch_fwd_c<D, true, true, false>(p, stream); else launch_fwd_c<D, true, false, false>(p, stream); }
    else            { if (drop) launch_fwd_c<D, false, true, false>(p, stream); else launch_fwd_c<D, false, false, false>(p, stream); }
    return hipGetLastError();
  }
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

}  // namespace DA_NS
