// Shared device helpers for the gfx950 differential-attention kernels.
//
// MFMA register layouts used throughout (wave64, verified on hardware):
//   v_mfma_f32_32x32x16_f16  D[32x32] += A[32x16] * B[16x32]
//     A operand: lane l holds row (l % 32), k = 8*(l / 32) .. +7   (8 halfs = 4 VGPRs)
//     B operand: lane l holds col (l % 32), k = 8*(l / 32) .. +7
//     C/D      : lane l holds col (l % 32); register r (0..15) is row 8*(r/4) + 4*(l/32) + (r%4)
//   ds_read_b64_tr_b16: inside each block of 16 lanes, lane n supplies the address of 4 consecutive
//     halfs of "row n/4, column chunk n%4"; lane n receives element n of rows 0..3 (a 4x16
//     transpose), i.e. result[j] = data of lane (4*j + n/4), element (n % 4).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

// The sources are compiled twice into one library: as they stand for fp16 tensors (namespace da),
// and with -DDA_BF16 for bf16 tensors (namespace da_bf16).  "half" in comments means the 16-bit
// element type of the build; everything that differs between the two is in this header.
#ifdef DA_BF16
#define DA_NS da_bf16
#define DA_MFMA_32x32x16 "v_mfma_f32_32x32x16_bf16"
#else
#define DA_NS da
#define DA_MFMA_32x32x16 "v_mfma_f32_32x32x16_f16"
#endif

namespace da_abi {
// dropout parameters as the kernels see them (one definition for both builds)
struct DropoutCfg {
  unsigned seed_lo, seed_hi;
  unsigned threshold;           // 0 (no dropout) .. 255: a pair is kept iff its random byte >= threshold
  float keep_scale;             // 1 / (1 - threshold/256)
};
}  // namespace da_abi

namespace DA_NS {

#ifdef DA_BF16
typedef __bf16 half_t;
typedef __bf16 h2 __attribute__((ext_vector_type(2)));
typedef __bf16 h4 __attribute__((ext_vector_type(4)));
typedef __bf16 h8 __attribute__((ext_vector_type(8)));
#else
typedef _Float16 half_t;
typedef _Float16 h2 __attribute__((ext_vector_type(2)));
typedef _Float16 h4 __attribute__((ext_vector_type(4)));
typedef _Float16 h8 __attribute__((ext_vector_type(8)));
#endif
typedef float f16v __attribute__((ext_vector_type(16)));
typedef float f4v __attribute__((ext_vector_type(4)));
typedef __fp16 tr4 __attribute__((vector_size(8)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;
constexpr float kEps = 1e-5f;

#define DA_LDS __attribute__((address_space(3)))

__device__ __forceinline__ f16v mfma32(h8 a, h8 b, f16v c) {
#ifdef DA_BF16
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
#else
  return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
#endif
}

// acc + x[0]*1 + x[1]*1 in one instruction: the sum of two rounded 16-bit values in fp32
__device__ __forceinline__ float add_pair(h2 x, float acc) {
  const h2 ones = {(half_t)1.0f, (half_t)1.0f};
#ifdef DA_BF16
  return __builtin_amdgcn_fdot2_f32_bf16(x, ones, acc, false);
#else
  return __builtin_amdgcn_fdot2(x, ones, acc, false);
#endif
}

// acc + a[0]*b[0] + a[1]*b[1] in one instruction, the products of 16-bit values exact and summed in fp32
__device__ __forceinline__ float dot_pair(h2 a, h2 b, float acc) {
#ifdef DA_BF16
  return __builtin_amdgcn_fdot2_f32_bf16(a, b, acc, false);
#else
  return __builtin_amdgcn_fdot2(a, b, acc, false);
#endif
}

// MFMA with the B operand held in an accumulation register (AGPR) and the result in ordinary
// VGPRs.  Used where B is a loop-invariant fragment: it then lives in the AGPR half of the register
// file for the whole kernel, at no cost in VGPRs and without copies.  Being inline assembly, the
// compiler does not know these are matrix instructions: the caller must put mfma_results_ready()
// between the last of them and the first VALU read of the result.
__device__ __forceinline__ f16v mfma32_bagpr(h8 a, h8 b, f16v c) {
  asm volatile(DA_MFMA_32x32x16 " %0, %1, %2, %0" : "+v"(c) : "v"(a), "a"(b));
  return c;
}
// The same, starting a sum: C is the constant zero.
__device__ __forceinline__ f16v mfma32_bagpr_first(h8 a, h8 b) {
  f16v c;
  asm volatile(DA_MFMA_32x32x16 " %0, %1, %2, 0" : "=&v"(c) : "v"(a), "a"(b));
  return c;
}
// The same, starting from a given accumulator value that stays as it is.
__device__ __forceinline__ f16v mfma32_bagpr_from(h8 a, h8 b, const f16v& c0) {
  f16v c;
  asm volatile(DA_MFMA_32x32x16 " %0, %1, %2, %3" : "=&v"(c) : "v"(a), "a"(b), "v"(c0));
  return c;
}
// Moves a fragment into AGPRs for good: after this the value is defined by an (empty) asm statement
// with an AGPR output, so the compiler has no VGPR original to copy from in front of a later use.
// A v_accvgpr_write directly in front of an inline-asm MFMA that reads the AGPR is a hazard the
// compiler covers for its own MFMAs only: the MFMA was observed to read the old register content.
__device__ __forceinline__ void keep_in_agpr(h8& x) { asm volatile("" : "+a"(x)); }

// Wait states that cover the write-back of an 8-pass MFMA before a VALU instruction reads it.
__device__ __forceinline__ void mfma_results_ready(f16v& x, f16v& y, f16v& z) {
  asm volatile("s_nop 15\n\ts_nop 3" : "+v"(x), "+v"(y), "+v"(z));
}
__device__ __forceinline__ void mfma_results_ready(f16v& x, f16v& y) {
  asm volatile("s_nop 15\n\ts_nop 3" : "+v"(x), "+v"(y));
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// v_permlane32_swap exchanges the upper half of its first register with the lower half of its
// second one.  Fed the same value in two DISTINCT registers it leaves (lower-half value,
// upper-half value) of the lane pair (l, l^32) in every lane.  The empty asm keeps the compiler
// from merging the two copies into one register, which would turn the swap into a self-swap.
struct LanePair { float lo, hi; };
__device__ __forceinline__ LanePair lane_pair(float x) {
  unsigned a = __builtin_bit_cast(unsigned, x), b = a;
  asm volatile("" : "+v"(b));
  auto r = __builtin_amdgcn_permlane32_swap(a, b, false, false);
  LanePair p;
  p.lo = __builtin_bit_cast(float, (unsigned)r[0]);
  p.hi = __builtin_bit_cast(float, (unsigned)r[1]);
  return p;
}
__device__ __forceinline__ float pair_max(float x) { LanePair p = lane_pair(x); return fmaxf(p.lo, p.hi); }
__device__ __forceinline__ float pair_sum(float x) { LanePair p = lane_pair(x); return p.lo + p.hi; }

// 4x16 transposing LDS read (see header comment); p must be 8-byte aligned.
__device__ __forceinline__ h4 lds_read_tr(const half_t* p) {
#ifdef DA_BF16
  typedef short tr4i __attribute__((ext_vector_type(4)));
  tr4i v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((DA_LDS tr4i*)(p));
#else
  tr4 v = __builtin_amdgcn_ds_read_tr16_b64_v4f16((DA_LDS tr4*)(p));
#endif
  return __builtin_bit_cast(h4, v);
}

// The same read, and a plain 16-byte read, at an LDS byte address (a 32-bit integer) plus a constant:
// the constant travels in the instruction's immediate offset field.
__device__ __forceinline__ h4 lds_read_tr_at(unsigned addr, int off) {
  DA_LDS char* p = (DA_LDS char*)(unsigned long)addr + off;
#ifdef DA_BF16
  typedef short tr4i __attribute__((ext_vector_type(4)));
  tr4i v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((DA_LDS tr4i*)p);
#else
  tr4 v = __builtin_amdgcn_ds_read_tr16_b64_v4f16((DA_LDS tr4*)p);
#endif
  return __builtin_bit_cast(h4, v);
}
template <class V>
__device__ __forceinline__ V lds_read_at(unsigned addr, int off) {
  return *(const DA_LDS V*)((DA_LDS char*)(unsigned long)addr + off);
}

__device__ __forceinline__ h8 join(h4 lo, h4 hi) {
  return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
}

#define DA_GLOBAL __attribute__((address_space(1)))

// ---- LDS tiles: dense rows, 16-byte chunks XOR-swizzled inside each row ------------------------
// A tile row of COLS halfs is CPR = COLS/8 chunks of 16 bytes; chunk c of row r is stored at chunk
// position c ^ swz_f<CPR>(r).  The functions are chosen so that both access patterns of the
// kernels hit every LDS bank once: (a) 16 consecutive rows reading the same chunk with 128-bit
// loads, (b) the transposing read, where 32 lanes read 4 consecutive rows x 4 consecutive chunks.
template <int CPR>
__device__ __forceinline__ int swz_f(int row) {
  if constexpr (CPR == 4) {
    return (row >> 2) & 3;
  } else if constexpr (CPR == 8) {
    const int k = (row >> 1) & 7;
    return ((k & 1) << 2) | (k >> 1);
  } else {
    return ((row & 3) << 2) | ((row >> 2) & 3);
  }
}

// Offset in halfs of element (row, col) of a swizzled tile with COLS halfs per row.
template <int COLS>
__device__ __forceinline__ int swz_off(int row, int col) {
  constexpr int CPR = COLS / 8;
  return row * COLS + ((((col >> 3) ^ swz_f<CPR>(row))) << 3) + (col & 7);
}

// One direct global->LDS load of 16 bytes per lane: lane l reads g_base + byte_off(l) and its
// bytes land at lds_base + 16*l; g_base and lds_base must be wave-uniform (they travel in scalar
// registers, so the per-lane address costs no vector arithmetic).  Written as inline assembly so
// that the compiler's wait-count insertion does not serialise later, unrelated LDS reads behind
// it; the caller orders it with wait_async_tiles() and a barrier before the data is read.
// The LDS base travels in M0, bound as an operand in that physical register, so the compiler
// owns M0: it sets it in front of the statement and knows it is live there.  The s_nop covers the
// wait state between a write of M0 and a direct-to-LDS load, which the compiler does not insert
// for an instruction it cannot see.
__device__ __forceinline__ void async_copy16(const half_t* g_base, unsigned byte_off, half_t* lds_base) {
  const unsigned lds_addr = (unsigned)(unsigned long)((DA_LDS char*)lds_base);
  asm volatile("s_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
               :: "v"(byte_off), "s"(g_base), "{m0}"(lds_addr) : "memory");
}

// Asynchronous copy of a [ROWS x COLS] fp16 tile whose rows are `stride` elements apart in global
// memory (each row contiguous) into a swizzled LDS tile with direct global->LDS loads: no
// registers, no LDS store instructions.  One wave-instruction moves a piece of 64 chunks (1 KiB,
// RPP whole rows); the hardware writes lane l's 16 bytes at (wave-uniform LDS base) + 16*l, so the
// swizzle is applied by choosing which global chunk of the piece each lane fetches.  NW waves
// share the tile's instructions round-robin.  Completion: s_waitcnt vmcnt(0), then a barrier.
template <int ROWS, int COLS, int NW>
struct AsyncTile {
  static constexpr int CPR = COLS / 8;
  static constexpr int RPP = 64 / CPR;        // rows per piece
  static constexpr int NINST = ROWS * CPR / 64;
  static constexpr int PER = (NINST + NW - 1) / NW;
  static_assert((ROWS * CPR) % 64 == 0 && 64 % CPR == 0, "tile must be a whole number of 1 KiB pieces of whole rows");
  // The swizzle of a piece depends on the piece index only through a few low bits; when the
  // wave's pieces (wave, wave + NW, ...) agree in those bits, one per-lane offset serves them all.
  static constexpr bool kOneOffset = (CPR == 4) || (CPR == 8 && NW % 2 == 0) || (CPR == 16 && NW % 4 == 0) ||
                                     (CPR == 32 && NW % 8 == 0);
  // byte offset, from the first row of piece `inst`, of the chunk that `lane` fetches
  __device__ static __forceinline__ unsigned lane_off(int inst, int lane, int stride) {
    const int L = inst * 64 + lane;
    const int row = L / CPR, cpos = L % CPR;
    return (unsigned)(((row - inst * RPP) * stride + ((cpos ^ swz_f<CPR>(row)) << 3)) * 2);
  }
  // number of instructions wave `wave` issues for one tile
  __device__ static __forceinline__ int count(int wave) {
    if (NINST % NW == 0) return PER;   // the same for every wave: a compile-time constant
    int n = 0;
#pragma unroll
    for (int k = 0; k < PER; ++k) n += (wave + NW * k < NINST) ? 1 : 0;
    return n;
  }
  // issues this wave's instructions k0 .. k1-1 (of PER) for the tile; `off0` = lane_off(wave, lane, stride)
  template <int K0 = 0, int K1 = PER>
  __device__ static __forceinline__ void issue_at(const half_t* gtile, half_t* lds_tile, int wave, int lane, unsigned off0,
                                                  int stride) {
#pragma unroll
    for (int k = K0; k < K1; ++k) {
      const int inst = wave + NW * k;
      if (NINST % NW == 0 || inst < NINST)
        async_copy16(gtile + (size_t)(inst * RPP) * stride, kOneOffset ? off0 : lane_off(inst, lane, stride),
                     lds_tile + inst * 512);
    }
  }
  template <int K0 = 0, int K1 = PER>
  __device__ static __forceinline__ void issue(const half_t* gtile, half_t* lds_tile, int wave, int lane, int stride = COLS) {
    issue_at<K0, K1>(gtile, lds_tile, wave, lane, lane_off(wave, lane, stride), stride);
  }
  // The same copy for a tile whose global rows end at `last_row` (relative to the tile's first row; it may be
  // negative when the whole tile lies past the end): a row beyond it reads row `last_row` instead, so no
  // address past the tensor's last row is formed and the LDS tile holds finite data everywhere.  Used for the
  // last tiles of a sequence whose length is not a multiple of the tile; costs a few VALU instructions per piece.
  template <int K0 = 0, int K1 = PER>
  __device__ static __forceinline__ void issue_clamped(const half_t* gtile, half_t* lds_tile, int wave, int lane, unsigned off0,
                                                       int stride, int last_row) {
    const int r_l = lane / CPR;                        // the lane's row inside a piece
#pragma unroll
    for (int k = K0; k < K1; ++k) {
      const int inst = wave + NW * k;
      if (NINST % NW == 0 || inst < NINST) {
        const int first = inst * RPP;                                  // first row of the piece
        const int base_row = first < last_row ? first : last_row;     // wave-uniform
        const int room = last_row - base_row;                          // rows the piece may advance: >= 0
        const int back = r_l > room ? r_l - room : 0;                  // rows this lane steps back
        const unsigned off = (kOneOffset ? off0 : lane_off(inst, lane, stride)) - (unsigned)(back * stride * 2);
        async_copy16(gtile + (long long)base_row * stride, off, lds_tile + inst * 512);
      }
    }
  }
};

__device__ __forceinline__ void wait_async_tiles() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

// Waits until at most `newest` (wave-uniform, 0..8) of this wave's vector-memory loads are still in
// flight.  Loads complete in issue order, so this is "everything except the last `newest` issued".
__device__ __forceinline__ void wait_async_tiles_except(int newest) {
  switch (newest) {
    case 0: asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); break;
    case 1: asm volatile("s_waitcnt vmcnt(1)" ::: "memory"); break;
    case 2: asm volatile("s_waitcnt vmcnt(2)" ::: "memory"); break;
    case 3: asm volatile("s_waitcnt vmcnt(3)" ::: "memory"); break;
    case 4: asm volatile("s_waitcnt vmcnt(4)" ::: "memory"); break;
    case 5: asm volatile("s_waitcnt vmcnt(5)" ::: "memory"); break;
    case 6: asm volatile("s_waitcnt vmcnt(6)" ::: "memory"); break;
    case 7: asm volatile("s_waitcnt vmcnt(7)" ::: "memory"); break;
    default: asm volatile("s_waitcnt vmcnt(8)" ::: "memory"); break;
  }
}

// ---- dropout ------------------------------------------------------------------------------------
// Keep/drop decisions come from a counter-based hash, so that forward, both backward kernels and the
// mask dump agree without storing anything: one 32-bit word per 2x2 block of (query, key) pairs,
// keyed on (seed, softmax stream, batch*head unit, query/2, key/2); the pair (q, k) owns byte
// 2*(q&1) + (k&1) of the word and is kept iff that byte >= threshold, threshold = round(256 p).
// The seed and the unit do not meet the counter directly: they are first mixed into two key words
// (once per workgroup and stream), and the counter is hashed under both, one entering by XOR before the
// first multiplication and one by addition after it.  Two seeds, however close, therefore give masks
// that are not index permutations of each other.
using da_abi::DropoutCfg;

struct DropoutKey { unsigned k1, k2; };

__device__ __forceinline__ DropoutKey dropout_key(const DropoutCfg& c, unsigned stream_unit) {
  unsigned a = c.seed_lo ^ 0x9E3779B9u;
  a *= 0x85EBCA6Bu; a ^= a >> 13;
  a += c.seed_hi;
  a *= 0xC2B2AE35u; a ^= a >> 16;
  a += stream_unit;
  a *= 0x27D4EB2Fu; a ^= a >> 15;
  a *= 0x165667B1u; a ^= a >> 13;
  unsigned b = a ^ 0x68E31DA4u;
  b *= 0xB5297A4Du; b ^= b >> 15;
  b += c.seed_hi ^ (stream_unit * 0x9E3779B1u);
  b *= 0x1B56C4E9u; b ^= b >> 16;
  return {a, b};
}

__device__ __forceinline__ unsigned dropout_word(const DropoutKey& key, unsigned half_n, unsigned qh, unsigned kh) {
  unsigned h = (qh * half_n + kh) ^ key.k1;
  h *= 0x9E3779B1u;
  h ^= h >> 15;
  h += key.k2;
  h *= 0xC2B2AE3Du;
  h ^= h >> 13;
  h *= 0x27D4EB2Fu;
  h ^= h >> 16;
  return h;
}
// The word of a 2x2 block serves two lanes: the kernels hold the block's two queries (or its two keys) in lanes
// l and l^1.  Of two neighbouring blocks each lane of the pair hashes one -- the even lane the first, the odd
// lane the second (`mine`) -- and takes the other from its neighbour, which halves the hash work.
// Every lane of the wave must be active.
__device__ __forceinline__ void dropout_words_shared(unsigned mine, bool odd_lane, unsigned& first, unsigned& second) {
  const unsigned other = (unsigned)__builtin_amdgcn_update_dpp(0, (int)mine, 0xB1 /* quad_perm 1,0,3,2 */, 0xF, 0xF, true);
  first = odd_lane ? other : mine;
  second = odd_lane ? mine : other;
}
// keep decision of pair (q, k) from the word of its 2x2 block
__device__ __forceinline__ bool dropout_keep(unsigned word, unsigned q, unsigned k, unsigned threshold) {
  return ((word >> (8 * (2 * (q & 1) + (k & 1)))) & 0xffu) >= threshold;
}

// Workgroup id -> logical tile id such that consecutive logical ids land on the same XCD
// (workgroups are dealt round-robin to the 8 XCDs, each with a private L2).
__device__ __forceinline__ int xcd_remap(int wg, int total) {
  constexpr int kXcd = 8;
  if (total % kXcd != 0) return wg;
  return (wg % kXcd) * (total / kXcd) + wg / kXcd;
}

// Workgroup id -> (batch*head unit, rank of the block inside the unit) for kernels whose blocks
// differ in length (causal mask).  Workgroups are dispatched in id order, so all units' blocks of
// rank 0 come first, then rank 1, ...: with rank 0 the longest loop this is longest-first list
// scheduling over the whole grid, which keeps the CUs evenly loaded to the end.  Unit = id % BH
// also keeps a unit on one XCD whenever BH is a multiple of 8.
struct UnitBlock { int unit, rank; };
__device__ __forceinline__ UnitBlock longest_first(int wg, int n_units) {
  return {wg % n_units, wg / n_units};
}

}  // namespace DA_NS
