// Shared device helpers for the gfx950 FlashAttention-2 kernels.
//
// Everything here is written for CDNA4 wave64 and the v_mfma_f32_32x32x16_{bf16,f16}
// instruction.  Register layouts of that instruction (lane = 32*h + c, h in {0,1}, c in 0..31):
//   A operand (32 x 16):  lane holds A[m = c][k = 8h + j],            j = 0..7
//   B operand (16 x 32):  lane holds B[k = 8h + j][n = c],            j = 0..7
//   C/D       (32 x 32):  lane holds C[m = 8*(i/4) + 4h + i%4][n = c], i = 0..15
// The k index is only a summation label, so any consistent assignment of the 8 values per lane
// works as long as A and B agree.  The kernels exploit this: an accumulator tile re-enters the
// next MFMA as a B operand straight from registers, with
//   element j of lane (c, h)  <->  row 16*t + 8*(j/4) + 4h + j%4   (t = which half of the 32 rows)
// and the matching A operand is fetched from row-major LDS tiles with ds_read_b64_tr_b16, the
// transposing LDS read of gfx950: within each group of 16 lanes, lane i receives elements
// e = 0..3 taken from lane (4e + i/4)'s 64-bit word, position i%4.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "fa2_params.hpp"

namespace fa2 {

typedef short s16x8 __attribute__((ext_vector_type(8)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

template <typename T>
struct Elem;

template <>
struct Elem<__bf16> {
  static __device__ __forceinline__ f32x16 mfma(s16x8 a, s16x8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a),
                                                   __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ s16x8 pack8(f32x8 x) {
    return __builtin_bit_cast(s16x8, __builtin_convertvector(x, bf16x8));
  }
  static __device__ __forceinline__ s16x4 pack4(f32x4 x) {
    return __builtin_bit_cast(s16x4, __builtin_convertvector(x, bf16x4));
  }
  static __device__ __forceinline__ unsigned pack2(float lo, float hi) {
    typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
    typedef float f32x2 __attribute__((ext_vector_type(2)));
    const f32x2 x = {lo, hi};
    return __builtin_bit_cast(unsigned, __builtin_convertvector(x, bf16x2));
  }
  static __device__ __forceinline__ float to_float(short x) {
    return __builtin_bit_cast(float, ((unsigned)(unsigned short)x) << 16);
  }
};

template <>
struct Elem<_Float16> {
  static __device__ __forceinline__ f32x16 mfma(s16x8 a, s16x8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a),
                                                  __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ s16x8 pack8(f32x8 x) {
    return __builtin_bit_cast(s16x8, __builtin_convertvector(x, f16x8));
  }
  static __device__ __forceinline__ s16x4 pack4(f32x4 x) {
    return __builtin_bit_cast(s16x4, __builtin_convertvector(x, f16x4));
  }
  static __device__ __forceinline__ unsigned pack2(float lo, float hi) {
    typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
    typedef float f32x2 __attribute__((ext_vector_type(2)));
    const f32x2 x = {lo, hi};
    return __builtin_bit_cast(unsigned, __builtin_convertvector(x, f16x2));
  }
  static __device__ __forceinline__ float to_float(short x) {
    return (float)__builtin_bit_cast(_Float16, x);
  }
};

// 32-bit pointer into LDS.
typedef const __attribute__((address_space(3))) short *lds_cptr;
__device__ __forceinline__ lds_cptr to_lds(const short *p) {
  return (lds_cptr)(const __attribute__((address_space(3))) void *)p;
}
__device__ __forceinline__ s16x8 lds_read_128(lds_cptr p) {
  return *reinterpret_cast<const __attribute__((address_space(3))) s16x8 *>(p);
}

// Transposing 64-bit LDS read (ds_read_b64_tr_b16).
__device__ __forceinline__ s16x4 lds_read_tr(const short *p) {
  return __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4 *)(p));
}
__device__ __forceinline__ s16x4 lds_read_tr(lds_cptr p) {
  return __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4 *)(p));
}

// A-operand fragment whose k index runs along the ROWS of a row-major LDS tile: two transposing
// reads, rows r0..r0+3 and r0+8..r0+11 as seen by this lane group.  `p` already points at this
// lane's (row, column) for the first read; `ld` is the tile's row pitch in elements.
__device__ __forceinline__ s16x8 lds_read_tr_frag(const short *p, int ld) {
  s16x4 lo = lds_read_tr(p);
  s16x4 hi = lds_read_tr(p + 8 * ld);
  return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
}

// Exchange between lane l and lane l^32 with v_permlane32_swap.  With both operands equal to x
// the instruction returns (x[l], x[l+32]) in lanes < 32 and (x[l-32], x[l]) in lanes >= 32.
// The two results are copied to scalars before any bit cast: __builtin_bit_cast applied directly
// to an element of the returned vector reads element 0 with this compiler.
struct HalfPair {
  float lo, hi;
};
__device__ __forceinline__ HalfPair both_halves(float x) {
  const unsigned u = __builtin_bit_cast(unsigned, x);
  auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  const unsigned a = r[0], b = r[1];
  return HalfPair{__builtin_bit_cast(float, a), __builtin_bit_cast(float, b)};
}
__device__ __forceinline__ float max_over_halves(float x) {
  const HalfPair p = both_halves(x);
  return fmaxf(p.lo, p.hi);
}
__device__ __forceinline__ float sum_over_halves(float x) {
  const HalfPair p = both_halves(x);
  return p.lo + p.hi;
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// Eight half-precision values times a constant, rounded back to half precision.
template <typename T>
__device__ __forceinline__ s16x8 scale8(s16x8 x, float mult) {
  f32x8 f;
#pragma unroll
  for (int j = 0; j < 8; j++) f[j] = Elem<T>::to_float(x[j]) * mult;
  return Elem<T>::pack8(f);
}

// Sixteen copies of one value, kept in sixteen registers: the form an MFMA takes as its C operand.
// The empty asm statement hides from the optimiser that the registers are equal; otherwise it
// rebuilds the block with sixteen moves in front of every use.
__device__ __forceinline__ f32x16 splat16(float x) {
  f32x16 r;
#pragma unroll
  for (int i = 0; i < 16; i++) r[i] = x;
  asm volatile("" : "+v"(r));
  return r;
}

// Load 8 consecutive 16-bit elements row[d0 .. d0+7], zero beyond `headdim` or when the row is
// out of range.  `vec` (uniform) says 16-byte loads are legal: headdim % 8 == 0 and every row
// start is 16-byte aligned.
__device__ __forceinline__ s16x8 load_chunk(const short *row, int d0, int headdim, bool row_ok,
                                            bool vec) {
  s16x8 r = {0, 0, 0, 0, 0, 0, 0, 0};
  if (!row_ok) return r;
  if (vec) {
    if (d0 < headdim) r = *reinterpret_cast<const s16x8 *>(row + d0);
  } else {
#pragma unroll
    for (int j = 0; j < 8; j++)
      if (d0 + j < headdim) r[j] = row[d0 + j];
  }
  return r;
}

__device__ __forceinline__ void store_chunk(short *row, int d0, int headdim, bool row_ok, bool vec,
                                            s16x8 v) {
  if (!row_ok) return;
  if (vec) {
    if (d0 < headdim) *reinterpret_cast<s16x8 *>(row + d0) = v;
  } else {
#pragma unroll
    for (int j = 0; j < 8; j++)
      if (d0 + j < headdim) row[d0 + j] = v[j];
  }
}

// Write a wave's transposed accumulator (DB blocks of 32 headdim rows x 32 sequence columns,
// lane (c, h) holding sequence position c) to a (seqlen, headdim) tensor.  The values go through
// a wave-private LDS patch of 32 x (DP + 8) elements so that global stores are 16-byte and
// row-contiguous.  The caller guarantees the patch is not in use by anyone else.
template <typename T, int DP>
__device__ __forceinline__ void store_transposed_acc(const f32x16 (&acc)[DP / 32], float mult,
                                                     short *patch, short *dst_rows,
                                                     int64_t stride_seq, int rows_valid,
                                                     int headdim, bool vec) {
  constexpr int LD = DP + 8;
  constexpr int CPR = DP / 8;
  const int lane = threadIdx.x & 63;
  const int c = lane & 31, h = lane >> 5;
#pragma unroll
  for (int db = 0; db < DP / 32; db++) {
#pragma unroll
    for (int g = 0; g < 4; g++) {
      f32x4 x = {acc[db][4 * g] * mult, acc[db][4 * g + 1] * mult, acc[db][4 * g + 2] * mult,
                 acc[db][4 * g + 3] * mult};
      *reinterpret_cast<s16x4 *>(patch + c * LD + 32 * db + 8 * g + 4 * h) = Elem<T>::pack4(x);
    }
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
  for (int it = 0; it < (32 * CPR) / 64; it++) {
    int id = lane + 64 * it;
    int r = id / CPR, cc = id % CPR;
    s16x8 v = *reinterpret_cast<const s16x8 *>(patch + r * LD + cc * 8);
    store_chunk(dst_rows + (int64_t)r * stride_seq, cc * 8, headdim, r < rows_valid, vec, v);
  }
}

// Workgroup index -> (batch*head, tile rank); rank 0 is the heaviest tile of a head.
//
// Heads are taken `group` at a time: all tiles of a group of heads, heaviest first, before the next
// group starts.  The tiles of one head re-read the same K/V (or Q/dO) rows, so they should run
// close together in time; with the heads merely round-robin over the whole grid, a problem with
// thousands of (batch, head) pairs would have as many different heads in flight as the chip has
// workgroup slots, nothing would be shared in L2 and every tile would stream its operand from HBM.
// Workgroups go to the 8 XCDs round-robin and `group` is a multiple of 8, so a head also stays on
// one XCD (one L2), `group / 8` heads sharing that L2 at a time.  The group size comes from the
// gfx950 table (per kernel and problem size).
__host__ __device__ __forceinline__ void map_workgroup(int i, int heads, int tiles_per_head, int group, int &bh,
                                              int &rank) {
  const int per_group = group * tiles_per_head;
  const int g = i / per_group;
  const int r = i - g * per_group;
  const int gsize = min(group, heads - g * group);  // the last group may be smaller
  bh = g * group + r % gsize;
  rank = r / gsize;
}

}  // namespace fa2

// ------------------------------------------------------------------------------------------
// Swizzled, unpadded LDS tiles filled by LDS-direct global loads.
//
// A tile of R rows x DP halves is stored with row pitch DP (no padding).  A row holds DP/8
// 16-byte chunks; logical chunk c of row r lives in slot c ^ swz<DP>(r).  The swizzle is chosen
// so that, on the 64-bank LDS of gfx950, both access patterns used by the kernels are free of
// bank conflicts:
//   * 16-byte row reads (ds_read_b128): 16 consecutive rows, same logical chunk;
//   * transposing reads (ds_read_b64_tr_b16): 4 consecutive rows x 4 consecutive chunks.
// global_load_lds_dwordx4 writes lane l's 16 bytes at (wave-uniform LDS base) + 16*l, so one
// wave-load fills 1 KiB of consecutive slots; the swizzle is applied on the global-address side
// (slot s of row r is loaded from chunk s ^ swz(r)).
// ------------------------------------------------------------------------------------------
template <int DP>
__host__ __device__ __forceinline__ int swz(int r);
template <>
__host__ __device__ __forceinline__ int swz<128>(int r) { return 4 * (r & 3) + ((r >> 2) & 3); }
// Rows of 256 halves span the 64 banks twice: the bank of a slot is its low four bits, so the
// 128-column pattern applied to those bits keeps both access patterns conflict-free.
template <>
__host__ __device__ __forceinline__ int swz<256>(int r) { return swz<128>(r); }
template <>
__host__ __device__ __forceinline__ int swz<64>(int r) { return 4 * ((r >> 1) & 1) + ((r >> 2) & 3); }
template <>
__host__ __device__ __forceinline__ int swz<32>(int r) { return (r >> 2) & 3; }

// Element offset of (row r, logical chunk c) in a swizzled tile.
template <int DP>
__host__ __device__ __forceinline__ int swz_off(int r, int c) { return r * DP + ((c ^ swz<DP>(r)) << 3); }

// LDS-direct load of 16 bytes per lane: lane l's data lands at lds_wave_base + 16*l.
// Written as inline assembly on purpose: with the compiler builtin every later LDS read is made
// to wait for the load (the compiler cannot tell which LDS bytes the DMA writes), which would
// serialise the prefetch.  The callers order these loads against LDS reads themselves with
// `s_waitcnt vmcnt(0)` followed by a workgroup barrier.
// LDS destinations are passed around as 32-bit byte addresses (wave-uniform integers): converting
// a generic pointer into an LDS address costs a null check and 64-bit arithmetic per load, an
// integer add does not.  lds_u32(p) does the conversion once.
// M0 is overwritten without being named as a clobber: the gfx9 backend treats M0 as a reserved
// register, sets it immediately before each of its own instructions that read it and never keeps
// a value in it across other code (naming it only draws -Winline-asm "reserved register").
__device__ __forceinline__ unsigned lds_u32(const short *p) {
  return (unsigned)__builtin_amdgcn_readfirstlane(
      (int)(unsigned)(uintptr_t)(__attribute__((address_space(3))) const void *)p);
}
__device__ __forceinline__ void load_lds_16(const short *gsrc, unsigned lds_wave_addr) {
  // State the uniformity the "s" constraint needs (folds away when the value is already scalar).
  lds_wave_addr = (unsigned)__builtin_amdgcn_readfirstlane((int)lds_wave_addr);
  asm volatile(
      "s_mov_b32 m0, %1\n\t"
      "s_nop 0\n\t"
      "global_load_lds_dwordx4 %0, off"
      :
      : "v"(gsrc), "s"(lds_wave_addr)
      : "memory");
}
// Same with the address split into a wave-uniform base (SGPR pair) and a per-lane byte offset.
__device__ __forceinline__ void load_lds_16(const short *uniform_base, unsigned lane_byte_offset,
                                            unsigned lds_wave_addr) {
  // State the uniformity the "s" constraints need (folds away when the value is already scalar).
  const uint64_t raw = (uint64_t)(uintptr_t)uniform_base;
  // (readfirstlane returns a signed int: go through unsigned so the low word is not sign-extended)
  const uint64_t hi = (unsigned)__builtin_amdgcn_readfirstlane((int)(unsigned)(raw >> 32));
  const uint64_t lo = (unsigned)__builtin_amdgcn_readfirstlane((int)(unsigned)raw);
  const uint64_t ubase = (hi << 32) | lo;
  uniform_base = (const short *)(uintptr_t)ubase;
  lds_wave_addr = (unsigned)__builtin_amdgcn_readfirstlane((int)lds_wave_addr);
  asm volatile(
      "s_mov_b32 m0, %2\n\t"
      "s_nop 0\n\t"
      "global_load_lds_dwordx4 %0, %1"
      :
      : "v"(lane_byte_offset), "s"(uniform_base), "s"(lds_wave_addr)
      : "memory");
}

// A 64-bit value that is the same in every lane, moved to scalar registers.  For values whose
// uniformity the compiler loses track of: address arithmetic on them then stays on the scalar unit.
__device__ __forceinline__ uint64_t uniform64(uint64_t x) {
  const uint64_t hi = (unsigned)__builtin_amdgcn_readfirstlane((int)(unsigned)(x >> 32));
  const uint64_t lo = (unsigned)__builtin_amdgcn_readfirstlane((int)(unsigned)x);
  return (hi << 32) | lo;
}
__device__ __forceinline__ const short *uniform_ptr(const short *p) {
  return (const short *)(uintptr_t)uniform64((uint64_t)(uintptr_t)p);
}

// s_waitcnt vmcnt(0) only (gfx9 encoding: expcnt and lgkmcnt fields left at their maxima).
__device__ __forceinline__ void wait_vmem_all() { __builtin_amdgcn_s_waitcnt(0x0F70); }
// s_waitcnt vmcnt(N) only, 0 <= N < 64: wait until at most N vector-memory loads of this wave are
// outstanding (vmcnt is split in the gfx9 encoding: bits 3:0 and 15:14).
template <int N>
__device__ __forceinline__ void wait_vmem() {
  static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit field");
  __builtin_amdgcn_s_waitcnt(0x0F70 | (N & 15) | ((N >> 4) << 14));
}

// Row pitch, in elements, of the LDS tiles of the fast kernels for head dimension DP.  The swizzle
// needs a power-of-two number of 16-byte chunks per row, so 96 columns live in rows of 128: the
// last four chunk slots of a row are never loaded and never read.
constexpr int lds_pitch(int dp) { return dp == 96 ? 128 : dp == 192 ? 256 : dp; }

// Items [part(n, units, u), part(n, units, u + 1)) are unit u's share of n items spread as evenly
// as integers allow over `units` units (equal shares when units divides n).
constexpr int part(int n, int units, int u) { return n * u / units; }

// Workgroup barrier between two tiles of a streaming loop, without the "wait for every
// outstanding LDS operation" the compiler puts in front of a barrier it can see.  The caller has
// already waited for its LDS-direct loads (vmcnt); the LDS reads still in flight at this point
// fetch fragments from a stage that nothing overwrites before the next barrier, so they may
// complete after it.
__device__ __forceinline__ void tile_barrier() { asm volatile("s_barrier" ::: "memory"); }

// Zero `elems` halves of LDS (a multiple of 8 per thread step) with the whole workgroup.  The
// padded kernels do this once before their first tile load: tile loads never touch the slots of
// columns beyond the head dimension, which the MFMAs read as part of their DP-wide fragments.
template <int NTHREADS>
__device__ __forceinline__ void zero_lds(short *smem, int elems) {
  const fa2::s16x8 z = {0, 0, 0, 0, 0, 0, 0, 0};
  for (int i = threadIdx.x * 8; i < elems; i += NTHREADS * 8) *reinterpret_cast<fa2::s16x8 *>(smem + i) = z;
}

// Streams ROWS x DP tiles of a (seqlen, headdim) matrix into swizzled LDS (row pitch lds_pitch(DP))
// with LDS-direct loads.  All NW waves of the workgroup take part; each wave issues LOADS loads of
// 1 KiB of LDS per tile.  A lane owns one 16-byte slot of a row; lanes whose slot holds no data
// (DP < pitch, or with PAD a head dimension of `chunks` 16-byte chunks below DP) are switched off
// for the load.
template <int DP, int ROWS, int NW, bool PAD = false>
struct TileLoader {
  static constexpr int LP = lds_pitch(DP);
  static constexpr int CPR = LP / 8;    // chunk slots per row
  static constexpr int RPL = 64 / CPR;  // rows per wave-load
  static constexpr int NL = ROWS / RPL; // wave-loads per tile
  static constexpr int LOADS = NL / NW; // per wave
  static_assert(NL % NW == 0 && LOADS >= 1, "tile must split evenly over the waves");
  // Multiples of NW*RPL rows keep the low four row bits the swizzle looks at, so a lane's
  // swizzled chunk does not depend on the load index.  Rows of 256 halves (two rows per wave-load,
  // eight rows per round of the four waves) are the exception: row bit 3 alternates with the load
  // index and flips bit 1 of the swizzle, so a lane has one chunk for even loads and one for odd.
  static constexpr bool BY_PARITY = (NW * RPL) % 16 != 0;
  static_assert(!BY_PARITY || (NW * RPL == 8 && LP == 256), "swizzle must be independent of the load index");
  static constexpr int TILE_ELEMS = ROWS * LP;

  const short *base;  // first row of the matrix for this (batch, head)
  int64_t stride;     // row stride in elements
  int wave;
  int row_in;         // this lane's row within the tile for load 0
  int chunk;          // this lane's global chunk index
  unsigned voff;      // byte offset of this lane inside a tile for load 0
  bool active;        // this lane's slot holds data
  int chunk_odd;      // BY_PARITY: the same three for odd load indices
  unsigned voff_odd;
  bool active_odd;

  static constexpr bool ALL_ACTIVE = LP == DP && !PAD;  // every slot of a row holds data

  // Wave-load i of wave `wave` fills LDS bytes [(i * NW + wave) * 1024, + 1024) of the tile, lane l
  // the 16 bytes at 16 * l: slot l % CPR of tile row i * NW * RPL + wave * RPL + l / CPR.  This is the
  // global 16-byte chunk of that row which the slot holds under the swizzle.
  static __host__ __device__ __forceinline__ int chunk_of(int lane, int wave, int i) {
    const int row = i * NW * RPL + wave * RPL + lane / CPR;
    return (lane % CPR) ^ swz<LP>(row);
  }

  __device__ __forceinline__ TileLoader(const short *base_, int64_t stride_, int chunks = DP / 8)
      : base(base_), stride(stride_) {
    const int lane = threadIdx.x & 63;
    wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    row_in = wave * RPL + lane / CPR;
    chunk = (lane % CPR) ^ swz<LP>(row_in);  // == chunk_of(lane, wave, 0)
    active = ALL_ACTIVE || chunk < (PAD ? chunks : DP / 8);
    voff = 2u * (unsigned)(row_in * (int)stride + chunk * 8);
    chunk_odd = BY_PARITY ? chunk ^ 2 : chunk;  // == chunk_of(lane, wave, odd i), see BY_PARITY
    active_odd = ALL_ACTIVE || chunk_odd < (PAD ? chunks : DP / 8);
    voff_odd = 2u * (unsigned)(row_in * (int)stride + chunk_odd * 8);
  }

  // Rows [row0, row0 + ROWS), all inside the matrix -> tile at LDS byte address `lds`.
  __device__ __forceinline__ void issue(int row0, unsigned lds) const {
#pragma unroll
    for (int i = 0; i < LOADS; i++) issue_one(row0, lds, i);
  }

  // Wave-load i (0 <= i < LOADS) of the same tile alone, for callers that spread a tile's loads
  // between other work.
  __device__ __forceinline__ void issue_one(int row0, unsigned lds, int i) const {
    const short *tile = base + (int64_t)row0 * stride;
    const bool odd = BY_PARITY && (i & 1);
    if (ALL_ACTIVE || (odd ? active_odd : active))
      load_lds_16(tile + (int64_t)(i * NW * RPL) * stride, odd ? voff_odd : voff,
                  lds + (unsigned)(i * NW + wave) * 1024u);
  }

  // Same, but rows at or beyond `nrows` are taken from row nrows - 1 (finite values that the
  // caller masks).
  __device__ __forceinline__ void issue_clamped(int row0, int nrows, unsigned lds) const {
#pragma unroll
    for (int i = 0; i < LOADS; i++) {
      const int r = min(row0 + i * NW * RPL + row_in, nrows - 1);
      const bool odd = BY_PARITY && (i & 1);
      if (ALL_ACTIVE || (odd ? active_odd : active))
        load_lds_16(base + (int64_t)r * stride + (odd ? chunk_odd : chunk) * 8,
                    lds + (unsigned)(i * NW + wave) * 1024u);
    }
  }
};
