// FlashAttention-2 forward and backward for gfx950 (CDNA4, wave64, MFMA).
//
// Takes the place of the reference's kernel/fused_mha_kernel.cu (forward
// :20-323, backward :325-735, launchers :891-916) with a different design:
//
//   * Every GEMM runs on v_mfma_f32_32x32x16_f16 with fp32 accumulation.
//   * A wave owns 32 "resident" sequence positions (queries in the forward and
//     in the dQ pass, keys in the dK/dV pass).  Their rows stay in registers as
//     MFMA B operands for the whole kernel.  The other sequence dimension is
//     streamed through LDS in 64-row tiles shared by the waves of a block.
//   * Tiles go global -> LDS with global_load_lds_dwordx4 (no registers in
//     between) into a 3-slot ring, two tiles ahead of their use; one barrier
//     per tile.  The LDS layout is XOR-swizzled so that both the row-wise
//     128-bit reads and the transposing ds_read_b64_tr_b16 reads are free of
//     bank conflicts without padding.
//   * The first GEMM is computed transposed, tile^T[streamed][resident], so a
//     lane holds 16 streamed positions of ONE resident position per 32x32
//     block.  Row statistics (max, sum, logsumexp, delta) are therefore plain
//     per-lane scalars plus one exchange between the two 32-lane halves.
//   * The accumulator registers of the first GEMM, rounded to fp16, are
//     already laid out as the B operand of the second GEMM, so P and dS never
//     travel through LDS.  The matching A operand (V^T, K^T, Q^T, dO^T) is read
//     transposed out of the same row-major tile.
//   * The backward is split into a dQ pass (query-block parallel) and a dK/dV
//     pass (key-block parallel): no atomics, no fp32 dQ scratch, deterministic.
//   * Work-group ids are remapped so that each XCD (private L2) works on whole
//     (batch, head) slices.
//
// Layouts: q/k/v/o/do/dq/dk/dv are (B, N, H, D) fp16, lse/delta are (B, H, N)
// fp32 (reference: kernel/fused_mha_kernel.cu:57-67).

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <math.h>
#include <mutex>
#include <tuple>

#include "fused_mha.h"
#include "block_map.h"


// Backward workspace of fused_mha_backward_noalloc (delta and lse*log2(e), fp32
// (batch, head, n) each): lives in the code object, one copy per GPU, so that
// entry point never allocates.  Host code must not use this name as an address;
// it asks the runtime for the device address once per device (scratch_for_device).
static __device__ __align__(256) unsigned char scratch[2 * (size_t)FUSED_MHA_NOALLOC_MAX_ROWS * sizeof(float)];

namespace {

typedef _Float16 half_t;
typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef _Float16 h4 __attribute__((ext_vector_type(4)));
typedef _Float16 h2 __attribute__((ext_vector_type(2)));
typedef short s4 __attribute__((ext_vector_type(4)));
typedef float f16v __attribute__((ext_vector_type(16)));
typedef float f4v __attribute__((ext_vector_type(4)));

constexpr int kResident = 32;      // resident positions per wave
constexpr int kTile = 64;          // streamed rows per LDS tile
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

template <int D>
struct TileGeom {
  static constexpr int kKSteps = D / 16;                   // MFMA k-steps over D
  static constexpr int kDBlocks = D / 32;                  // 32-row blocks over D
};

__device__ __forceinline__ f16v mfma(h8 a, h8 b, f16v c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// dS for two neighbouring positions: fp16(-p.lo * x0) and fp16(-p.hi * x1), the products in fp32, as
// two mixed-precision FMAs that read the fp16 halves of p directly (the same bits as converting p to
// fp32, multiplying and converting back, in 2 instructions instead of 5).
typedef unsigned u4v __attribute__((ext_vector_type(4)));
__device__ __forceinline__ unsigned neg_mul_to_f16x2(unsigned p_pair, float x0, float x1) {
  unsigned r = 0;
  asm("v_fma_mixlo_f16 %0, %1, -%2, 0 op_sel_hi:[1,0,0]" : "+v"(r) : "v"(p_pair), "v"(x0));
  asm("v_fma_mixhi_f16 %0, %1, -%2, 0 op_sel:[1,0,0] op_sel_hi:[1,0,0]" : "+v"(r) : "v"(p_pair), "v"(x1));
  return r;
}
// y[.] = fp16(-p[.] * x[.]) for the 8 values of one B-operand fragment
__device__ __forceinline__ h8 neg_mul_to_f16x8(h8 p, const float* x) {
  const u4v pp = __builtin_bit_cast(u4v, p);
  u4v r;
#pragma unroll
  for (int j = 0; j < 4; ++j) r[j] = neg_mul_to_f16x2(pp[j], x[2 * j], x[2 * j + 1]);
  return __builtin_bit_cast(h8, r);
}

// Combine a value with the one held by the lane 32 positions away.
__device__ __forceinline__ float other_half(float x) {
  int xi = __float_as_int(x);
  auto r = __builtin_amdgcn_permlane32_swap(xi, xi, false, false);
  // r[0]: lanes 0-31 keep own, lanes 32-63 get lane-32's; r[1] the converse.
  int mine_or_other = (threadIdx.x & 32) ? r[0] : r[1];
  return __int_as_float(mine_or_other);
}

// Streamed-row index of accumulator register r in row-block rb for half hh.
__device__ __forceinline__ int acc_row(int rb, int r, int hh) {
  return rb * 32 + 8 * (r >> 2) + 4 * hh + (r & 3);
}

// Store a [D][32 resident] fp32 accumulator, scaled, as fp16 rows of a dense
// (B, N, H, D) tensor, through a staging tile in LDS that belongs to the wave
// (32 rows of kStagePitch bytes): each lane first writes the 4-feature pieces it
// holds of its own row, then the wave reads the tile back row-wise, so that
// every row leaves as whole 16-byte pieces written by neighbouring lanes (a
// 256-byte row by 16 lanes, as the reference's epilogue does with its 128-bit
// stores, kernel/fused_mha_kernel.cu:318-322, 714-734).  Lane (i, hh) owns row
// row0 + i; per 32-feature block it holds features 8*g + 4*hh + 0..3 for g = 0..3.
// The caller makes sure (with a block barrier) that nobody still reads what the
// staging tile overwrites.
template <int D>
struct StageGeom {
  // bytes per row: a row plus 8, so that the lanes of a half wave, which write 8 bytes each to
  // 32 different rows, spread over the banks; the rows are read back as 8-byte pieces.
  // (Measured: no bank conflicts with D = 64; with D = 128 four conflict cycles per 8-byte
  // store instruction remain whatever the padding or swizzle, 64 cycles per wave and launch.)
  static constexpr int kPitch = D * 2 + 8;
  static constexpr int kBytes = kResident * kPitch;  // per wave
};
template <int D>
__device__ __forceinline__ void store_resident(half_t* __restrict__ base, long row_stride, int row0, int n,
                                               const f16v (&acc)[TileGeom<D>::kDBlocks], float mul, int lane,
                                               char* __restrict__ stage, int my_row = -1,
                                               int upper_off = 16 * StageGeom<D>::kPitch) {
  // my_row: the row (0..31, relative to row0) this lane's column of the accumulator belongs
  // to, when that is not lane & 31; upper_off: where rows 16..31 are staged, relative to `stage`,
  // when the staging tile is not contiguous (see fmha_bwd_dq_spill_kernel for both)
  constexpr int kPitch = StageGeom<D>::kPitch;
  const int i = my_row < 0 ? (lane & 31) : my_row, hh = lane >> 5;
  char* mine = stage + (i & 15) * kPitch + (i >> 4) * upper_off + hh * 8;
#pragma unroll
  for (int db = 0; db < TileGeom<D>::kDBlocks; ++db) {
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      h4 v;
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] = (half_t)(acc[db][4 * g + e] * mul);
      *reinterpret_cast<h4*>(mine + (db * 32 + 8 * g) * 2) = v;
    }
  }
  __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): the wave's own writes have landed
  asm volatile("" ::: "memory");
  constexpr int kLanesPerRow = D / 8, kRowsPerPass = 64 / kLanesPerRow;
  const int r_in = lane / kLanesPerRow, ch = lane % kLanesPerRow;
#pragma unroll
  for (int pass = 0; pass < kResident / kRowsPerPass; ++pass) {
    const int r = pass * kRowsPerPass + r_in;
    const char* src = stage + (r & 15) * kPitch + (r >> 4) * upper_off + ch * 16;
    const h4 lo = *reinterpret_cast<const h4*>(src);
    const h4 hi = *reinterpret_cast<const h4*>(src + 8);
    const h8 v = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    if (row0 + r < n) *reinterpret_cast<h8*>(base + (long)(row0 + r) * row_stride + ch * 8) = v;
  }
}

__device__ __forceinline__ void slice_and_block(int blocks_per_slice, int& slice, int& blk) {
  fmha_slice_and_block(blockIdx.x, gridDim.x / blocks_per_slice, blocks_per_slice, slice, blk);
}

// Blocks of a persistent work group (schedule: block_map.h).
struct PersistentBlocks {
  int total;
  __device__ __forceinline__ int lin(int r) const {  // >= total: this group has no block in round r
    return fmha_persistent_block(r, blockIdx.x, gridDim.x);
  }
  __device__ __forceinline__ int next_round(int r) const {  // the next round with a block for this group, or -1
    return fmha_persistent_next_round(r, blockIdx.x, gridDim.x, total);
  }
};

// ---------------------------------------------------------------------------
// 64-row tiles copied global -> LDS by global_load_lds_dwordx4 (no registers in
// between).  One wave-level instruction moves 1 KiB: 16 rows x 64 bytes, every
// 4 lanes reading one 64-byte row segment.  The tile is an array of such 1 KiB
// blocks, block (R, C) = rows 16R..16R+15, bytes 64C..64C+63 of each row.
// Inside a block the 16-byte chunk c4 of row r16 sits at
//     r16 * 64 + ((c4 ^ (r16 >> 2)) * 16),
// which makes both read patterns below bank-conflict free without padding:
//   rows:  16 lanes read the same chunk of 16 consecutive rows  (128-bit reads)
//   cols:  16 lanes read 4 rows x 32 bytes, transposed         (ds_read_b64_tr_b16)
// ---------------------------------------------------------------------------
template <int D>
struct SwzTile {
  static constexpr int kNC = D / 32;              // 64-byte column groups per row
  static constexpr int kBytes = kTile * D * 2;
  static constexpr int kInstrs = 4 * kNC;         // 1 KiB copies per tile
  __host__ __device__ static constexpr int block_off(int R, int C) { return (R * kNC + C) * 1024; }
};

// Per-lane source of copy instruction t (block R = t / kNC, C = t % kNC):
// byte offset from the tile's first row, and the row inside the tile.
template <int D>
__device__ __forceinline__ void copy_src(int t, int lane, int row_stride, int& row, int& goff) {
  const int R = t / SwzTile<D>::kNC, C = t % SwzTile<D>::kNC;
  const int r16 = lane >> 2, pos = lane & 3;
  const int c4 = pos ^ (r16 >> 2);
  row = 16 * R + r16;
  goff = (row * row_stride + (4 * C + c4) * 8) * 2;  // bytes
}

// One 1 KiB copy: lane l fetches 16 bytes at tile_base + voff and they land in
// LDS at lds_block + 16 * l.  Written as inline asm on purpose: the compiler's
// wait-count insertion then knows nothing of the copy, so it cannot make later
// LDS reads wait for it (it cannot tell the ring slots apart and would wait for
// every copy in flight); the waits for these copies are the explicit wait_vm<>
// calls in the kernels.  tile_base and lds_block must be wave-uniform.
// The LDS address travels in m0, which the compiler reserves for itself and
// does not accept as a clobber: the statement saves and restores it, so a value
// the compiler keeps there (indirect register indexing, its own LDS copies)
// survives.
__device__ __forceinline__ void copy16(const half_t* tile_base, int voff, char* lds_block) {
  const unsigned lds_addr = (unsigned)(uintptr_t)(__attribute__((address_space(3))) char*)lds_block;
  unsigned saved_m0;
  asm volatile(
      "s_mov_b32 %0, m0\n\t"
      "s_mov_b32 m0, %3\n\t"
      "s_nop 0\n\t"
      "global_load_lds_dwordx4 %1, %2\n\t"
      "s_mov_b32 m0, %0"
      : "=&s"(saved_m0)
      : "v"(voff), "s"(tile_base), "s"(lds_addr)
      : "memory");
}
// The same for data that is read once (the non-temporal hint keeps it from displacing
// the tiles other work groups re-read out of the L2).
__device__ __forceinline__ void copy16_stream(const half_t* tile_base, int voff, char* lds_block) {
  const unsigned lds_addr = (unsigned)(uintptr_t)(__attribute__((address_space(3))) char*)lds_block;
  unsigned saved_m0;
  asm volatile(
      "s_mov_b32 %0, m0\n\t"
      "s_mov_b32 m0, %3\n\t"
      "s_nop 0\n\t"
      "global_load_lds_dwordx4 %1, %2 nt\n\t"
      "s_mov_b32 m0, %0"
      : "=&s"(saved_m0)
      : "v"(voff), "s"(tile_base), "s"(lds_addr)
      : "memory");
}

// The same with 4 bytes per lane (256 bytes per instruction): lane l fetches the
// dword at base + voff and it lands in LDS at lds_dst + 4 * l.
__device__ __forceinline__ void copy4(const float* base, int voff, char* lds_dst) {
  const unsigned lds_addr = (unsigned)(uintptr_t)(__attribute__((address_space(3))) char*)lds_dst;
  unsigned saved_m0;
  asm volatile(
      "s_mov_b32 %0, m0\n\t"
      "s_mov_b32 m0, %3\n\t"
      "s_nop 0\n\t"
      "global_load_lds_dword %1, %2\n\t"
      "s_mov_b32 m0, %0"
      : "=&s"(saved_m0)
      : "v"(voff), "s"(base), "s"(lds_addr)
      : "memory");
}

// rows pattern: lane (i, hh) reads chunk 2*kk + hh of row rb*32 + i.
// Two lane offsets (kk even / odd); the rest is an immediate.
template <int D>
__device__ __forceinline__ void swz_rows_off(int lane, int (&off)[2]) {
  const int i = lane & 31, hh = lane >> 5, r16 = i & 15, g = r16 >> 2;
  const int base = (i >> 4) * SwzTile<D>::kNC * 1024 + r16 * 64;
  off[0] = base + ((hh ^ g) * 16);
  off[1] = base + (((2 + hh) ^ g) * 16);
}
template <int D>
__device__ __forceinline__ h8 swz_rows(const char* tile, int rb, int kk, const int (&off)[2]) {
  return *reinterpret_cast<const h8*>(tile + off[kk & 1] + SwzTile<D>::block_off(2 * rb, kk >> 1));
}
// cols pattern: MFMA A operand, rows = features db*32 + (lane & 31), k = streamed
// rows of chunk c16 in accumulator order.  Two lane offsets (rows +0 / +8).
template <int D>
__device__ __forceinline__ void swz_cols_off(int lane, int (&off)[2]) {
  const int L = lane & 15, half = (lane >> 4) & 1, hh = lane >> 5;
  const int c4 = 2 * half + ((L & 3) >> 1);
#pragma unroll
  for (int e = 0; e < 2; ++e) {
    const int r16 = 8 * e + 4 * hh + (L >> 2);
    off[e] = r16 * 64 + ((c4 ^ (r16 >> 2)) * 16) + (L & 1) * 8;
  }
}
template <int D>
__device__ __forceinline__ h8 swz_cols(const char* tile, int c16, int db, const int (&off)[2]) {
  typedef __attribute__((address_space(3))) s4 lds_s4;
  const char* p = tile + SwzTile<D>::block_off(c16, db);
  s4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s4*)(p + off[0]));
  s4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s4*)(p + off[1]));
  return __builtin_bit_cast(h8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
}

// The same reads through LDS addresses formed by the caller (tile + off[e]) and hidden from the optimiser:
// seen whole, it may split tile + off[e] + constant into a loop-invariant part per fragment, kept in a
// register each (and spilled), and the ring slot; opaque, the constant is the instruction's immediate offset.
__device__ __forceinline__ unsigned opaque_lds_address(const char* p) {
  unsigned a = (unsigned)(uintptr_t)(__attribute__((address_space(3))) const char*)p;
  asm volatile("" : "+v"(a));
  return a;
}
template <int D>
__device__ __forceinline__ h8 swz_rows_at(unsigned a_even, unsigned a_odd, int rb, int kk) {
  typedef __attribute__((address_space(3))) h8 lds_h8;
  return *(const lds_h8*)(uintptr_t)(((kk & 1) ? a_odd : a_even) + (unsigned)SwzTile<D>::block_off(2 * rb, kk >> 1));
}
template <int D>
__device__ __forceinline__ h8 swz_cols_at(unsigned a0, unsigned a1, int c16, int db) {
  typedef __attribute__((address_space(3))) s4 lds_s4;
  const unsigned o = SwzTile<D>::block_off(c16, db);
  s4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s4*)(uintptr_t)(a0 + o));
  s4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s4*)(uintptr_t)(a1 + o));
  return __builtin_bit_cast(h8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
}

// s_waitcnt vmcnt(N) with the other counters left alone.  Issued through the
// builtin (not inline asm) so that the compiler's wait-count bookkeeping sees it.
template <int N>
__device__ __forceinline__ void wait_vm() {
  static_assert(N >= 0 && N < 64, "vmcnt immediate");  // bits 3:0 and 15:14 of the immediate
  __builtin_amdgcn_s_waitcnt(0x0F70 | (N & 15) | ((N >> 4) << 14));
}
__device__ __forceinline__ void block_barrier() {
  __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): this wave's LDS reads have landed
  asm volatile("" ::: "memory");       // keep LDS accesses on their side of the barrier
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}
// Wait until at most min(later, kMax) * kPer of this wave's copies are in flight.
template <int kPer, int kMax>
__device__ __forceinline__ void wait_vm_tiles(int later) {
  if constexpr (kMax == 0) {
    wait_vm<0>();
  } else {
    if (later >= kMax) wait_vm<kMax * kPer>();
    else wait_vm_tiles<kPer, kMax - 1>(later);
  }
}
template <int V>
struct IntTag { static constexpr int value = V; };

// 16 bytes per lane to p + kOffset bytes, with the non-temporal hint (data that is read once, by a later
// kernel).  Inline asm because the compiler keeps the hint only on the first of several stores that share
// a base address; like the tile copies it is therefore invisible to the compiler's wait counts.
template <int kOffset>
__device__ __forceinline__ void store16_stream(half_t* p, h8 v, IntTag<kOffset>) {
  asm volatile("global_store_dwordx4 %0, %1, off offset:%2 nt" : : "v"(p), "v"(v), "n"(kOffset) : "memory");
}

// Element strides of a (batch, n, head, d) tensor whose last dimension is
// contiguous.  The dense layout of reference kernel/fused_mha_kernel.cu:57-59 is
// {n*head*d, head*d, d}.
struct Strides {
  long b;
  int n, h;
};

// ---------------------------------------------------------------------------
// Forward.  Block = 8 waves = 256 queries, wave = 32 queries; K/V tiles of 64
// keys stream through a 3-slot LDS ring, copied asynchronously two tiles ahead.
//
// Online softmax as in reference kernel/fused_mha_kernel.cu:159-181, except
// that the running max is only raised (and O, l rescaled) when it grew by more
// than kRescaleLog2 in the exp2 domain, which is rare after the first tiles;
// probabilities then stay below 2^kRescaleLog2 and the final O/l is unchanged.
//
// The two waves that share a SIMD (w and w+4) run the same three steps per
// tile, scores (MFMA), softmax (VALU), accumulate (MFMA), in rotated order:
// waves 0-3 do  accumulate(j-1), scores(j), softmax(j)  in iteration j, waves
// 4-7 do  softmax(j-1), accumulate(j-1), scores(j).  Both need exactly K(j)
// and V(j-1) in iteration j, so one barrier per iteration is enough, and one
// wave's MFMA stretch coincides with the other's VALU stretch.
// ---------------------------------------------------------------------------
constexpr float kRescaleLog2 = 8.f;
constexpr int kFwdWaves = 8;
constexpr int kFwdThreads = kFwdWaves * 64;
constexpr int kFwdBlockQ = kFwdWaves * kResident;
constexpr int kRing = 3;
constexpr int kFwdBlockKernelMaxN = 1024;  // D = 64, causal: longest sequence the one-block kernel takes

// The kernel is persistent: the launch has one work group per CU (fewer for small
// problems) and each walks its own list of blocks (PersistentBlocks).  While a block's
// last tiles are being worked on, the first K and V tiles of the group's next block are
// already copied into the ring slots that come next, and the next block's Q rows are
// loaded during the last iteration (which no longer needs Q); O leaves through staging
// tiles of its own in LDS.  So a block boundary costs one pipeline fill, not a work-group
// launch, a round trip to HBM and an epilogue during which the CU has nothing else to do.
template <int D, bool CAUSAL>
__global__ void __launch_bounds__(kFwdThreads, 1)
fmha_fwd_kernel(const half_t* __restrict__ Q, const half_t* __restrict__ K, const half_t* __restrict__ V,
                Strides qs, Strides ks, Strides vs, half_t* __restrict__ O, float* __restrict__ LSE, int H, int N,
                int nmb, int total, float c, int negate_q) {
  using G = TileGeom<D>;
  using T = SwzTile<D>;
  constexpr int kIPW = T::kInstrs / kFwdWaves;  // copy instructions per wave per tile
  // K ring then V ring, kRing slots each, then per wave a staging tile for 64 features of
  // its 32 output rows.  The copies into the ring are inline asm (see copy16), so slots
  // can be addressed at run time.
  __shared__ __attribute__((aligned(1024))) char smem[2 * kRing * T::kBytes + kFwdWaves * StageGeom<64>::kBytes];
  char* const k_ring = smem;
  char* const v_ring = smem + kRing * T::kBytes;

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int i = lane & 31, hh = lane >> 5;
  char* const stage = smem + 2 * kRing * T::kBytes + wave * StageGeom<64>::kBytes;
  const int rs = H * D;  // O is dense
  const int nt_all = (N + kTile - 1) / kTile;
  const PersistentBlocks pb{total};
  const int slices = total / nmb;

  struct Block {
    const half_t *q, *k, *v;  // first row of the (batch, head) slice
    long o_off, stat_off;     // of the slice in O and in LSE
    int m0, nt;               // first query of the block; tiles it streams
  };
  auto decode = [&](int lin) __attribute__((always_inline)) {
    int bh, mb;
    fmha_slice_and_block(lin, slices, nmb, bh, mb);
    const int mblk = CAUSAL ? nmb - 1 - mb : mb;  // heavy blocks first
    const int b = bh / H, h = bh - b * H;
    Block B;
    B.q = Q + b * qs.b + (long)h * qs.h;
    B.k = K + b * ks.b + (long)h * ks.h;
    B.v = V + b * vs.b + (long)h * vs.h;
    B.o_off = ((long)b * N * H + h) * D;
    B.stat_off = ((long)b * H + h) * N;
    B.m0 = mblk * kFwdBlockQ;
    B.nt = CAUSAL ? min(nt_all, (min(B.m0 + kFwdBlockQ, N) - 1) / kTile + 1) : nt_all;
    return B;
  };

  // this wave's share of every tile copy
  int c_row[kIPW], c_kgoff[kIPW], c_vgoff[kIPW], c_blk[kIPW];
#pragma unroll
  for (int u = 0; u < kIPW; ++u) {
    const int t = wave * kIPW + u;
    copy_src<D>(t, lane, ks.n, c_row[u], c_kgoff[u]);
    copy_src<D>(t, lane, vs.n, c_row[u], c_vgoff[u]);
    c_blk[u] = t * 1024;
  }
  auto copy_tile = [&](const half_t* src, int src_rs, const int (&goff)[kIPW], char* dst, int tile_idx)
                       __attribute__((always_inline)) {
    const int row0 = tile_idx * kTile;
    const half_t* tp = src + (long)row0 * src_rs;  // wave-uniform
    if (row0 + kTile <= N) {
#pragma unroll
      for (int u = 0; u < kIPW; ++u) copy16(tp, goff[u], dst + c_blk[u]);
    } else {
#pragma unroll
      for (int u = 0; u < kIPW; ++u) {  // rows past the end re-read row N-1
        const int back = max(row0 + c_row[u] - (N - 1), 0);
        copy16(tp, goff[u] - back * src_rs * 2, dst + c_blk[u]);
      }
    }
  };

  h8 qf[G::kKSteps];
  auto load_q = [&](const Block& B) __attribute__((always_inline)) {
    const half_t* qp = B.q + (long)min(B.m0 + wave * kResident + i, N - 1) * qs.n + hh * 8;
#pragma unroll
    for (int kk = 0; kk < G::kKSteps; ++kk) qf[kk] = *reinterpret_cast<const h8*>(qp + kk * 16);
  };

  int k_off[2], v_off[2];
  swz_rows_off<D>(lane, k_off);
  swz_cols_off<D>(lane, v_off);

  // state of the block being worked on
  int q0w = 0, qi = 0, ntw = 0;
  f16v o[G::kDBlocks];
  float m_run = -INFINITY, l_run = 0.f;
  f16v s[2];   // scores of the tile in flight
  h8 pf[4];    // its probabilities, fp16, B-operand order

  // The fragment reads of both GEMMs run kLead MFMAs ahead of their use.  The order is written out
  // and pinned with scheduling barriers: left to itself the scheduler, once registers get scarce,
  // puts every read right before its MFMA, which then waits a full LDS round trip each time.
  constexpr int kLead = 4;
  auto scores = [&](const char* Kl, int t) __attribute__((always_inline)) {
    if (t >= ntw) return;
    constexpr int kN = 2 * G::kKSteps;  // MFMA n: key block rb = n & 1, feature step kk = n >> 1
    h8 frag[kLead];
#pragma unroll
    for (int n = 0; n < kLead; ++n) frag[n] = swz_rows<D>(Kl, n & 1, n >> 1, k_off);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int n = 0; n < kN; ++n) {
      const int rb = n & 1, kk = n >> 1;
      if (kk == 0) {
        f16v zero;
#pragma unroll
        for (int r = 0; r < 16; ++r) zero[r] = 0.f;
        s[rb] = mfma(frag[n % kLead], qf[kk], zero);
      } else {
        s[rb] = mfma(frag[n % kLead], qf[kk], s[rb]);
      }
      if (n + kLead < kN) frag[n % kLead] = swz_rows<D>(Kl, (n + kLead) & 1, (n + kLead) >> 1, k_off);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  auto softmax = [&](int t) __attribute__((always_inline)) {
    if (t < 0 || t >= ntw) return;
    const int key0 = t * kTile;
    if ((CAUSAL && key0 + kTile - 1 > q0w) || (key0 + kTile > N)) {
#pragma unroll
      for (int rb = 0; rb < 2; ++rb)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          int key = key0 + acc_row(rb, r, hh);
          if ((CAUSAL && key > qi) || key >= N) s[rb][r] = -INFINITY;
        }
    }
    float mx = s[0][0];
#pragma unroll
    for (int rb = 0; rb < 2; ++rb)
#pragma unroll
      for (int r = 0; r < 16; ++r) mx = fmaxf(mx, s[rb][r]);
    mx = fmaxf(mx, other_half(mx));
    const float m_new = fmaxf(m_run, mx);
    if (__builtin_amdgcn_ballot_w64((m_new - m_run) * c > kRescaleLog2) != 0) {
      const float alpha = fast_exp2((m_run - m_new) * c);
      m_run = m_new;
      l_run *= alpha;
#pragma unroll
      for (int db = 0; db < G::kDBlocks; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) o[db][r] *= alpha;
    }
    // Row sums with plain fp32 adds: the dot-product instructions share the
    // matrix pipeline and stall behind the other wave's MFMAs.
    const float mc = m_run * c;
    float l0 = 0.f, l1 = 0.f;
#pragma unroll
    for (int c16 = 0; c16 < 4; ++c16) {
#pragma unroll
      for (int e = 0; e < 8; e += 2) {
        const float p0 = fast_exp2(fmaf(s[c16 >> 1][(c16 & 1) * 8 + e], c, -mc));
        const float p1 = fast_exp2(fmaf(s[c16 >> 1][(c16 & 1) * 8 + e + 1], c, -mc));
        pf[c16][e] = (half_t)p0;
        pf[c16][e + 1] = (half_t)p1;
        l0 += p0;
        l1 += p1;
      }
    }
    l_run += l0 + l1;
  };
  auto accumulate = [&](const char* Vl, int t) __attribute__((always_inline)) {
    if (t < 0 || t >= ntw) return;
    constexpr int kDB = G::kDBlocks, kN = 4 * kDB;  // MFMA n: key chunk c16 = n / kDB, feature block db = n % kDB
    h8 frag[kLead];
#pragma unroll
    for (int n = 0; n < kLead; ++n) frag[n] = swz_cols<D>(Vl, n / kDB, n % kDB, v_off);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int n = 0; n < kN; ++n) {
      o[n % kDB] = mfma(frag[n % kLead], pf[n / kDB], o[n % kDB]);
      if (n + kLead < kN) frag[n % kLead] = swz_cols<D>(Vl, (n + kLead) / kDB, (n + kLead) % kDB, v_off);
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  const bool first_group = wave < kFwdWaves / 2;
  // Iteration j of a block: K(j) sits in K slot s0, V(j-1) in V slot s2; K(j+2) is copied
  // into K slot s2 and V(j+1) into V slot s1, where tiles past the block's last one are the
  // first tiles of the group's next block (at most K(0), K(1) and V(0) of it).  The slots
  // rotate after every iteration but a block's last, so the next block finds its tile 0 in s0.
  auto run = [&](auto group_tag) __attribute__((always_inline)) {
    constexpr bool kFirst = decltype(group_tag)::value == 0;
    int lin_cur = pb.lin(0), round = 0;
    {
      const Block first = decode(lin_cur);
      copy_tile(first.k, ks.n, c_kgoff, k_ring, 0);
      if (first.nt > 1) copy_tile(first.k, ks.n, c_kgoff, k_ring + T::kBytes, 1);
      copy_tile(first.v, vs.n, c_vgoff, v_ring, 0);
      load_q(first);
    }
    int s0 = 0, s1 = 1, s2 = 2;
    // Copies this wave issued in the previous iteration: all it may leave in flight at the top of
    // an iteration (the tiles needed now were issued earlier).  0 at a block's first iteration:
    // everything issued so far (Q rows, the previous block's output rows) is waited for there, so
    // that no wait for a register load is left to be placed inside the loop, where it would also
    // wait for the copies in flight.
    int in_flight = 0;
    for (;;) {
      // Only what the main loop needs is decoded here; the next block and the output addresses are
      // worked out after it, so that they do not occupy scalar registers across it.
      const half_t *cur_k, *cur_v;
      int nt;
      {
        const Block cur = decode(lin_cur);
        cur_k = cur.k;
        cur_v = cur.v;
        nt = cur.nt;
        q0w = cur.m0 + wave * kResident;
      }
      qi = q0w + i;
      ntw = nt;
      if (CAUSAL) {
        ntw = min(nt, (min(q0w + kResident, N) - 1) / kTile + 1);
        if (q0w >= N) ntw = 0;
      }
#pragma unroll
      for (int db = 0; db < G::kDBlocks; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) o[db][r] = 0.f;
      m_run = -INFINITY;
      l_run = 0.f;
      auto wait_and_sync = [&]() __attribute__((always_inline)) {
        if (in_flight == 2 * kIPW) wait_vm<2 * kIPW>();
        else if (in_flight == kIPW) wait_vm<kIPW>();
        else wait_vm<0>();
        block_barrier();
      };
      auto compute = [&](int j, auto drain_tag) __attribute__((always_inline)) {
        constexpr bool kDrain = decltype(drain_tag)::value != 0;
        const char* Kl = k_ring + s0 * T::kBytes;
        const char* Vl = v_ring + s2 * T::kBytes;
        if (kFirst) {
          accumulate(Vl, j - 1);
          if (!kDrain) { scores(Kl, j); softmax(j); }
        } else {
          softmax(j - 1);
          accumulate(Vl, j - 1);
          if (!kDrain) scores(Kl, j);
        }
        if (!kDrain) { const int t = s0; s0 = s1; s1 = s2; s2 = t; }
      };
      // main part: both tiles to copy belong to this block
      int j = 0;
      for (; j + 2 < nt; ++j) {
        wait_and_sync();
        if (j == 0 && negate_q) {
#pragma unroll
          for (int kk = 0; kk < G::kKSteps; ++kk) qf[kk] = -qf[kk];
        }
        copy_tile(cur_k, ks.n, c_kgoff, k_ring + s2 * T::kBytes, j + 2);
        copy_tile(cur_v, vs.n, c_vgoff, v_ring + s1 * T::kBytes, j + 1);
        in_flight = 2 * kIPW;
        compute(j, IntTag<0>{});
      }
      // tail: the last two tiles, during which the first tiles of the next block are copied
      const int round_next = pb.next_round(round);
      const int lin_next = round_next >= 0 ? pb.lin(round_next) : -1;
      int pre_k = 0, pre_v = 0;  // tiles of the next block already issued
      {
        Block nxt = decode(lin_next >= 0 ? lin_next : lin_cur);
        for (; j < nt; ++j) {
          wait_and_sync();
          if (j == 0 && negate_q) {
#pragma unroll
            for (int kk = 0; kk < G::kKSteps; ++kk) qf[kk] = -qf[kk];
          }
          in_flight = 0;
          const int ek = j + 2, ev = j + 1;
          if (ek < nt) {
            copy_tile(cur_k, ks.n, c_kgoff, k_ring + s2 * T::kBytes, ek);
            in_flight += kIPW;
          } else if (lin_next >= 0 && ek - nt == pre_k && pre_k < min(2, nxt.nt)) {
            copy_tile(nxt.k, ks.n, c_kgoff, k_ring + s2 * T::kBytes, pre_k);
            ++pre_k;
            in_flight += kIPW;
          }
          if (ev < nt) {
            copy_tile(cur_v, vs.n, c_vgoff, v_ring + s1 * T::kBytes, ev);
            in_flight += kIPW;
          } else if (lin_next >= 0 && ev - nt == pre_v && pre_v < 1) {
            copy_tile(nxt.v, vs.n, c_vgoff, v_ring + s1 * T::kBytes, 0);
            ++pre_v;
            in_flight += kIPW;
          }
          compute(j, IntTag<0>{});
        }
        // The last iteration has no tile of its own, only the second half of tile nt - 1.  Q was last used
        // by scores(nt - 1), an iteration ago: the next block's rows are loaded over it.  This is a separate
        // copy of the code so that, in the compiler's eyes, those loads never flow into a use of Q without the
        // wait at the top of the next block between them.
        wait_and_sync();
        in_flight = 0;
        if (lin_next >= 0) load_q(nxt);
        compute(nt, IntTag<1>{});
      }
      // the block's output: O rows through this wave's staging tile, 64 features at a time
      {
        const Block cur = decode(lin_cur);
        const float l_tot = l_run + other_half(l_run);
        const float inv = 1.f / l_tot;
#pragma unroll
        for (int part = 0; part < D / 64; ++part)
          store_resident<64>(O + cur.o_off + part * 64, rs, q0w, N, *reinterpret_cast<const f16v(*)[2]>(&o[2 * part]),
                             inv, lane, stage);
        if (hh == 0 && qi < N) LSE[cur.stat_off + qi] = (m_run * c + __builtin_amdgcn_logf(l_tot)) * kLn2;
      }
      if (lin_next < 0) break;
      lin_cur = lin_next;
      round = round_next;
      {
        // what a short previous block could not prefetch
        const Block cur = decode(lin_cur);
        if (pre_k < 1) copy_tile(cur.k, ks.n, c_kgoff, k_ring + s0 * T::kBytes, 0);
        if (pre_k < 2 && cur.nt > 1) copy_tile(cur.k, ks.n, c_kgoff, k_ring + s1 * T::kBytes, 1);
        if (pre_v < 1) copy_tile(cur.v, vs.n, c_vgoff, v_ring + s0 * T::kBytes, 0);
      }
      in_flight = 0;
    }
  };
  // Each group runs its own copy of the loop: no joins between the two
  // orders inside the loop, so no register shuffling at branch merges.
  if (first_group) run(IntTag<0>{});
  else run(IntTag<1>{});
}

// The forward with one block per work group (no persistence, output staged in the rings once the
// block is done, fragment reads scheduled by hints): with D = 64 it needs few enough registers
// and little enough LDS (48 KiB) for two work groups per CU, which the persistent kernel does not.
// The launcher uses it for D = 64 when that matters more than the persistent kernel's balancing
// and prefetching: without causal masking (all blocks weigh the same) and for short sequences.
template <int D, bool CAUSAL>
__global__ void __launch_bounds__(kFwdThreads, 1)
fmha_fwd_block_kernel(const half_t* __restrict__ Q, const half_t* __restrict__ K, const half_t* __restrict__ V,
                Strides qs, Strides ks, Strides vs, half_t* __restrict__ O, float* __restrict__ LSE, int H, int N,
                int nmb, float c, int negate_q) {
  using G = TileGeom<D>;
  using T = SwzTile<D>;
  constexpr int kIPW = T::kInstrs / kFwdWaves;  // copy instructions per wave per tile
  // K ring then V ring, kRing slots each.  The copies into the ring are inline
  // asm (see copy16), so slots can be addressed at run time.
  __shared__ __attribute__((aligned(1024))) char smem[2 * kRing * T::kBytes];
  char* const k_ring = smem;
  char* const v_ring = smem + kRing * T::kBytes;

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int i = lane & 31, hh = lane >> 5;
  int bh, mb;
  slice_and_block(nmb, bh, mb);
  const int mblk = CAUSAL ? nmb - 1 - mb : mb;  // heavy blocks first
  const int b = bh / H, h = bh - b * H;
  const int rs = H * D;  // O is dense
  const long head_off = ((long)b * N * H + h) * D;
  const half_t* Qb = Q + b * qs.b + (long)h * qs.h;
  const half_t* Kb = K + b * ks.b + (long)h * ks.h;
  const half_t* Vb = V + b * vs.b + (long)h * vs.h;

  const int m0 = mblk * kFwdBlockQ;
  const int q0w = m0 + wave * kResident;
  const int qi = q0w + i;

  // nt: tiles the block streams; ntw: tiles this wave has unmasked keys in.
  int nt = (N + kTile - 1) / kTile;
  int ntw = nt;
  if (CAUSAL) {
    nt = min(nt, (min(m0 + kFwdBlockQ, N) - 1) / kTile + 1);
    ntw = min(nt, (min(q0w + kResident, N) - 1) / kTile + 1);
    if (q0w >= N) ntw = 0;
  }

  // this wave's share of every tile copy
  int c_row[kIPW], c_kgoff[kIPW], c_vgoff[kIPW], c_blk[kIPW];
#pragma unroll
  for (int u = 0; u < kIPW; ++u) {
    const int t = wave * kIPW + u;
    copy_src<D>(t, lane, ks.n, c_row[u], c_kgoff[u]);
    copy_src<D>(t, lane, vs.n, c_row[u], c_vgoff[u]);
    c_blk[u] = t * 1024;
  }
  auto copy_tile = [&](const half_t* src, int src_rs, const int (&goff)[kIPW], char* dst, int tile_idx)
                       __attribute__((always_inline)) {
    const int row0 = tile_idx * kTile;
    const half_t* tp = src + (long)row0 * src_rs;  // wave-uniform
    if (row0 + kTile <= N) {
#pragma unroll
      for (int u = 0; u < kIPW; ++u) copy16(tp, goff[u], dst + c_blk[u]);
    } else {
#pragma unroll
      for (int u = 0; u < kIPW; ++u) {  // rows past the end re-read row N-1
        const int back = max(row0 + c_row[u] - (N - 1), 0);
        copy16(tp, goff[u] - back * src_rs * 2, dst + c_blk[u]);
      }
    }
  };

  copy_tile(Kb, ks.n, c_kgoff, k_ring, 0);
  if (nt > 1) copy_tile(Kb, ks.n, c_kgoff, k_ring + T::kBytes, 1);
  copy_tile(Vb, vs.n, c_vgoff, v_ring, 0);

  h8 qf[G::kKSteps];
  {
    const half_t* qp = Qb + (long)min(qi, N - 1) * qs.n + hh * 8;
#pragma unroll
    for (int kk = 0; kk < G::kKSteps; ++kk) {
      qf[kk] = *reinterpret_cast<const h8*>(qp + kk * 16);
      if (negate_q) qf[kk] = -qf[kk];
    }
  }

  int k_off[2], v_off[2];
  swz_rows_off<D>(lane, k_off);
  swz_cols_off<D>(lane, v_off);

  f16v o[G::kDBlocks];
#pragma unroll
  for (int db = 0; db < G::kDBlocks; ++db)
#pragma unroll
    for (int r = 0; r < 16; ++r) o[db][r] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;
  f16v s[2];   // scores of the tile in flight
  h8 pf[4];    // its probabilities, fp16, B-operand order

  auto scores = [&](const char* Kl, int t) __attribute__((always_inline)) {
    if (t >= ntw) return;
#pragma unroll
    for (int rb = 0; rb < 2; ++rb)
#pragma unroll
      for (int r = 0; r < 16; ++r) s[rb][r] = 0.f;
#pragma unroll
    for (int kk = 0; kk < G::kKSteps; ++kk) {
#pragma unroll
      for (int rb = 0; rb < 2; ++rb) s[rb] = mfma(swz_rows<D>(Kl, rb, kk, k_off), qf[kk], s[rb]);
    }
    // LDS reads run kLead MFMAs ahead of their use.
    constexpr int kN = 2 * G::kKSteps, kLead = 4;
    __builtin_amdgcn_sched_group_barrier(0x100, kLead, 0);
#pragma unroll
    for (int n = 0; n < kN - kLead; ++n) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    }
    __builtin_amdgcn_sched_group_barrier(0x008, kLead, 0);
  };
  auto softmax = [&](int t) __attribute__((always_inline)) {
    if (t < 0 || t >= ntw) return;
    const int key0 = t * kTile;
    if ((CAUSAL && key0 + kTile - 1 > q0w) || (key0 + kTile > N)) {
#pragma unroll
      for (int rb = 0; rb < 2; ++rb)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          int key = key0 + acc_row(rb, r, hh);
          if ((CAUSAL && key > qi) || key >= N) s[rb][r] = -INFINITY;
        }
    }
    float mx = s[0][0];
#pragma unroll
    for (int rb = 0; rb < 2; ++rb)
#pragma unroll
      for (int r = 0; r < 16; ++r) mx = fmaxf(mx, s[rb][r]);
    mx = fmaxf(mx, other_half(mx));
    const float m_new = fmaxf(m_run, mx);
    if (__builtin_amdgcn_ballot_w64((m_new - m_run) * c > kRescaleLog2) != 0) {
      const float alpha = fast_exp2((m_run - m_new) * c);
      m_run = m_new;
      l_run *= alpha;
#pragma unroll
      for (int db = 0; db < G::kDBlocks; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) o[db][r] *= alpha;
    }
    // Row sums with plain fp32 adds: the dot-product instructions share the
    // matrix pipeline and stall behind the other wave's MFMAs.
    const float mc = m_run * c;
    float l0 = 0.f, l1 = 0.f;
#pragma unroll
    for (int c16 = 0; c16 < 4; ++c16) {
#pragma unroll
      for (int e = 0; e < 8; e += 2) {
        const float p0 = fast_exp2(fmaf(s[c16 >> 1][(c16 & 1) * 8 + e], c, -mc));
        const float p1 = fast_exp2(fmaf(s[c16 >> 1][(c16 & 1) * 8 + e + 1], c, -mc));
        pf[c16][e] = (half_t)p0;
        pf[c16][e + 1] = (half_t)p1;
        l0 += p0;
        l1 += p1;
      }
    }
    l_run += l0 + l1;
  };
  auto accumulate = [&](const char* Vl, int t) __attribute__((always_inline)) {
    if (t < 0 || t >= ntw) return;
#pragma unroll
    for (int c16 = 0; c16 < 4; ++c16) {
#pragma unroll
      for (int db = 0; db < G::kDBlocks; ++db) o[db] = mfma(swz_cols<D>(Vl, c16, db, v_off), pf[c16], o[db]);
    }
    // LDS reads (two per MFMA) run kLead MFMAs ahead of their use.
    constexpr int kN = 4 * G::kDBlocks, kLead = 4;
    __builtin_amdgcn_sched_group_barrier(0x100, 2 * kLead, 0);
#pragma unroll
    for (int n = 0; n < kN - kLead; ++n) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
    }
    __builtin_amdgcn_sched_group_barrier(0x008, kLead, 0);
  };

  const bool first_group = wave < kFwdWaves / 2;
  // Everything issued so far (Q rows, first copies) is waited for here, once,
  // so that no wait for a register load is left to be placed inside the loop,
  // where it would also wait for the copies in flight.
  wait_vm<0>();
  // Iteration j: K(j) sits in K slot j % 3, V(j-1) in V slot (j-1) % 3; K(j+2)
  // is copied into K slot (j+2) % 3 and V(j+1) into V slot (j+1) % 3.
  auto run = [&](auto group_tag) __attribute__((always_inline)) {
    constexpr bool kFirst = decltype(group_tag)::value == 0;
    int s0 = 0, s1 = 1, s2 = 2;  // j % 3, (j+1) % 3, (j+2) % 3
    for (int j = 0; j <= nt; ++j) {
      // K(j) and V(j-1) were issued two iterations ago; what the previous
      // iteration issued (K(j+1), V(j)) may still be in flight.
      if (j + 1 < nt) wait_vm<2 * kIPW>();
      else if (j < nt) wait_vm<kIPW>();
      else wait_vm<0>();
      block_barrier();
      if (j + 2 < nt) copy_tile(Kb, ks.n, c_kgoff, k_ring + s2 * T::kBytes, j + 2);
      if (j + 1 < nt) copy_tile(Vb, vs.n, c_vgoff, v_ring + s1 * T::kBytes, j + 1);
      const char* Kl = k_ring + s0 * T::kBytes;
      const char* Vl = v_ring + s2 * T::kBytes;
      if (kFirst) {
        accumulate(Vl, j - 1);
        if (j < nt) { scores(Kl, j); softmax(j); }
      } else {
        softmax(j - 1);
        accumulate(Vl, j - 1);
        if (j < nt) scores(Kl, j);
      }
      const int t = s0; s0 = s1; s1 = s2; s2 = t;
    }
  };
  // Each group runs its own copy of the loop: no joins between the two
  // orders inside the loop, so no register shuffling at branch merges.
  if (first_group) run(IntTag<0>{});
  else run(IntTag<1>{});

  const float l_tot = l_run + other_half(l_run);
  const float inv = 1.f / l_tot;
  static_assert(kFwdWaves * StageGeom<D>::kBytes <= 2 * kRing * T::kBytes, "the output staging tiles fit the rings");
  block_barrier();  // every wave is done with the rings: they become the staging tiles
  store_resident<D>(O + head_off, rs, q0w, N, o, inv, lane, smem + wave * StageGeom<D>::kBytes);
  if (hh == 0 && qi < N) LSE[((long)b * H + h) * N + qi] = (m_run * c + __builtin_amdgcn_logf(l_tot)) * kLn2;
}

// ---------------------------------------------------------------------------
// delta[b][h][n] = sum_d dO * O in fp32.  One 16-byte chunk per thread.
// Takes the place of the two PyTorch ops at reference
// flash_attn_interface.py:43-44 (which work in fp16).  Also writes the
// logsumexp scaled to the exp2 domain, lse2 = lse * log2(e), behind delta in
// the workspace, so the dK/dV pass gets both row statistics with one copy.
// ---------------------------------------------------------------------------
template <int D>
__global__ void __launch_bounds__(256)
fmha_bwd_delta_kernel(const half_t* __restrict__ O, const half_t* __restrict__ dO, Strides gs,
                      const float* __restrict__ LSE, float* __restrict__ delta, float* __restrict__ lse2, int H, int N,
                      long rows) {
  constexpr int kLanesPerRow = D / 8;
  const long t = (long)blockIdx.x * blockDim.x + threadIdx.x;
  const long row = t / kLanesPerRow;  // (b*N + n)*H + h: O is dense, dO has its own strides
  const int c = (int)(t % kLanesPerRow);
  const long bn = row / H;
  const int h = (int)(row % H);
  const long b = bn / N;
  const int n = (int)(bn % N);
  float acc = 0.f;
  if (row < rows) {
    h8 a = *reinterpret_cast<const h8*>(O + row * D + c * 8);
    h8 g = *reinterpret_cast<const h8*>(dO + b * gs.b + (long)n * gs.n + (long)h * gs.h + c * 8);
#pragma unroll
    for (int j = 0; j < 8; ++j) acc = fmaf((float)a[j], (float)g[j], acc);
  }
#pragma unroll
  for (int off = kLanesPerRow / 2; off > 0; off >>= 1) acc += __shfl_xor(acc, off);
  if (row < rows && c == 0) {
    const long at = (b * H + h) * N + n;
    delta[at] = acc;
    lse2[at] = LSE[at] * kLog2e;
  }
}

// ---------------------------------------------------------------------------
// Backward, dQ pass.  Block = 128 queries = 4 pairs of waves; a pair owns 32
// queries and splits the work (two waves per SIMD fit):
//   wave A (waves 0-3), tile j: S^T = K Q^T, P^T = exp(S^T - lse) -> P^T(j) to LDS
//   wave B (waves 4-7), tile j: dS^T(j-1) = P^T(j-1) o T(j-1), dQ^T += K(j-1)^T dS^T(j-1),
//                               then dP^T = V(j) dO^T, T(j) = dP^T - delta (kept in registers,
//                               as -T: the GEMM runs on -dO with accumulators that start at delta)
// (formulas: reference kernel/fused_mha_kernel.cu:598-603, 653-656, 680-683).
// B runs one tile behind A for the part that needs P^T, so one barrier per tile
// is enough and neither wave waits for the other inside a tile.  lse and delta
// belong to the resident query, so they are per-lane scalars.  P^T travels in
// the accumulator layout, lane for lane (double-buffered).  K tiles of 64 keys
// stream through a 4-slot LDS ring (B still needs tile j-1), V tiles through a
// 3-slot ring, both copied two tiles ahead.
// ---------------------------------------------------------------------------
constexpr int kDqPairs = 4;
constexpr int kDqWaves = 2 * kDqPairs;
constexpr int kDqThreads = kDqWaves * 64;
constexpr int kDqBlockQ = kDqPairs * kResident;

// STATS: the kernel also produces the two row statistics of the backward,
// delta = rowsum(dO o O) and lse2 = lse * log2(e), for its own queries, uses
// them and stores them in the workspace for the dK/dV pass (which must then be
// launched after this one); fmha_bwd_delta_kernel is not needed in that case.
// Otherwise delta is read from the workspace.
template <int D, bool CAUSAL, bool STATS>
__global__ void __launch_bounds__(kDqThreads, 1)
fmha_bwd_dq_kernel(const half_t* __restrict__ Q, const half_t* __restrict__ K, const half_t* __restrict__ V,
                   const half_t* __restrict__ O, const half_t* __restrict__ dO, Strides qs, Strides ks, Strides vs,
                   Strides gs, const float* __restrict__ LSE, float* __restrict__ delta, float* __restrict__ lse2,
                   half_t* __restrict__ dQ, int H, int N, int nmb, float c, float scale) {
  using G = TileGeom<D>;
  using T = SwzTile<D>;
  constexpr int kIPW = T::kInstrs / kDqWaves;  // copies per wave per tile, per tensor
  // K ring (4), V ring (3), then two buffers of per pair a 64x32 fp16 block (4 KiB) of P^T
  constexpr int kPBytes = kDqPairs * 4096;
  __shared__ __attribute__((aligned(1024))) char smem[7 * T::kBytes + 2 * kPBytes];
  char* const k_ring = smem;
  char* const v_ring = smem + 4 * T::kBytes;
  char* const p_xchg = smem + 7 * T::kBytes;

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int pair = wave & (kDqPairs - 1);
  const bool role_b = wave >= kDqPairs;
  const int i = lane & 31, hh = lane >> 5;
  int bh, mb;
  slice_and_block(nmb, bh, mb);
  const int mblk = CAUSAL ? nmb - 1 - mb : mb;  // heavy blocks first
  const int b = bh / H, h = bh - b * H;
  const int rs = H * D;  // O and dQ are dense
  const long head_off = ((long)b * N * H + h) * D;
  const half_t* Kb = K + b * ks.b + (long)h * ks.h;
  const half_t* Vb = V + b * vs.b + (long)h * vs.h;

  const int m0 = mblk * kDqBlockQ;
  const int q0w = m0 + pair * kResident;
  const int qi = q0w + i;
  const int qrow = min(qi, N - 1);

  int nt = (N + kTile - 1) / kTile;  // tiles the block streams
  int ntw = nt;                      // tiles this pair takes part in
  if (CAUSAL) {
    nt = min(nt, (min(m0 + kDqBlockQ, N) - 1) / kTile + 1);
    ntw = min(nt, (min(q0w + kResident, N) - 1) / kTile + 1);
    if (q0w >= N) ntw = 0;
  }

  int c_row[kIPW], c_kgoff[kIPW], c_vgoff[kIPW], c_blk[kIPW];
#pragma unroll
  for (int u = 0; u < kIPW; ++u) {
    const int t = wave * kIPW + u;
    copy_src<D>(t, lane, ks.n, c_row[u], c_kgoff[u]);
    copy_src<D>(t, lane, vs.n, c_row[u], c_vgoff[u]);
    c_blk[u] = t * 1024;
  }
  auto copy_tiles = [&](int j) __attribute__((always_inline)) {
    const int row0 = j * kTile;
    const half_t* kp = Kb + (long)row0 * ks.n;  // wave-uniform
    const half_t* vp = Vb + (long)row0 * vs.n;
    char* kdst = k_ring + (j & 3) * T::kBytes;
    char* vdst = v_ring + (j % 3) * T::kBytes;
    if (row0 + kTile <= N) {
#pragma unroll
      for (int u = 0; u < kIPW; ++u) copy16(kp, c_kgoff[u], kdst + c_blk[u]);
#pragma unroll
      for (int u = 0; u < kIPW; ++u) copy16(vp, c_vgoff[u], vdst + c_blk[u]);
    } else {
#pragma unroll
      for (int u = 0; u < kIPW; ++u) {  // rows past the end re-read row N-1
        const int back = max(row0 + c_row[u] - (N - 1), 0);
        copy16(kp, c_kgoff[u] - back * ks.n * 2, kdst + c_blk[u]);
      }
#pragma unroll
      for (int u = 0; u < kIPW; ++u) {
        const int back = max(row0 + c_row[u] - (N - 1), 0);
        copy16(vp, c_vgoff[u] - back * vs.n * 2, vdst + c_blk[u]);
      }
    }
  };

  copy_tiles(0);
  if (nt > 1) copy_tiles(1);

  // resident rows of this wave: Q for role A, dO for role B; and the row statistic it needs
  h8 rf[G::kKSteps];
  const long stat_at = ((long)b * H + h) * N + qrow;
  float stat;
  {
    const half_t* rp = (role_b ? dO + b * gs.b + (long)h * gs.h + (long)qrow * gs.n
                               : Q + b * qs.b + (long)h * qs.h + (long)qrow * qs.n) + hh * 8;
#pragma unroll
    for (int kk = 0; kk < G::kKSteps; ++kk) rf[kk] = *reinterpret_cast<const h8*>(rp + kk * 16);
    if (STATS) {
      if (role_b) {
        // delta of this lane's query.  The lane has every other 8-feature chunk of
        // the row; the partial sums are combined in the order of
        // fmha_bwd_delta_kernel's shuffle tree, so both give the same bits.
        const half_t* op = O + head_off + (long)qrow * rs + hh * 8;
        float part[G::kKSteps];
#pragma unroll
        for (int kk = 0; kk < G::kKSteps; ++kk) {
          const h8 ov = *reinterpret_cast<const h8*>(op + kk * 16);
          part[kk] = 0.f;
#pragma unroll
          for (int e = 0; e < 8; ++e) part[kk] = fmaf((float)ov[e], (float)rf[kk][e], part[kk]);
        }
#pragma unroll
        for (int stride = G::kKSteps / 2; stride > 0; stride >>= 1)
#pragma unroll
          for (int kk = 0; kk < stride; ++kk) part[kk] += part[kk + stride];
        stat = part[0] + other_half(part[0]);
        if (hh == 0 && qi < N) delta[stat_at] = stat;
      } else {
        stat = LSE[stat_at] * kLog2e;
        if (hh == 0 && qi < N) lse2[stat_at] = stat;
      }
    } else {
      stat = role_b ? delta[stat_at] : LSE[stat_at] * kLog2e;
    }
    // Role B works with -dO: its first GEMM then gives delta - dP^T on top of
    // accumulators that start at delta, with no subtraction afterwards.
    if (role_b) {
#pragma unroll
      for (int kk = 0; kk < G::kKSteps; ++kk) rf[kk] = -rf[kk];
    }
  }

  int r_off[2], c_off[2];
  swz_rows_off<D>(lane, r_off);
  swz_cols_off<D>(lane, c_off);
  char* const p_mine = p_xchg + pair * 4096 + lane * 16;  // + buffer * kPBytes + rb * 2048 + half * 1024

  // first GEMM of a tile: rows of K (role A) or V (role B) against the resident
  // rows, on top of the value `init` in every accumulator element
  auto gemm1 = [&](const char* tile_lds, f16v (&x)[2], float init) __attribute__((always_inline)) {
#pragma unroll
    for (int rb = 0; rb < 2; ++rb)
#pragma unroll
      for (int r = 0; r < 16; ++r) x[rb][r] = init;
#pragma unroll
    for (int kk = 0; kk < G::kKSteps; ++kk) {
#pragma unroll
      for (int rb = 0; rb < 2; ++rb) x[rb] = mfma(swz_rows<D>(tile_lds, rb, kk, r_off), rf[kk], x[rb]);
    }
    constexpr int kN = 2 * G::kKSteps, kLead = 4;
    __builtin_amdgcn_sched_group_barrier(0x100, kLead, 0);
#pragma unroll
    for (int n = 0; n < kN - kLead; ++n) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    }
    __builtin_amdgcn_sched_group_barrier(0x008, kLead, 0);
  };
  // P^T = exp2(S^T*c - lse2) -> LDS.  MASKED tiles straddle the diagonal or the
  // end of the sequence.
  auto probabilities = [&](const f16v (&x)[2], char* pw, int key0, auto masked_tag) __attribute__((always_inline)) {
    constexpr bool MASKED = decltype(masked_tag)::value != 0;
#pragma unroll
    for (int rb = 0; rb < 2; ++rb) {
      h8 y0, y1;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        float p = fast_exp2(fmaf(x[rb][r], c, -stat));
        if (MASKED) {
          const int key = key0 + acc_row(rb, r, hh);
          if ((CAUSAL && key > qi) || key >= N) p = 0.f;
        }
        if (r < 8) y0[r] = (half_t)p; else y1[r - 8] = (half_t)p;
      }
      *reinterpret_cast<h8*>(pw + rb * 2048) = y0;
      *reinterpret_cast<h8*>(pw + rb * 2048 + 1024) = y1;
    }
  };
  // Per iteration: wait for tile j (issued two iterations ago; the copies of tile
  // j+1 may still be in flight), one barrier, issue the copies of tile j+2.
  auto step_sync = [&](int j) __attribute__((always_inline)) {
    if (j + 1 < nt) wait_vm<2 * kIPW>();
    else wait_vm<0>();
    block_barrier();
    if (j + 2 < nt) copy_tiles(j + 2);
  };

  wait_vm<0>();  // resident rows, statistics and the first copies
  f16v dq[G::kDBlocks];  // role B's accumulator
  if (!role_b) {
    for (int j = 0; j <= nt; ++j) {
      step_sync(j);
      if (j < ntw) {
        const int key0 = j * kTile;
        const bool masked = (CAUSAL && key0 + kTile - 1 > q0w) || (key0 + kTile > N);
        f16v x[2];
        gemm1(k_ring + (j & 3) * T::kBytes, x, 0.f);
        char* pw = p_mine + (j & 1) * kPBytes;
        if (masked) probabilities(x, pw, key0, IntTag<1>{});
        else probabilities(x, pw, key0, IntTag<0>{});
      }
    }
  } else {
#pragma unroll
    for (int db = 0; db < G::kDBlocks; ++db)
#pragma unroll
      for (int r = 0; r < 16; ++r) dq[db][r] = 0.f;
    f16v x[2];  // delta - dP^T of the previous tile
#pragma unroll
    for (int rb = 0; rb < 2; ++rb)
#pragma unroll
      for (int r = 0; r < 16; ++r) x[rb][r] = 0.f;
    for (int j = 0; j <= nt; ++j) {
      step_sync(j);
      if (j >= 1 && j - 1 < ntw) {  // the part that needs P^T, one tile behind
        const char* Kl = k_ring + ((j - 1) & 3) * T::kBytes;
        const char* pr = p_mine + ((j - 1) & 1) * kPBytes;
        h8 y[4];
#pragma unroll
        for (int rb = 0; rb < 2; ++rb) {
          const h8 p0 = *reinterpret_cast<const h8*>(pr + rb * 2048);
          const h8 p1 = *reinterpret_cast<const h8*>(pr + rb * 2048 + 1024);
          float xr[16];
#pragma unroll
          for (int e = 0; e < 16; ++e) xr[e] = x[rb][e];
          y[rb * 2] = neg_mul_to_f16x8(p0, xr);
          y[rb * 2 + 1] = neg_mul_to_f16x8(p1, xr + 8);
        }
#pragma unroll
        for (int c16 = 0; c16 < 4; ++c16) {
#pragma unroll
          for (int db = 0; db < G::kDBlocks; ++db) dq[db] = mfma(swz_cols<D>(Kl, c16, db, c_off), y[c16], dq[db]);
        }
        constexpr int kN = 4 * G::kDBlocks, kLead = 4;
        __builtin_amdgcn_sched_group_barrier(0x100, 2 * kLead, 0);
#pragma unroll
        for (int n = 0; n < kN - kLead; ++n) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
        }
        __builtin_amdgcn_sched_group_barrier(0x008, kLead, 0);
      }
      if (j < ntw) gemm1(v_ring + (j % 3) * T::kBytes, x, stat);
    }
  }
  static_assert(kDqPairs * StageGeom<D>::kBytes <= 7 * T::kBytes, "the output staging tiles fit the rings");
  block_barrier();  // every wave is done with the rings: they become the staging tiles
  if (role_b) store_resident<D>(dQ + head_off, rs, q0w, N, dq, scale, lane, smem + pair * StageGeom<D>::kBytes);
}

// ---------------------------------------------------------------------------
// Backward, dK/dV pass.  Block = 128 keys = 4 pairs of waves; a pair owns 32
// keys and splits the work so that each wave keeps only one accumulator and one
// of K / V in registers (two waves per SIMD fit):
//   wave A (waves 0-3), tile j:   S = Q K^T, P = exp(S - lse) -> P(j) to LDS,
//                                 dV^T += dO^T P
//   wave B (waves 4-7), tile j:   dS(j-1) = P(j-1) o T(j-1),  dK^T += Q(j-1)^T dS(j-1),
//                                 then dP = dO(j) V^T, T(j) = dP - delta (kept in registers, as -T:
//                                 the GEMM runs on -V with accumulators loaded with delta)
// (formulas: reference kernel/fused_mha_kernel.cu:598-603, 618-629, 653-656,
// 697-712; key-block-parallel launch as at :908-915).  B runs one tile behind A
// for the part that needs P, so one barrier per tile is enough and neither wave
// waits for the other inside a tile.  P travels in the accumulator layout, lane
// for lane (double-buffered).  Q tiles of 64 queries stream through a 4-slot
// LDS ring (B still needs tile j-1), dO tiles and the tile's lse2/delta rows
// through 3-slot rings, all copied two tiles ahead.
// ---------------------------------------------------------------------------
constexpr int kKvPairs = 4;
constexpr int kKvWaves = 2 * kKvPairs;
constexpr int kKvThreads = kKvWaves * 64;
constexpr int kKvBlockKeys = kKvPairs * kResident;

//
// SPILL: wave B also writes every dS tile it forms (fp16, without the scale factor) to
// the workspace `dS`, for fmha_bwd_dq_spill_kernel, which then needs no S and dP of
// its own.  Layout per (batch, head) slice, np = n rounded up to 128:
//   [np / 128 query blocks][np / 64 key tiles] x 16 KiB, the tile a block of 128 queries
//   streams per 64 keys, made of 16 pieces of 1 KiB:
//   [2 halves of 32 keys][2 query tiles of 64][4 chunks of 16 queries] x 1 KiB.
// A 1 KiB piece is what one store instruction of wave B writes: lane l = 32 * hh + i
// (key i, half hh) puts the 16 bytes of registers it holds for the chunk at 16 * l
// (consecutive lanes, consecutive addresses); inside a chunk position 8*hh + e holds
// query 8*(e >> 2) + 4*hh + (e & 3).  Rows of keys at or past n are written as zeros; (key tile, query
// tile) pairs above the diagonal are not written (and not read) under causal masking.
template <int D, bool CAUSAL, bool SPILL>
__global__ void __launch_bounds__(kKvThreads, 1)
fmha_bwd_dkdv_kernel(const half_t* __restrict__ Q, const half_t* __restrict__ K, const half_t* __restrict__ V,
                     const half_t* __restrict__ dO, Strides qs, Strides ks, Strides vs, Strides gs,
                     const float* __restrict__ delta, const float* __restrict__ lse2,
                     half_t* __restrict__ dK, half_t* __restrict__ dV, half_t* __restrict__ dS, int np, int H, int N,
                     int nnb, float c, float scale) {
  using G = TileGeom<D>;
  using T = SwzTile<D>;
  constexpr int kIPW = T::kInstrs / kKvWaves;  // copies per wave per tile, per tensor
  // Q ring (4), dO ring (3), per stats slot 64 lse2 then 64 delta values (1 KiB, half
  // unused), and the P exchange: 2 buffers x per pair two 32x32 fp16 blocks (two 16-byte halves per lane each, in separate 1 KiB planes so that the 16-byte accesses are free of bank conflicts).
  constexpr int kStBytes = 1024;
  constexpr int kPBytes = kKvPairs * 2 * 2048;
  __shared__ __attribute__((aligned(1024))) char smem[7 * T::kBytes + 3 * kStBytes + 2 * kPBytes];
  char* const q_ring = smem;
  char* const g_ring = smem + 4 * T::kBytes;
  char* const st_ring = smem + 7 * T::kBytes;
  char* const p_xchg = st_ring + 3 * kStBytes;

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int pair = wave & (kKvPairs - 1);
  const bool role_b = wave >= kKvPairs;
  const int i = lane & 31, hh = lane >> 5;
  int bh, nblk;
  slice_and_block(nnb, bh, nblk);  // causal: low key blocks are the heavy ones and come first
  const int b = bh / H, h = bh - b * H;
  const int rs = H * D;  // dK and dV are dense
  const long head_off = ((long)b * N * H + h) * D;
  const half_t* Qb = Q + b * qs.b + (long)h * qs.h;
  const half_t* dOb = dO + b * gs.b + (long)h * gs.h;
  const float* delta_b = delta + ((long)b * H + h) * N;
  const float* lse2_b = lse2 + ((long)b * H + h) * N;

  const int n0 = nblk * kKvBlockKeys;
  const int k0w = n0 + pair * kResident;
  const int ki = k0w + i;
  const int krow = min(ki, N - 1);

  const int nt = (N + kTile - 1) / kTile;
  const int t_begin = CAUSAL ? n0 / kTile : 0;
  const int n_it = nt - t_begin;  // >= 1

  // this wave's share of every tile copy
  int c_row[kIPW], c_qgoff[kIPW], c_ggoff[kIPW], c_blk[kIPW];
#pragma unroll
  for (int u = 0; u < kIPW; ++u) {
    const int t = wave * kIPW + u;
    copy_src<D>(t, lane, qs.n, c_row[u], c_qgoff[u]);
    copy_src<D>(t, lane, gs.n, c_row[u], c_ggoff[u]);
    c_blk[u] = t * 1024;
  }
  auto copy_tiles = [&](int it) __attribute__((always_inline)) {  // tile t_begin + it
    const int row0 = (t_begin + it) * kTile;
    const half_t* qp = Qb + (long)row0 * qs.n;   // wave-uniform
    const half_t* gp = dOb + (long)row0 * gs.n;
    char* qdst = q_ring + (it & 3) * T::kBytes;
    char* gdst = g_ring + (it % 3) * T::kBytes;
    if (row0 + kTile <= N) {
#pragma unroll
      for (int u = 0; u < kIPW; ++u) copy16(qp, c_qgoff[u], qdst + c_blk[u]);
#pragma unroll
      for (int u = 0; u < kIPW; ++u) copy16(gp, c_ggoff[u], gdst + c_blk[u]);
    } else {
#pragma unroll
      for (int u = 0; u < kIPW; ++u) {  // rows past the end re-read row N-1
        const int back = max(row0 + c_row[u] - (N - 1), 0);
        copy16(qp, c_qgoff[u] - back * qs.n * 2, qdst + c_blk[u]);
      }
#pragma unroll
      for (int u = 0; u < kIPW; ++u) {
        const int back = max(row0 + c_row[u] - (N - 1), 0);
        copy16(gp, c_ggoff[u] - back * gs.n * 2, gdst + c_blk[u]);
      }
    }
    if (wave == 0) {  // lane l: lse2 and delta of row row0 + l (rows past the end re-read row N-1)
      const int at = min(row0 + lane, N - 1) * 4;
      copy4(lse2_b, at, st_ring + (it % 3) * kStBytes);
      copy4(delta_b, at, st_ring + (it % 3) * kStBytes + 256);
    }
  };

  copy_tiles(0);
  if (n_it > 1) copy_tiles(1);

  // resident rows of this wave: K for role A, V for role B
  h8 rf[G::kKSteps];
  {
    const half_t* rp = (role_b ? V + b * vs.b + (long)h * vs.h + (long)krow * vs.n
                               : K + b * ks.b + (long)h * ks.h + (long)krow * ks.n) + hh * 8;
#pragma unroll
    for (int kk = 0; kk < G::kKSteps; ++kk) {
      rf[kk] = *reinterpret_cast<const h8*>(rp + kk * 16);
      // Role B works with -V: its first GEMM then gives delta - dP on top of
      // accumulators loaded with delta, with no subtraction afterwards.
      if (role_b) rf[kk] = -rf[kk];
    }
  }

  int r_off[2], c_off[2];
  swz_rows_off<D>(lane, r_off);
  swz_cols_off<D>(lane, c_off);
  const int st_off = hh * 16 + (role_b ? 256 : 0);   // + (rb * 32 + 8 * g) * 4: this role's quad
  char* const p_mine = p_xchg + pair * 4096 + lane * 16;  // + buffer * kPBytes + rb * 2048 + half * 1024

  f16v acc[G::kDBlocks];  // dV^T (role A) or dK^T (role B)
#pragma unroll
  for (int db = 0; db < G::kDBlocks; ++db)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[db][r] = 0.f;

  // first GEMM of a tile: rows of Q (role A) or dO (role B) against the resident
  // rows, on top of what x holds
  // Both GEMMs read their LDS fragments kLead MFMAs ahead of their use, in an order that is written out and
  // pinned (see the forward: scheduling hints alone are dropped when registers get scarce).
  constexpr int kLead = 4;
  auto gemm1 = [&](const char* tile_lds, f16v (&x)[2]) __attribute__((always_inline)) {
    const unsigned a0 = opaque_lds_address(tile_lds + r_off[0]), a1 = opaque_lds_address(tile_lds + r_off[1]);
    constexpr int kN = 2 * G::kKSteps;  // MFMA n: row block rb = n & 1, feature step kk = n >> 1
    h8 frag[kLead];
#pragma unroll
    for (int n = 0; n < kLead; ++n) frag[n] = swz_rows_at<D>(a0, a1, n & 1, n >> 1);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int n = 0; n < kN; ++n) {
      x[n & 1] = mfma(frag[n % kLead], rf[n >> 1], x[n & 1]);
      if (n + kLead < kN) frag[n % kLead] = swz_rows_at<D>(a0, a1, (n + kLead) & 1, (n + kLead) >> 1);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  // second GEMM: columns of dO (role A) or Q (role B) against the fp16 operand y
  auto gemm2 = [&](const char* tile_lds, const h8 (&y)[4]) __attribute__((always_inline)) {
    const unsigned a0 = opaque_lds_address(tile_lds + c_off[0]), a1 = opaque_lds_address(tile_lds + c_off[1]);
    constexpr int kDB = G::kDBlocks, kN = 4 * kDB;  // MFMA n: chunk c16 = n / kDB, feature block db = n % kDB
    h8 frag[kLead];
#pragma unroll
    for (int n = 0; n < kLead; ++n) frag[n] = swz_cols_at<D>(a0, a1, n / kDB, n % kDB);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int n = 0; n < kN; ++n) {
      acc[n % kDB] = mfma(frag[n % kLead], y[n / kDB], acc[n % kDB]);
      if (n + kLead < kN) frag[n % kLead] = swz_cols_at<D>(a0, a1, (n + kLead) / kDB, (n + kLead) % kDB);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  // P = exp2(S*c - lse2), fp16, in B-operand order.  MASKED tiles straddle the
  // diagonal or the end of the sequence.
  auto probabilities = [&](const f16v (&x)[2], h8 (&y)[4], const char* Sl, int q0, auto masked_tag)
                           __attribute__((always_inline)) {
    constexpr bool MASKED = decltype(masked_tag)::value != 0;
#pragma unroll
    for (int rb = 0; rb < 2; ++rb)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const f4v l4 = *reinterpret_cast<const f4v*>(Sl + (rb * 32 + 8 * g) * 4);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          float p = fast_exp2(fmaf(x[rb][4 * g + e], c, -l4[e]));
          if (MASKED) {
            const int q = q0 + rb * 32 + 8 * g + 4 * hh + e;
            if ((CAUSAL && ki > q) || q >= N) p = 0.f;
          }
          y[rb * 2 + (g >> 1)][(g & 1) * 4 + e] = (half_t)p;
        }
      }
  };
  auto tile_active = [&](int it) __attribute__((always_inline)) {
    return !CAUSAL || (t_begin + it) * kTile + kTile - 1 >= k0w;
  };

  // Per iteration: wait for tile `it` (issued two iterations ago; the copies of tile
  // it+1 may still be in flight), one barrier, issue the copies of tile it+2.
  auto step_wait = [&](int it) __attribute__((always_inline)) {
    if (it + 1 < n_it) {
      if (wave == 0) wait_vm<2 * kIPW + 2>();
      else wait_vm<2 * kIPW>();
    } else {
      wait_vm<0>();
    }
    block_barrier();
  };
  auto step_sync = [&](int it) __attribute__((always_inline)) {
    step_wait(it);
    if (it + 2 < n_it) copy_tiles(it + 2);
  };
  // where this lane's registers of dS go (SPILL): its key's 32 bytes in chunk 0 of query tile 0 of
  // query block 0; per query tile t: + (t >> 1) * np * 128 + (t & 1) * 2048, per chunk + 512 (elements)
  half_t* const ds_lane = SPILL ? dS + ((long)bh * (np >> 7)) * np * 128 + (long)(k0w >> 6) * 8192 +
                                      ((k0w >> 5) & 1) * 4096 + lane * 8
                                : nullptr;
  wait_vm<0>();  // resident rows and the first copies: nothing is left for the compiler to wait on in the loops
  if (!role_b) {
    for (int it = 0; it <= n_it; ++it) {
      step_sync(it);
      if (it < n_it && tile_active(it)) {
        const char* Ql = q_ring + (it & 3) * T::kBytes;
        const char* Gl = g_ring + (it % 3) * T::kBytes;
        const char* Sl = st_ring + (it % 3) * kStBytes + st_off;
        const int q0 = (t_begin + it) * kTile;
        const bool masked = (CAUSAL && q0 < k0w + kResident - 1) || (q0 + kTile > N);
        f16v x[2];
        h8 y[4];
#pragma unroll
        for (int rb = 0; rb < 2; ++rb)
#pragma unroll
          for (int r = 0; r < 16; ++r) x[rb][r] = 0.f;
        gemm1(Ql, x);
        if (masked) probabilities(x, y, Sl, q0, IntTag<1>{});
        else probabilities(x, y, Sl, q0, IntTag<0>{});
        char* pw = p_mine + (it & 1) * kPBytes;
#pragma unroll
        for (int rb = 0; rb < 2; ++rb) {
          *reinterpret_cast<h8*>(pw + rb * 2048) = y[rb * 2];
          *reinterpret_cast<h8*>(pw + rb * 2048 + 1024) = y[rb * 2 + 1];
        }
        gemm2(Gl, y);
      }
    }
  } else {
    f16v x[2];  // delta - dP of the previous tile
#pragma unroll
    for (int rb = 0; rb < 2; ++rb)
#pragma unroll
      for (int r = 0; r < 16; ++r) x[rb][r] = 0.f;
    for (int it = 0; it <= n_it; ++it) {
      // SPILL: this wave issues its tile copies and, after the second GEMM, the four stores of dS.  The wait
      // at the top of the next iteration leaves at most as many operations in flight as those stores, the
      // newest: every copy issued so far has then landed, whatever order stores and copies complete in.
      if (SPILL) step_wait(it);
      else step_sync(it);
      const bool prev_active = it >= 1 && tile_active(it - 1);
      h8 y[4];
      if (prev_active) {  // the part that needs P, one tile behind
        const char* pr = p_mine + ((it - 1) & 1) * kPBytes;
#pragma unroll
        for (int rb = 0; rb < 2; ++rb) {
          const h8 p0 = *reinterpret_cast<const h8*>(pr + rb * 2048);
          const h8 p1 = *reinterpret_cast<const h8*>(pr + rb * 2048 + 1024);
          float xr[16];
#pragma unroll
          for (int e = 0; e < 16; ++e) xr[e] = x[rb][e];
          y[rb * 2] = neg_mul_to_f16x8(p0, xr);
          y[rb * 2 + 1] = neg_mul_to_f16x8(p1, xr + 8);
        }
        if (SPILL) {
          if (k0w + kResident > N && ki >= N) {  // keys past the end contribute nothing to dQ
#pragma unroll
            for (int c16 = 0; c16 < 4; ++c16)
#pragma unroll
              for (int e = 0; e < 8; ++e) y[c16][e] = (half_t)0.f;
          }
        }
      }
      if (SPILL && it + 2 < n_it) copy_tiles(it + 2);
      if (prev_active) gemm2(q_ring + ((it - 1) & 3) * T::kBytes, y);
      if (SPILL && prev_active) {
        // dS(it - 1) leaves here, between the two GEMMs and away from the tile copies, which all waves issue
        // right after the barrier: the stores go through the same path and would queue behind them.
        const int t = t_begin + it - 1;  // the query tile
        half_t* dst = ds_lane + (long)(t >> 1) * np * 128 + (t & 1) * 2048;
        store16_stream(dst, y[0], IntTag<0>{});
        store16_stream(dst, y[1], IntTag<1024>{});
        store16_stream(dst, y[2], IntTag<2048>{});
        store16_stream(dst, y[3], IntTag<3072>{});
      }
      if (it < n_it && tile_active(it)) {
        const char* Gl = g_ring + (it % 3) * T::kBytes;
        const char* Sl = st_ring + (it % 3) * kStBytes + st_off;
#pragma unroll
        for (int rb = 0; rb < 2; ++rb)
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            const f4v d4 = *reinterpret_cast<const f4v*>(Sl + (rb * 32 + 8 * g) * 4);
#pragma unroll
            for (int e = 0; e < 4; ++e) x[rb][4 * g + e] = d4[e];
          }
        __builtin_amdgcn_sched_barrier(0);  // keep the delta loads out of the GEMM's read/MFMA pipeline
        gemm1(Gl, x);
      }
    }
  }

  static_assert(kKvWaves * StageGeom<D>::kBytes <= 7 * T::kBytes, "the output staging tiles fit the rings");
  block_barrier();  // every wave is done with the rings: they become the staging tiles
  char* const stage = smem + wave * StageGeom<D>::kBytes;
  if (!role_b) store_resident<D>(dV + head_off, rs, k0w, N, acc, 1.f, lane, stage);
  else store_resident<D>(dK + head_off, rs, k0w, N, acc, scale, lane, stage);
}

// ---------------------------------------------------------------------------
// Backward, dQ from spilled dS: dQ = scale * dS K, one GEMM, for callers whose
// workspace holds the dS tiles fmha_bwd_dkdv_kernel<.., SPILL> wrote (layout there).
// A block is P = 1 or 2 of the 128-query panels of the workspace; computing wave
// w of 4 P owns its 32 queries and computes per 64 keys
//     dQ^T[d][q] += K^T[d][key] dS^T[key][q]
// with both operands read transposed out of LDS (the K tile as everywhere else, the
// dS tile as its 1 KiB pieces), so the order of the keys inside a 16-key step is the
// same for both.
// What bounds the kernel is the path that copies tiles into LDS (64 bytes per clock and
// CU at best), then HBM (dS is read once):
//   * with P = 2 a K tile serves 256 queries, so per 32 KiB of dS only 16 KiB of K go through it (P = 1 is
//     for launches with too few blocks to balance otherwise);
//   * four more waves do nothing but copy, two the dS tiles (half of the pieces each) and two the
//     K tiles: issuing a tile's copy instructions holds a wave for about as long as its
//     share of the MFMAs takes; and a wave's copies complete in order, so a wave that
//     issued both kinds would wait for young dS copies whenever it needs an older K tile;
//   * the launch is persistent (PersistentBlocks) and the tiles of a work group's blocks
//     form ONE sequence that runs through the rings without regard to block boundaries;
//     an output block leaves through staging tiles of its own while the copies of the
//     next blocks' tiles are already in flight.  Both rings are filled two tiles ahead: behind the dS copies
//     that a CU has in flight, a K tile takes as long to arrive as they do, L2 hit or not;
//   * the LDS is full with that, so the epilogue stages a wave's output rows in the 4 KiB of the block's last dS
//     tile that hold the wave's own queries and that no other wave reads.
// The queries of a chunk sit in the order the dK/dV pass's registers held them (bits
// 2 and 3 of the position inside 16 swapped); the epilogue puts the rows back in place.
// (formula: reference kernel/fused_mha_kernel.cu:680-683.)
// ---------------------------------------------------------------------------
constexpr int kDsCopyWaves = 4;    // waves that only copy tiles: two for dS, two for K
constexpr int kDsPanelQ = 128;     // queries per panel of the workspace
constexpr int kDsRingS = 3;   // dS tiles
constexpr int kDsRingK = 3;   // K tiles
constexpr int kDsPanelTileBytes = kTile * kDsPanelQ * 2;
constexpr int kDsStageD = 32;          // features staged at a time in the epilogue
constexpr int ds_threads(int panels) { return (4 * panels + kDsCopyWaves) * 64; }

template <int D, bool CAUSAL, int kDsPanels>
__global__ void __launch_bounds__(ds_threads(kDsPanels), 1)
fmha_bwd_dq_spill_kernel(const half_t* __restrict__ K, Strides ks, const half_t* __restrict__ dS, int np,
                         half_t* __restrict__ dQ, int H, int N, int nqb, int total, float scale) {
  using T = SwzTile<D>;             // K tile: 64 keys x D features
  constexpr int kKIPW = T::kInstrs / 2;              // K copies per K-copying wave and tile
  constexpr int kDsWaves = 4 * kDsPanels;            // computing waves
  constexpr int kDsBlockQ = kDsPanels * kDsPanelQ;
  constexpr int kDsTileBytes = kDsPanels * kDsPanelTileBytes;
  constexpr int kSIPW = kDsTileBytes / 1024 / 2;     // dS copies per dS-copying wave and tile: half of the pieces
  constexpr int kDB = D / 32;       // 32-feature blocks
  static_assert(16 * StageGeom<kDsStageD>::kPitch <= 2048, "half a staging tile must fit into two dS pieces");
  __shared__ __attribute__((aligned(1024))) char smem[kDsRingS * kDsTileBytes + kDsRingK * T::kBytes];
  char* const s_ring = smem;
  char* const k_ring = smem + kDsRingS * kDsTileBytes;

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const bool computes = wave < kDsWaves;             // then two waves that copy dS and two that copy K
  const int qb = wave & (kDsWaves - 1);              // computing wave: its 32 queries of the block
  const bool copies_k = wave >= kDsWaves + 2;
  const int cw = wave & 1;                           // copying wave: which half of its tensor's copies
  const int i = lane & 31;
  const int rs = H * D;  // dQ is dense
  const int nt_all = (N + kTile - 1) / kTile;
  const int n_panels = np / kDsPanelQ;
  const int slices = total / nqb;
  const PersistentBlocks pb{total};

  // A position in the work group's sequence of tiles: block (round, number), tile j of its nt.
  struct Cursor {
    int round, lin, j, nt, mblk;
    const half_t* base;  // dS copies: this wave's pieces of the block's tile 0; K copies: the slice's K rows
    long out_off;        // consumer: element offset of the slice in dQ
  };
  auto open = [&](int round, bool for_k) __attribute__((always_inline)) {
    Cursor c;
    c.round = round;
    c.lin = round >= 0 ? pb.lin(round) : 0;
    int bh, mb;
    fmha_slice_and_block(c.lin, slices, nqb, bh, mb);
    c.mblk = CAUSAL ? nqb - 1 - mb : mb;  // heavy blocks first
    const int b = bh / H, h = bh - b * H;
    c.j = 0;
    c.nt = CAUSAL ? min(nt_all, 2 * kDsPanels * (c.mblk + 1)) : nt_all;
    // the pieces of a dS-copying wave: with two panels per block one whole panel (the last block of a sequence
    // may have one panel only: the second wave then re-reads the first), else one half of the panel
    const int panel = kDsPanels == 2 ? min(2 * c.mblk + cw, n_panels - 1) : c.mblk;
    const int first_piece = kDsPanels == 2 ? 0 : cw * kSIPW;
    c.base = for_k ? K + b * ks.b + (long)h * ks.h
                   : dS + (((long)bh * n_panels + panel) * np) * kDsPanelQ + first_piece * 512;
    c.out_off = ((long)b * N * H + h) * D;
    return c;
  };
  auto advance = [&](Cursor& c, bool for_k) __attribute__((always_inline)) {  // to the next tile of the sequence
    if (++c.j == c.nt) {
      const int r = pb.next_round(c.round);
      if (r >= 0) c = open(r, for_k);
      else c.round = -1;  // past the end
    }
  };
  int n_tiles = 0;  // tiles in this work group's sequence
  for (int r = 0; r >= 0; r = pb.next_round(r)) {
    int bh, mb;
    fmha_slice_and_block(pb.lin(r), slices, nqb, bh, mb);
    const int mblk = CAUSAL ? nqb - 1 - mb : mb;
    n_tiles += CAUSAL ? min(nt_all, 2 * kDsPanels * (mblk + 1)) : nt_all;
  }

  // K copies: this wave's half of a tile (as in the other kernels).  dS copies: this wave's kSIPW pieces of
  // 1 KiB, lane l fetching 16 bytes.  In memory a piece is [2 halves][32 keys] x 16 bytes; in LDS it
  // becomes [32 keys][2 halves] x 16 bytes (rows of 16 queries), and the pieces of odd query chunks land rotated
  // by 128 bytes (LDS offset o holds row-major byte (o - 128) mod 1024), which keeps the two halves of a 32-lane
  // transposing read on different banks.
  int c_row[kKIPW], c_kgoff[kKIPW], c_kblk[kKIPW];
#pragma unroll
  for (int u = 0; u < kKIPW; ++u) {
    const int t = cw * kKIPW + u;
    copy_src<D>(t, lane, ks.n, c_row[u], c_kgoff[u]);
    c_kblk[u] = t * 1024;
  }
  int c_sgoff[2];  // even and odd pieces; + piece * 1024
  {
    const int at = (lane - 8) & 63;  // position (key, half) = (at >> 1, at & 1) in LDS of what lane l fetches of an odd piece
    c_sgoff[0] = ((lane & 1) * 32 + (lane >> 1)) * 16;
    c_sgoff[1] = ((at & 1) * 32 + (at >> 1)) * 16;
  }
  auto copy_s = [&](const Cursor& c, int slot) __attribute__((always_inline)) {
    const half_t* sp = c.base + (long)c.j * (kDsPanelTileBytes / 2);  // wave-uniform
    char* dst = s_ring + slot * kDsTileBytes + cw * kSIPW * 1024;
#pragma unroll
    for (int u = 0; u < kSIPW; ++u) copy16_stream(sp, c_sgoff[u & 1] + u * 1024, dst + u * 1024);
  };
  auto copy_k = [&](const Cursor& c, int slot) __attribute__((always_inline)) {
    const int row0 = c.j * kTile;
    const half_t* kp = c.base + (long)row0 * ks.n;  // wave-uniform
    char* dst = k_ring + slot * T::kBytes;
    if (row0 + kTile <= N) {
#pragma unroll
      for (int u = 0; u < kKIPW; ++u) copy16(kp, c_kgoff[u], dst + c_kblk[u]);
    } else {
#pragma unroll
      for (int u = 0; u < kKIPW; ++u) {  // rows past the end re-read row N-1 (their dS rows are zero)
        const int back = max(row0 + c_row[u] - (N - 1), 0);
        copy16(kp, c_kgoff[u] - back * ks.n * 2, dst + c_kblk[u]);
      }
    }
  };

  // LDS offsets of this lane's transposing reads.  K tile: as in the other kernels.  dS tile: key step kc,
  // read e: key row (kc & 1) * 16 + 8 * e + 4 * hhk + (L >> 2) of the piece [panel][(kc >> 1)][query tile][chunk
  // 2 * (qb & 1) + lane bit 4], 8 bytes at (L & 3) * 8 of its 32-byte row, plus the rotation of odd chunks.
  int c_off[2];
  swz_cols_off<D>(lane, c_off);
  // the first of this wave's pieces of a dS tile: two adjacent ones per 32 keys
  const int own_pieces = (qb >> 2) * kDsPanelTileBytes + (((qb >> 1) & 1) * 4 + 2 * (qb & 1)) * 1024;
  int s_off[2][2];
  {
    const int L = lane & 15, odd = (lane >> 4) & 1, hhk = lane >> 5;
#pragma unroll
    for (int kcl = 0; kcl < 2; ++kcl)
#pragma unroll
      for (int e = 0; e < 2; ++e) {
        const int in_piece = (kcl * 16 + 8 * e + 4 * hhk + (L >> 2)) * 32 + (L & 3) * 8;
        s_off[kcl][e] = own_pieces + odd * 1024 + ((in_piece + odd * 128) & 1023);
      }
  }
  auto s_frag = [&](const char* tile, int kc) __attribute__((always_inline)) {
    typedef __attribute__((address_space(3))) s4 lds_s4;
    const char* p = tile + (kc >> 1) * 8192;
    s4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s4*)(p + s_off[kc & 1][0]));
    s4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s4*)(p + s_off[kc & 1][1]));
    return __builtin_bit_cast(h8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
  };

  f16v acc[kDB];
#pragma unroll
  for (int db = 0; db < kDB; ++db)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[db][r] = 0.f;
  // column i of the accumulator is the query at position i of the wave's 32: bits 2 and 3 swapped
  const int my_row = (i & 0x13) | ((i & 8) >> 1) | ((i & 4) << 1);

  constexpr int kAheadS = kDsRingS - 1, kAheadK = kDsRingK - 1;
  // the copying waves run ahead of the sequence: kAhead tiles are issued before the first is used
  Cursor ahead = open(0, copies_k);
  if (!computes) {
    const int n_first = min(copies_k ? kAheadK : kAheadS, n_tiles);
    for (int t = 0; t < n_first; ++t) {
      if (copies_k) copy_k(ahead, t);
      else copy_s(ahead, t);
      advance(ahead, copies_k);
    }
  }
  Cursor cur = open(0, false);
  int slot_s = 0, slot_k = 0;                                    // ring slots of tile t
  int next_s = kAheadS % kDsRingS, next_k = kAheadK % kDsRingK;  // ring slots of the tiles to copy next
  for (int t = 0; t < n_tiles; ++t) {
    // tile t must have landed; the copies of the tiles after it (at most kAhead - 1 of them) may be in flight
    const int later = n_tiles - 1 - t;
    if (!computes) {
      if (copies_k) wait_vm_tiles<kKIPW, kAheadK - 1>(later);
      else wait_vm_tiles<kSIPW, kAheadS - 1>(later);
    }
    block_barrier();  // tile t is visible to all; everybody is done with tile t - 1, whose slots are reused now
    if (!computes && ahead.round >= 0) {
      if (copies_k) copy_k(ahead, next_k);
      else copy_s(ahead, next_s);
      advance(ahead, copies_k);
    }
    const int qt = 2 * kDsPanels * cur.mblk + (qb >> 1);                          // this wave's query tile
    const int jend = qt >= nt_all ? 0 : (CAUSAL ? min(cur.nt, qt + 1) : cur.nt);  // tiles this wave takes part in
    if (computes && cur.j < jend) {
      const char* Kl = k_ring + slot_k * T::kBytes;
      const char* Sl = s_ring + slot_s * kDsTileBytes;
      // MFMA n: key step kc = n / kDB, feature block db = n % kDB; the K fragments are read kLead MFMAs ahead, the
      // four dS fragments up front (order pinned, see the forward)
      constexpr int kN = 4 * kDB, kLead = 4;
      h8 bfrag[4], afrag[kLead];
#pragma unroll
      for (int kc = 0; kc < 4; ++kc) bfrag[kc] = s_frag(Sl, kc);
#pragma unroll
      for (int n = 0; n < kLead; ++n) afrag[n] = swz_cols<D>(Kl, n / kDB, n % kDB, c_off);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int n = 0; n < kN; ++n) {
        acc[n % kDB] = mfma(afrag[n % kLead], bfrag[n / kDB], acc[n % kDB]);
        if (n + kLead < kN) afrag[n % kLead] = swz_cols<D>(Kl, (n + kLead) / kDB, (n + kLead) % kDB, c_off);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    if (computes && cur.j == cur.nt - 1) {
      // the block's last tile: the wave's rows leave, staged where its own part of the tile was (rows 0..15 in
      // the pieces of keys 0..31, rows 16..31 in those of keys 32..63); the slot is not refilled before the
      // barrier of the next tile
      char* stage = s_ring + slot_s * kDsTileBytes + own_pieces;
      half_t* out = dQ + cur.out_off;
      const int row0 = cur.mblk * kDsBlockQ + qb * kResident;
#pragma unroll
      for (int part = 0; part < kDB; ++part) {
        store_resident<kDsStageD>(out + part * kDsStageD, rs, row0, N, *reinterpret_cast<const f16v(*)[1]>(&acc[part]),
                                  scale, lane, stage, my_row, 8192);
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[part][r] = 0.f;
      }
    }
    advance(cur, false);
    slot_s = slot_s + 1 == kDsRingS ? 0 : slot_s + 1;
    slot_k = slot_k + 1 == kDsRingK ? 0 : slot_k + 1;
    next_s = next_s + 1 == kDsRingS ? 0 : next_s + 1;
    next_k = next_k + 1 == kDsRingK ? 0 : next_k + 1;
  }
}

// ---------------------------------------------------------------------------
// Host side: validation and launches.
// ---------------------------------------------------------------------------
// Limits of the 32-bit arithmetic in the kernels and of what a launch can take:
//   - a (batch, head) row of lse / delta is addressed with 32-bit byte offsets (n < 2^29);
//   - the dense row stride head * d and the per-lane byte offsets built from it are 32-bit
//     (head * d < 2^24, the bound the strided entry points put on the sequence stride);
//   - a launch holds fewer than 2^32 threads: the finest non-persistent grids are the 128-row
//     blocks of the backward at 512 threads each (fewer than 2^23 blocks) and the delta pass
//     at one thread per 8 features of a row (batch * head * n * d / 8 < 2^32).
// Checked up front, so that nothing is enqueued for a problem a later pass would refuse.
int check_shape(int batch, int head, int m, int n, int d) {
  if (batch <= 0 || head <= 0 || n <= 0 || m != n) return FUSED_MHA_ERR_BAD_SHAPE;
  if (d != 64 && d != 128) return FUSED_MHA_ERR_BAD_HEAD_DIM;
  if (n >= (1 << 29)) return FUSED_MHA_ERR_TOO_LARGE;
  if ((long)head * d >= (1L << 24)) return FUSED_MHA_ERR_TOO_LARGE;
  const long blocks = (long)((n + 127) / 128) * batch * head;
  if (blocks >= (1L << 23)) return FUSED_MHA_ERR_TOO_LARGE;
  if ((long)batch * head * n * (d / 8) >= (1L << 32)) return FUSED_MHA_ERR_TOO_LARGE;
  return FUSED_MHA_OK;
}

// Launch through the C API: the status returned belongs to this launch alone
// (the <<<>>> form plus hipGetLastError would also report, and clear, an error
// left behind by earlier, unrelated work on the thread).
template <typename... Params, typename... Args>
hipError_t launch(void (*kernel)(Params...), unsigned grid, unsigned block, hipStream_t stream, Args... args) {
  static_assert(sizeof...(Params) == sizeof...(Args), "argument count");
  auto pack = [](Params... p) { return std::tuple<Params...>(p...); };
  std::tuple<Params...> vals = pack(args...);  // converted to the kernel's parameter types
  void* ptrs[sizeof...(Params)];
  int idx = 0;
  std::apply([&](auto&... v) { ((ptrs[idx++] = (void*)&v), ...); }, vals);
  return hipLaunchKernel((const void*)kernel, dim3(grid), dim3(block), ptrs, 0, stream);
}

// Work groups of a persistent launch over `total` blocks: one per CU of the current device,
// rounded down to a multiple of 8 (the XCDs take work-group ids round-robin), or one per block
// when there are no more blocks than that.
unsigned persistent_grid(int total) {
  static std::mutex mu;
  static int cus[64] = {};
  int dev = 0, n = 0;
  if (hipGetDevice(&dev) == hipSuccess && dev >= 0 && dev < 64) {
    std::lock_guard<std::mutex> lock(mu);
    if (!cus[dev]) {
      int v = 0;
      if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && v > 0) cus[dev] = v;
    }
    n = cus[dev];
  }
  if (n < 8) n = 256;  // the query failed: MI355X has 256
  n &= ~7;
  return (unsigned)(total <= n ? total : n);
}

bool misaligned(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) != 0; }

// Strides from the C structure, or the dense layout when the caller gave none.
Strides to_strides(const fused_mha_strides* st, int head, int n, int d) {
  if (!st) return Strides{(long)n * head * d, head * d, d};
  return Strides{(long)st->batch, (int)st->seq, (int)st->head};
}

// Every row must start on a 16-byte boundary (strides in multiples of 8 halves);
// the per-lane byte offsets inside a 64-row tile are 32-bit.
bool bad_strides(const fused_mha_strides* st) {
  if (!st) return false;
  if (st->batch < 0 || st->seq < 0 || st->head < 0) return true;
  if ((st->batch | st->seq | st->head) & 7) return true;
  return st->seq >= (1 << 24) || st->head >= (1LL << 31);
}

template <int D, bool CAUSAL>
int launch_forward(const void* q, const void* k, const void* v, Strides qs, Strides ks, Strides vs, void* o, void* lse,
                   int batch, int head, int n, float scale, hipStream_t stream) {
  const int nmb = (n + kFwdBlockQ - 1) / kFwdBlockQ;
  const int total = nmb * batch * head;
  const unsigned grid = persistent_grid(total);
  // scale == 0 would turn the masked scores (-inf) into NaN when multiplied; a
  // tiny positive factor gives the same uniform softmax and keeps -inf * c = -inf.
  const float c = fmaxf(fabsf(scale) * kLog2e, 1e-30f);
  if constexpr (D == 64) {
    if (!CAUSAL || n <= kFwdBlockKernelMaxN) {  // see fmha_fwd_block_kernel
      const hipError_t rc = launch(fmha_fwd_block_kernel<D, CAUSAL>, (unsigned)total, kFwdThreads, stream,
                                   (const half_t*)q, (const half_t*)k, (const half_t*)v, qs, ks, vs, (half_t*)o,
                                   (float*)lse, head, n, nmb, c, scale < 0.f ? 1 : 0);
      return rc == hipSuccess ? FUSED_MHA_OK : FUSED_MHA_ERR_LAUNCH;
    }
  }
  const hipError_t rc = launch(fmha_fwd_kernel<D, CAUSAL>, grid, kFwdThreads, stream, (const half_t*)q,
                               (const half_t*)k, (const half_t*)v, qs, ks, vs, (half_t*)o, (float*)lse, head, n, nmb, total, c,
                               scale < 0.f ? 1 : 0);
  return rc == hipSuccess ? FUSED_MHA_OK : FUSED_MHA_ERR_LAUNCH;
}

int dispatch_forward(const void* q, const fused_mha_strides* q_st, const void* k, const fused_mha_strides* k_st,
                     const void* v, const fused_mha_strides* v_st, void* o, void* lse, int batch, int head, int m,
                     int n, int d, float scale, int causal, void* stream) {
  if (!q || !k || !v || !o || !lse) return FUSED_MHA_ERR_NULL_POINTER;
  if (int rc = check_shape(batch, head, m, n, d)) return rc;
  if (!isfinite(scale)) return FUSED_MHA_ERR_BAD_SCALE;
  if (misaligned(q) || misaligned(k) || misaligned(v) || misaligned(o) || misaligned(lse))
    return FUSED_MHA_ERR_MISALIGNED;
  if (bad_strides(q_st) || bad_strides(k_st) || bad_strides(v_st)) return FUSED_MHA_ERR_BAD_STRIDE;
  hipStream_t s = (hipStream_t)stream;
  const Strides qs = to_strides(q_st, head, n, d), ks = to_strides(k_st, head, n, d), vs = to_strides(v_st, head, n, d);
#define FMHA_FWD(DD, CC) launch_forward<DD, CC>(q, k, v, qs, ks, vs, o, lse, batch, head, n, scale, s)
  if (d == 128) return causal ? FMHA_FWD(128, true) : FMHA_FWD(128, false);
  return causal ? FMHA_FWD(64, true) : FMHA_FWD(64, false);
#undef FMHA_FWD
}

enum BwdPass { kPassDelta = 1, kPassDq = 2, kPassDkDv = 4, kPassAll = 7 };

// Workspace of the backward: delta and lse * log2(e), fp32 (batch, head, n) each; then, for
// the spill path, at the next multiple of 256 bytes, the fp16 dS tiles
// (batch * head slices of np * np elements, np = n rounded up to 128).
size_t stats_bytes(int batch, int head, int n) { return 2 * (size_t)batch * head * n * sizeof(float); }
size_t spill_offset(int batch, int head, int n) { return (stats_bytes(batch, head, n) + 255) & ~(size_t)255; }
int padded_n(int n) { return (n + 127) & ~127; }
size_t spill_bytes(int batch, int head, int n) {
  const size_t np = (size_t)padded_n(n);
  return (size_t)batch * head * np * np * sizeof(half_t);
}

template <int D, bool CAUSAL>
int launch_backward(int passes, bool spill, const void* q, const void* k, const void* v, const void* o,
                    const void* d_o, Strides qs, Strides ks, Strides vs, Strides gs, const void* lse, float* delta,
                    void* dq, void* dk, void* dv, int batch, int head, int n, float scale, hipStream_t stream) {
  // Without the spill and with all three passes asked for, the dQ pass produces delta and lse2 itself.
  const bool dq_makes_stats = !spill && (passes & kPassAll) == kPassAll;
  float* lse2 = delta + (long)batch * head * n;
  half_t* ds = spill ? (half_t*)((char*)delta + spill_offset(batch, head, n)) : nullptr;
  const int np = padded_n(n);
  if ((passes & kPassDelta) && !dq_makes_stats) {
    const long rows = (long)batch * n * head;
    const long threads = rows * (D / 8);
    if (launch(fmha_bwd_delta_kernel<D>, (unsigned)((threads + 255) / 256), 256, stream, (const half_t*)o,
               (const half_t*)d_o, gs, (const float*)lse, delta, lse2, head, n, rows) != hipSuccess)
      return FUSED_MHA_ERR_LAUNCH;
  }
  const float c = scale * kLog2e;
  auto dq_pass = [&]() {
    if (spill) {
      // two panels per block when that leaves every work group at least two blocks (a heavy and a light one)
      const int nqb2 = (n + 2 * kDsPanelQ - 1) / (2 * kDsPanelQ), total2 = nqb2 * batch * head;
      if (total2 >= 2 * persistent_grid(total2))
        return launch(fmha_bwd_dq_spill_kernel<D, CAUSAL, 2>, persistent_grid(total2), ds_threads(2), stream,
                      (const half_t*)k, ks, (const half_t*)ds, np, (half_t*)dq, head, n, nqb2, total2, scale);
      const int nqb = np / kDsPanelQ, total = nqb * batch * head;
      return launch(fmha_bwd_dq_spill_kernel<D, CAUSAL, 1>, persistent_grid(total), ds_threads(1), stream,
                    (const half_t*)k, ks, (const half_t*)ds, np, (half_t*)dq, head, n, nqb, total, scale);
    }
    const int nmb = (n + kDqBlockQ - 1) / kDqBlockQ;
    auto kernel = dq_makes_stats ? fmha_bwd_dq_kernel<D, CAUSAL, true> : fmha_bwd_dq_kernel<D, CAUSAL, false>;
    return launch(kernel, (unsigned)nmb * batch * head, kDqThreads, stream, (const half_t*)q, (const half_t*)k,
                  (const half_t*)v, (const half_t*)o, (const half_t*)d_o, qs, ks, vs, gs, (const float*)lse, delta, lse2,
                  (half_t*)dq, head, n, nmb, c, scale);
  };
  auto dkdv_pass = [&]() {
    const int nnb = (n + kKvBlockKeys - 1) / kKvBlockKeys;
    auto kernel = spill ? fmha_bwd_dkdv_kernel<D, CAUSAL, true> : fmha_bwd_dkdv_kernel<D, CAUSAL, false>;
    return launch(kernel, (unsigned)nnb * batch * head, kKvThreads, stream, (const half_t*)q, (const half_t*)k,
                  (const half_t*)v, (const half_t*)d_o, qs, ks, vs, gs, (const float*)delta, (const float*)lse2,
                  (half_t*)dk, (half_t*)dv, ds, np, head, n, nnb, c, scale);
  };
  // The spilling dK/dV pass feeds the dQ pass; otherwise the dQ pass (which may make the statistics) goes first.
  if (spill) {
    if ((passes & kPassDkDv) && dkdv_pass() != hipSuccess) return FUSED_MHA_ERR_LAUNCH;
    if ((passes & kPassDq) && dq_pass() != hipSuccess) return FUSED_MHA_ERR_LAUNCH;
  } else {
    if ((passes & kPassDq) && dq_pass() != hipSuccess) return FUSED_MHA_ERR_LAUNCH;
    if ((passes & kPassDkDv) && dkdv_pass() != hipSuccess) return FUSED_MHA_ERR_LAUNCH;
  }
  return FUSED_MHA_OK;
}

int dispatch_backward(int passes, const void* q, const fused_mha_strides* q_st, const void* k,
                      const fused_mha_strides* k_st, const void* v, const fused_mha_strides* v_st, const void* o,
                      const void* d_o, const fused_mha_strides* g_st, const void* lse, void* workspace,
                      size_t workspace_bytes, void* dq, void* dk, void* dv, int batch, int head, int m, int n, int d,
                      float scale, int causal, void* stream) {
  const bool need_o = passes & kPassDelta, need_dq = passes & kPassDq, need_dkdv = passes & kPassDkDv;
  if (!d_o || !workspace || !lse || (need_o && !o) || ((need_dq || need_dkdv) && (!q || !k || !v)) ||
      (need_dq && !dq) || (need_dkdv && (!dk || !dv)))
    return FUSED_MHA_ERR_NULL_POINTER;
  if (int rc = check_shape(batch, head, m, n, d)) return rc;
  if (!isfinite(scale)) return FUSED_MHA_ERR_BAD_SCALE;
  if (workspace_bytes < stats_bytes(batch, head, n)) return FUSED_MHA_ERR_BAD_SHAPE;
  // A workspace with room for the dS tiles selects the spill path (5 GEMMs executed instead of 7).
  const bool spill = spill_bytes(batch, head, n) <= FUSED_MHA_SPILL_MAX_BYTES &&
                     workspace_bytes >= spill_offset(batch, head, n) + spill_bytes(batch, head, n);
  if (misaligned(q) || misaligned(k) || misaligned(v) || misaligned(o) || misaligned(d_o) || misaligned(lse) ||
      misaligned(workspace) || misaligned(dq) || misaligned(dk) || misaligned(dv))
    return FUSED_MHA_ERR_MISALIGNED;
  if (bad_strides(q_st) || bad_strides(k_st) || bad_strides(v_st) || bad_strides(g_st)) return FUSED_MHA_ERR_BAD_STRIDE;
  hipStream_t s = (hipStream_t)stream;
  float* delta = (float*)workspace;
  const Strides qs = to_strides(q_st, head, n, d), ks = to_strides(k_st, head, n, d),
                vs = to_strides(v_st, head, n, d), gs = to_strides(g_st, head, n, d);
#define FMHA_BWD(DD, CC) \
  launch_backward<DD, CC>(passes, spill, q, k, v, o, d_o, qs, ks, vs, gs, lse, delta, dq, dk, dv, batch, head, n, \
                          scale, s)
  if (d == 128) return causal ? FMHA_BWD(128, true) : FMHA_BWD(128, false);
  return causal ? FMHA_BWD(64, true) : FMHA_BWD(64, false);
#undef FMHA_BWD
}

// Device address of `scratch` on the current device, looked up on the first call
// per device (each GPU holds its own copy of the array at its own address).
constexpr int kMaxDevices = 64;
int scratch_for_device(void** out) {
  static std::mutex mu;
  static void* ptrs[kMaxDevices] = {};
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return FUSED_MHA_ERR_RUNTIME;
  std::lock_guard<std::mutex> lock(mu);
  if (!ptrs[dev]) {
    void* p = nullptr;
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) return FUSED_MHA_ERR_RUNTIME;
    ptrs[dev] = p;
  }
  *out = ptrs[dev];
  return FUSED_MHA_OK;
}

}  // namespace

extern "C" {

int fused_mha_forward(const void* query_ptr, const void* key_ptr, const void* value_ptr, void* output_ptr,
                      void* lse_ptr, int batch, int head, int m, int n, int d, float scale, int causal,
                      void* stream) {
  return dispatch_forward(query_ptr, nullptr, key_ptr, nullptr, value_ptr, nullptr, output_ptr, lse_ptr, batch, head,
                          m, n, d, scale, causal, stream);
}

int fused_mha_forward_strided(const void* query_ptr, const fused_mha_strides* query_strides, const void* key_ptr,
                              const fused_mha_strides* key_strides, const void* value_ptr,
                              const fused_mha_strides* value_strides, void* output_ptr, void* lse_ptr, int batch,
                              int head, int n, int d, float scale, int causal, void* stream) {
  return dispatch_forward(query_ptr, query_strides, key_ptr, key_strides, value_ptr, value_strides, output_ptr,
                          lse_ptr, batch, head, n, n, d, scale, causal, stream);
}

size_t fused_mha_backward_min_workspace_bytes(int batch, int head, int n, int d) {
  if (check_shape(batch, head, n, n, d) != FUSED_MHA_OK) return 0;
  return stats_bytes(batch, head, n);
}

size_t fused_mha_backward_workspace_bytes(int batch, int head, int n, int d) {
  if (check_shape(batch, head, n, n, d) != FUSED_MHA_OK) return 0;
  if (spill_bytes(batch, head, n) > FUSED_MHA_SPILL_MAX_BYTES) return stats_bytes(batch, head, n);
  return spill_offset(batch, head, n) + spill_bytes(batch, head, n);
}

int fused_mha_backward(const void* query_ptr, const void* key_ptr, const void* value_ptr, const void* output_ptr,
                       const void* d_output_ptr, const void* lse_ptr, void* workspace, size_t workspace_bytes,
                       void* d_query_ptr, void* d_key_ptr, void* d_value_ptr, int batch, int head, int m, int n,
                       int d, float scale, int causal, void* stream) {
  return dispatch_backward(kPassAll, query_ptr, nullptr, key_ptr, nullptr, value_ptr, nullptr, output_ptr,
                           d_output_ptr, nullptr, lse_ptr, workspace, workspace_bytes, d_query_ptr, d_key_ptr,
                           d_value_ptr, batch, head, m, n, d, scale, causal, stream);
}

int fused_mha_backward_noalloc(const void* query_ptr, const void* key_ptr, const void* value_ptr,
                               const void* output_ptr, const void* d_output_ptr, const void* lse_ptr,
                               void* d_query_ptr, void* d_key_ptr, void* d_value_ptr, int batch, int head, int m,
                               int n, int d, float scale, int causal, void* stream) {
  if (int rc = check_shape(batch, head, m, n, d)) return rc;
  const size_t rows = (size_t)batch * head * n;
  if (rows > (size_t)FUSED_MHA_NOALLOC_MAX_ROWS) return FUSED_MHA_ERR_SCRATCH_LIMIT;
  void* ws = nullptr;
  if (int rc = scratch_for_device(&ws)) return rc;
  // Every workspace element the dK/dV pass reads is written by the dQ pass of
  // the same call (rows 0 .. batch*head*n-1 of both halves), so nothing from
  // an earlier call is ever read and nothing needs clearing.
  return dispatch_backward(kPassAll, query_ptr, nullptr, key_ptr, nullptr, value_ptr, nullptr, output_ptr,
                           d_output_ptr, nullptr, lse_ptr, ws, 2 * rows * sizeof(float), d_query_ptr, d_key_ptr,
                           d_value_ptr, batch, head, m, n, d, scale, causal, stream);
}

int fused_mha_backward_strided(const void* query_ptr, const fused_mha_strides* query_strides, const void* key_ptr,
                               const fused_mha_strides* key_strides, const void* value_ptr,
                               const fused_mha_strides* value_strides, const void* output_ptr,
                               const void* d_output_ptr, const fused_mha_strides* d_output_strides,
                               const void* lse_ptr, void* workspace, size_t workspace_bytes, void* d_query_ptr,
                               void* d_key_ptr, void* d_value_ptr, int batch, int head, int n, int d, float scale,
                               int causal, void* stream) {
  return dispatch_backward(kPassAll, query_ptr, query_strides, key_ptr, key_strides, value_ptr, value_strides,
                           output_ptr, d_output_ptr, d_output_strides, lse_ptr, workspace, workspace_bytes,
                           d_query_ptr, d_key_ptr, d_value_ptr, batch, head, n, n, d, scale, causal, stream);
}

int fused_mha_backward_delta(const void* output_ptr, const void* d_output_ptr, const void* lse_ptr, void* workspace,
                             size_t workspace_bytes, int batch, int head, int n, int d, void* stream) {
  return dispatch_backward(kPassDelta, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, output_ptr, d_output_ptr,
                           nullptr, lse_ptr, workspace, workspace_bytes, nullptr, nullptr, nullptr, batch, head, n, n,
                           d, 1.f, 0, stream);
}

int fused_mha_backward_dq(const void* query_ptr, const void* key_ptr, const void* value_ptr,
                          const void* d_output_ptr, const void* lse_ptr, void* workspace, size_t workspace_bytes,
                          void* d_query_ptr, int batch, int head, int n, int d, float scale, int causal,
                          void* stream) {
  return dispatch_backward(kPassDq, query_ptr, nullptr, key_ptr, nullptr, value_ptr, nullptr, nullptr, d_output_ptr,
                           nullptr, lse_ptr, workspace, workspace_bytes, d_query_ptr, nullptr, nullptr, batch, head, n,
                           n, d, scale, causal, stream);
}

int fused_mha_backward_dkdv(const void* query_ptr, const void* key_ptr, const void* value_ptr,
                            const void* d_output_ptr, const void* lse_ptr, void* workspace, size_t workspace_bytes,
                            void* d_key_ptr, void* d_value_ptr, int batch, int head, int n, int d, float scale,
                            int causal, void* stream) {
  return dispatch_backward(kPassDkDv, query_ptr, nullptr, key_ptr, nullptr, value_ptr, nullptr, nullptr, d_output_ptr,
                           nullptr, lse_ptr, workspace, workspace_bytes, nullptr, d_key_ptr, d_value_ptr, batch, head,
                           n, n, d, scale, causal, stream);
}

const char* fused_mha_error_string(int code) {
  switch (code) {
    case FUSED_MHA_OK: return "ok";
    case FUSED_MHA_ERR_NULL_POINTER: return "a required pointer is NULL";
    case FUSED_MHA_ERR_BAD_SHAPE: return "bad shape: need batch, head, n > 0, m == n and a large enough workspace";
    case FUSED_MHA_ERR_BAD_HEAD_DIM: return "head dimension must be 64 or 128";
    case FUSED_MHA_ERR_MISALIGNED: return "a pointer is not 16-byte aligned";
    case FUSED_MHA_ERR_LAUNCH: return "the HIP runtime refused a kernel launch";
    case FUSED_MHA_ERR_BAD_SCALE: return "scale must be finite";
    case FUSED_MHA_ERR_TOO_LARGE:
      return "problem too large: need n < 2^29, head * d < 2^24, ceil(n/128) * batch * head < 2^23 and "
             "batch * head * n * d / 8 < 2^32";
    case FUSED_MHA_ERR_BAD_STRIDE:
      return "strides must be non-negative multiples of 8 elements, sequence stride below 2^24, head stride below 2^31";
    case FUSED_MHA_ERR_SCRATCH_LIMIT:
      return "batch * head * n exceeds FUSED_MHA_NOALLOC_MAX_ROWS, the size of the static scratch";
    case FUSED_MHA_ERR_RUNTIME: return "a HIP runtime query failed (current device, scratch address)";
    default: return "unknown fused_mha error code";
  }
}

}  // extern "C"
