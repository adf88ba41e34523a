// Mapping of work-group ids to (slice, block) for the attention kernels; plain
// C++ so that a host program can check it exhaustively.
#ifndef FMHA_BLOCK_MAP_H_
#define FMHA_BLOCK_MAP_H_

#if defined(__HIPCC__)
#define FMHA_HOST_DEVICE __host__ __device__ inline
#else
#define FMHA_HOST_DEVICE inline
#endif

// Work-group id -> (batch*head slice, block inside the slice).  Consecutive
// work-group ids go round-robin over the 8 XCDs, each with a private L2; the
// remap hands every XCD whole (batch, head) slices, so the blocks that stream
// the same K/V (or Q/dO) rows share one L2.  An XCD takes its slices in groups
// of kSlicesInFlight: inside a group the blocks are ordered block-index major,
// and callers number blocks heaviest first, so under causal masking the heavy
// blocks of a group start before its light ones while the rows being streamed
// at any time (kSlicesInFlight slices) stay within the 4 MiB L2.
// When the slice count is no multiple of 8, the slices / 8 (rounded down)
// slices per XCD are handled as above by the first work-group ids; the blocks
// of the remaining slices % 8 slices follow in slice-major order, cut into 8
// contiguous runs, one per XCD, so that each of those slices is shared by as
// few XCDs as possible.
#ifndef FMHA_SLICES_IN_FLIGHT
#define FMHA_SLICES_IN_FLIGHT 2
#endif
constexpr int kSlicesInFlight = FMHA_SLICES_IN_FLIGHT;
FMHA_HOST_DEVICE void fmha_slice_and_block(int lin, int slices, int blocks_per_slice, int& slice,
                                                            int& blk) {
  const int q = slices >> 3, r = slices & 7;
  const int main_blocks = 8 * q * blocks_per_slice;
  if (lin < main_blocks) {
    const int xcd = lin & 7, slot = lin >> 3;  // slot: 0 .. q * blocks_per_slice - 1 inside the XCD
    const int group_blocks = kSlicesInFlight * blocks_per_slice;
    const int group = slot / group_blocks, within = slot - group * group_blocks;
    const int first = group * kSlicesInFlight;
    const int g = (q - first < kSlicesInFlight ? q - first : kSlicesInFlight);  // slices in this group
    blk = within / g;
    slice = xcd * q + first + (within - blk * g);
  } else {
    const int rem = lin - main_blocks, n_rem = r * blocks_per_slice;
    const int xcd = rem & 7, slot = rem >> 3;
    const int idx = xcd * (n_rem >> 3) + (xcd < (n_rem & 7) ? xcd : (n_rem & 7)) + slot;  // position in the slice-major list
    const int s = idx / blocks_per_slice;
    slice = 8 * q + s;
    blk = idx - s * blocks_per_slice;
  }
}

// Persistent launches: G work groups (one per CU) share the `total` blocks numbered as above.
// Work group w takes, in round r, block r * G + w for even r and r * G + (w mirrored inside its
// XCD, i.e. among the work groups congruent to w modulo 8) for odd r.  Both keep the block number
// congruent to w modulo 8, so the block stays on w's XCD, and the alternation pairs the heavy
// blocks of one round with the light blocks of the next (blocks are numbered heaviest first).
// G must be a multiple of 8 unless the launch has a single round (total <= G).
// fmha_persistent_block: the block of work group w in round r; >= total means none.
// fmha_persistent_next_round: the next round after r in which w has a block, or -1.
FMHA_HOST_DEVICE int fmha_persistent_block(int r, int w, int G) {
  const int p = (r & 1) ? (((G >> 3) - 1 - (w >> 3)) << 3) + (w & 7) : w;
  return r * G + p;
}
FMHA_HOST_DEVICE int fmha_persistent_next_round(int r, int w, int G, int total) {
  for (++r; (long)r * G < total; ++r)
    if (fmha_persistent_block(r, w, G) < total) return r;
  return -1;
}
#endif  // FMHA_BLOCK_MAP_H_
