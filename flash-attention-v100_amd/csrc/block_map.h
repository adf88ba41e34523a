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
#endif  // FMHA_BLOCK_MAP_H_
