// Lane offsets of the HBM -> LDS copies whose slab offset rides in the copy's scalar offset.
//
// A buffer copy's range check covers the lane offset only; the scalar offset is added afterwards, unchecked.  A lane
// whose lane offset passes the check must therefore stay inside the operand for every scalar offset the kernel ever
// pairs it with.  Rows of A past the end fail the check by construction (their offset starts beyond the last row);
// columns of B past the end would not - (k, column >= N) is a valid offset of some element of a later row, and on
// the last slab the scalar offset pushes it past the end of B.  Those lanes get kCopyOutOfRange instead, which fails
// the check against any operand these kernels accept (sizes below 2^32 - 1024 bytes), so they read zeros and touch
// no memory.
//
// Plain functions of integers, compiled for the device by the kernels and for the host by the test that enumerates
// every (lane offset, scalar offset) pair of ragged shapes against the operand's size.
#pragma once

#if defined(__HIPCC__)
#define TFCC_OFFSETS_HD __host__ __device__ __forceinline__
#else
#define TFCC_OFFSETS_HD inline
#endif

namespace tfcc_rocm {
namespace copy_offsets {

constexpr unsigned kCopyOutOfRange = 0xffffff00u;

// ---- int8 kernel of 256 x 256 tiles, slabs of BK bytes of k, 256 threads.
// B slot s (16 bytes) of a slab holds k row s / 16, physical chunk s % 16; copy c of a thread moves slot
// c * 256 + tid.  The logical chunk is the inverse of physical = ((chunk >> 1) ^ k) & 7 | (chunk & 1) << 3.
TFCC_OFFSETS_HD unsigned w4_b_lane_offset(int tid, int c, unsigned n0, unsigned N) {
  const int k = (tid >> 4) + 16 * c, ph = tid & 15;
  const int chunk = ((((ph & 7) ^ k) & 7) << 1) | (ph >> 3);
  const unsigned col = n0 + ((unsigned)chunk << 4);
  return col < N ? (unsigned)k * N + col : kCopyOutOfRange;
}
// scalar offset of slab `slab` (of KT) on the B side
TFCC_OFFSETS_HD unsigned w4_b_slab_offset(unsigned slab, unsigned KT, unsigned BK, unsigned N) {
  const unsigned sl = slab < KT - 1 ? slab : KT - 1;
  return sl * BK * N;
}
// A slot s holds row s / CH, physical chunk s % CH (CH = BK / 16); logical chunk = physical ^ swizzle(row)
TFCC_OFFSETS_HD unsigned w4_a_lane_offset(int tid, int c, unsigned m0, unsigned K, int BK) {
  const int CH = BK / 16, RPS = 256 / BK;
  const int row = tid / CH + c * (256 / CH), phys = tid % CH;
  const int swz = (row / RPS) & (CH - 1);
  return (m0 + (unsigned)row) * K + ((unsigned)(phys ^ swz) << 4);
}

// ---- fp32 kernel of one wavefront per 32 rows: B image of a ring slab, BCH = BN / 4 chunks of four floats per k row,
// slot s = unit * 64 + lane holds k row s / BCH, chunk s % BCH.  Offsets in bytes.
TFCC_OFFSETS_HD unsigned w96_b_lane_offset(int slot, int BCH, unsigned n0, unsigned N, unsigned ldb) {
  const int k = slot / BCH, ch = slot % BCH;
  const unsigned col = n0 + (unsigned)ch * 4u;
  return col < N ? ((unsigned)k * ldb + col) * 4u : kCopyOutOfRange;
}

}  // namespace copy_offsets
}  // namespace tfcc_rocm
