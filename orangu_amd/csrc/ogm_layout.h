// Tile-planar weight layout shared by the host repacker and the device kernels.
//
// A matrix is a flat sequence of "units" in row-major order: one unit is one GGUF block
// (Q8_0: 34 B / 32 weights; Q4_K: 144 B / 256; Q6_K: 210 B / 256; engine/quant.rs:638-787).
// Units are grouped 64 to a tile.  A unit is cut into 16-byte pieces plus a short tail; inside
// a tile, piece p of lane l sits at p*1024 + l*16 and the tails follow all pieces, lane after
// lane.  A wave whose lane l owns unit (tile*64 + l) therefore reads each piece of its 64
// units as one contiguous, 16-byte-aligned kilobyte, whatever the block size.  No byte of a
// block is changed, dropped or reinterpreted; the last tile is zero-padded.
//
//   type   pieces                                   tail
//   Q8_0   2  (qs[0..32))                           d      (2 B)
//   Q4_K   9  (d,dmin,scales | qs[0..128))          -
//   Q6_K   13 (ql[0..128) | qh[0..64) | scales)     d      (2 B)
#pragma once
#include <stddef.h>
#include <stdint.h>

#define OGM_Q8_0 8u
#define OGM_Q4_K 12u
#define OGM_Q6_K 14u

#define OGM_TILE_UNITS 64u

struct OgmLayout {
  uint32_t block_bytes;   // raw bytes per unit
  uint32_t block_elems;   // weights per unit
  uint32_t pieces;        // 16-byte pieces per unit
  uint32_t tail_bytes;    // bytes after the pieces (0 or 2)
  uint32_t piece_off;     // raw offset of piece 0 inside the block
  uint32_t tail_off;      // raw offset of the tail inside the block
  uint32_t tile_bytes;    // 64 * block_bytes
};

#if defined(__HIPCC__) || defined(__CUDACC__)
#define OGM_HD __host__ __device__
#else
#define OGM_HD
#endif

OGM_HD inline bool ogm_layout_for(uint32_t ggml_type, OgmLayout *l) {
  switch (ggml_type) {
    case OGM_Q8_0:  // d:f16 | qs:i8[32]
      *l = OgmLayout{34, 32, 2, 2, 2, 0, 64 * 34};
      return true;
    case OGM_Q4_K:  // d:f16 | dmin:f16 | scales:u8[12] | qs:u8[128]
      *l = OgmLayout{144, 256, 9, 0, 0, 0, 64 * 144};
      return true;
    case OGM_Q6_K:  // ql:u8[128] | qh:u8[64] | scales:i8[16] | d:f16
      *l = OgmLayout{210, 256, 13, 2, 0, 208, 64 * 210};
      return true;
    default:
      return false;
  }
}
