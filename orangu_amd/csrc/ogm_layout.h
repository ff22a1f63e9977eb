// Tile-planar weight layout shared by the host repacker and the device kernels.
//
// A matrix is out_dim rows of `upr` blocks ("units"; one unit is one GGUF block: Q8_0 34 B / 32
// weights, Q4_0 and IQ4_NL 18 B / 32, Q5_0 22 B / 32, Q5_1 24 B / 32, Q2_K 84 B / 256, Q3_K 110 B / 256, Q4_K 144 B / 256,
// Q5_K 176 B / 256, Q6_K 210 B / 256, IQ4_XS 136 B / 256; engine/quant.rs:537-871, 1350-1375).  A *tile* holds 64
// units: R consecutive rows x C consecutive blocks, R = 64 / C.  C = 4 when a row has a multiple of four
// blocks, and also when filling its last column tile with zero units adds at most a tenth to the row (11, 19,
// 22, 23 blocks and every count from 27 on): bytes that no kernel's sums read, which keep row blocks at 16 rows
// -- a row of 43 blocks (11008 inputs) in tiles one block wide would make row blocks of 64 rows and a quarter as
// many workgroups in the decode GEMV.  Other rows take C = 2, else 1.  Tiles are ordered [row block][column
// tile]; inside a tile the unit of (row r, block c) is lane c*R + r.
//
// A unit is cut into 16-byte pieces plus a short tail; piece p of lane l sits at p*1024 + l*16
// and the tails follow all pieces, lane after lane.  So
//   * a wave whose lane l owns the tile's unit l reads every piece of its 64 units as one
//     contiguous, 16-byte-aligned kilobyte, whatever the block size (decode GEMV);
//   * the R rows of one block column are R consecutive lanes, i.e. a contiguous run of R*16
//     bytes per piece, which is what a tiled GEMM over a row block fetches (prefill GEMM).
// No byte of a block is changed, dropped or reinterpreted; rows beyond out_dim in the last row
// block, and blocks beyond a row's last in a padded column tile, are zero units.  A block whose size is not piece-sized or piece-sized plus two (Q3_K: 110)
// has its last piece zero-padded to 16 bytes: tile_bytes is then 64 * 16 * pieces.
//
//   type   pieces                                   tail
//   Q8_0   2  (qs[0..32))                           d      (2 B)
//   Q4_0   1  (qs[0..16))                           d      (2 B)      (IQ4_NL the same)
//   Q5_0   1  (qs[0..16))                           d, qh  (6 B)
//   Q5_1   1  (qs[0..16))                           d, m, qh (8 B)
//   Q2_K   5  (scales[0..16) | qs[0..64))           d, dmin (4 B)
//   IQ4_XS 9  (d,scales_h,scales_l,qs[0..8) | qs[8..24) | ... | qs[120..128) + 8 bytes of padding)   -
//   Q3_K   7  (hmask[0..32) | qs[0..64) | scales,d + 2 bytes of padding)   -
//   Q4_K   9  (d,dmin,scales | qs[0..128))          -
//   Q5_K   11 (d,dmin,scales | qh[0..32) | qs)      -
//   Q6_K   13 (ql[0..128) | qh[0..64) | scales)     d      (2 B)
#pragma once
#include <stddef.h>
#include <stdint.h>

#define OGM_Q4_0 2u
#define OGM_Q5_0 6u
#define OGM_Q5_1 7u
#define OGM_Q8_0 8u
#define OGM_Q2_K 10u
#define OGM_Q3_K 11u
#define OGM_Q4_K 12u
#define OGM_Q5_K 13u
#define OGM_Q6_K 14u
#define OGM_IQ4_NL 20u
#define OGM_IQ4_XS 23u

#define OGM_TILE_UNITS 64u

struct OgmLayout {
  uint32_t block_bytes;   // raw bytes per unit
  uint32_t block_elems;   // weights per unit
  uint32_t pieces;        // 16-byte pieces per unit
  uint32_t tail_bytes;    // bytes kept after all pieces (0, 2, 4, 6 or 8), lane after lane
  uint32_t piece_off;     // raw offset of piece 0 inside the block
  uint32_t tail_off;      // raw offset of the tail inside the block
  uint32_t tile_bytes;    // 64 * block_bytes
};

// Shape of the tiling of one matrix.
struct OgmTiling {
  uint32_t upr;   // blocks per row
  uint32_t C;     // blocks per tile row (1, 2 or 4)
  uint32_t R;     // rows per tile (64 / C)
  uint32_t nct;   // column tiles per row block (ceil(upr / C): the last one may hold zero units)
  uint32_t nrb;   // row blocks (ceil(out_dim / R))
};

#if defined(__HIPCC__)
#define OGM_HD __host__ __device__
#else
#define OGM_HD
#endif

OGM_HD inline bool ogm_layout_for(uint32_t ggml_type, OgmLayout *l) {
  switch (ggml_type) {
    case OGM_Q4_0:    // d:f16 | qs:u8[16]
    case OGM_IQ4_NL:  // d:f16 | qs:u8[16] (codebook indices)
      *l = OgmLayout{18, 32, 1, 2, 2, 0, 64 * 18};
      return true;
    case OGM_Q5_0:  // d:f16 | qh:u32 | qs:u8[16]
      *l = OgmLayout{22, 32, 1, 6, 6, 0, 64 * 22};
      return true;
    case OGM_Q5_1:  // d:f16 | m:f16 | qh:u32 | qs:u8[16]
      *l = OgmLayout{24, 32, 1, 8, 8, 0, 64 * 24};
      return true;
    case OGM_Q2_K:  // scales:u8[16] | qs:u8[64] | d:f16 | dmin:f16
      *l = OgmLayout{84, 256, 5, 4, 0, 80, 64 * 84};
      return true;
    case OGM_IQ4_XS:  // d:f16 | scales_h:u16 | scales_l:u8[4] | qs:u8[128]; the last piece holds 8 bytes
      *l = OgmLayout{136, 256, 9, 0, 0, 0, 64 * 144};
      return true;
    case OGM_Q8_0:  // d:f16 | qs:i8[32]
      *l = OgmLayout{34, 32, 2, 2, 2, 0, 64 * 34};
      return true;
    case OGM_Q3_K:  // hmask:u8[32] | qs:u8[64] | scales:u8[12] | d:f16; the last piece holds 14 bytes
      *l = OgmLayout{110, 256, 7, 0, 0, 0, 64 * 112};
      return true;
    case OGM_Q4_K:  // d:f16 | dmin:f16 | scales:u8[12] | qs:u8[128]
      *l = OgmLayout{144, 256, 9, 0, 0, 0, 64 * 144};
      return true;
    case OGM_Q5_K:  // d:f16 | dmin:f16 | scales:u8[12] | qh:u8[32] | qs:u8[128]
      *l = OgmLayout{176, 256, 11, 0, 0, 0, 64 * 176};
      return true;
    case OGM_Q6_K:  // ql:u8[128] | qh:u8[64] | scales:i8[16] | d:f16
      *l = OgmLayout{210, 256, 13, 2, 0, 208, 64 * 210};
      return true;
    default:
      return false;
  }
}

OGM_HD inline OgmTiling ogm_tiling_for(uint32_t upr, uint32_t out_dim) {
  OgmTiling t;
  t.upr = upr;
  const uint32_t pad = (4u - upr % 4u) % 4u;   // zero units a row would need to fill its last tile of four
  t.C = (pad == 0 || pad * 10u <= upr) ? 4u : ((upr % 2u == 0) ? 2u : 1u);
  t.R = OGM_TILE_UNITS / t.C;
  t.nct = (upr + t.C - 1u) / t.C;
  t.nrb = (out_dim + t.R - 1) / t.R;
  return t;
}

// Tile index and lane of the unit (row, block).
OGM_HD inline void ogm_unit_place(const OgmTiling &t, uint32_t row, uint32_t block, size_t *tile,
                                  uint32_t *lane) {
  *tile = (size_t)(row / t.R) * t.nct + block / t.C;
  *lane = (block % t.C) * t.R + row % t.R;
}
