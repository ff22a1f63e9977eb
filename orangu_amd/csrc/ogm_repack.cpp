// Host-side repack of raw GGUF rows into the tile-planar layout, and its exact inverse.
// The layout itself (64-unit tiles of R rows x C blocks) is described in ogm_layout.h.  Input is QuantMatrix::raw_bytes()
// (engine/loader.rs:608-610): out_dim rows of row_bytes, rows contiguous.
#include <string.h>

#include "../../include/orangu_mi355x.h"
#include "ogm_layout.h"

extern "C" int ogm_supports_type(uint32_t ggml_type) {
  return ggml_type == OGM_Q8_0 || ggml_type == OGM_Q5_0 || ggml_type == OGM_Q4_0 || ggml_type == OGM_IQ4_NL ||
         ggml_type == OGM_Q3_K || ggml_type == OGM_Q4_K || ggml_type == OGM_Q5_K || ggml_type == OGM_Q6_K ||
         ggml_type == OGM_Q5_1 || ggml_type == OGM_Q2_K || ggml_type == OGM_IQ4_XS;
}

extern "C" int ogm_supports(uint32_t ggml_type, uint32_t in_dim) {
  OgmLayout l;
  if (!ogm_layout_for(ggml_type, &l) || in_dim == 0) return 0;
  return in_dim % l.block_elems == 0;
}

extern "C" int ogm_block_layout(uint32_t ggml_type, uint32_t *block_bytes, uint32_t *block_elems) {
  OgmLayout l;
  if (!ogm_layout_for(ggml_type, &l)) return OGM_ERR_UNSUPPORTED;
  if (block_bytes) *block_bytes = l.block_bytes;
  if (block_elems) *block_elems = l.block_elems;
  return OGM_OK;
}

// Bytes of the raw block that piece p holds: 16, except a last piece that runs off the block.
static uint32_t piece_bytes(const OgmLayout &l, uint32_t p) {
  const uint32_t left = l.block_bytes - (l.piece_off + p * 16);
  return left < 16 ? left : 16;
}

static size_t n_tiles_for(const OgmLayout &l, uint32_t in_dim, uint32_t out_dim) {
  const OgmTiling t = ogm_tiling_for(in_dim / l.block_elems, out_dim);
  return (size_t)t.nrb * t.nct;
}

extern "C" size_t ogm_repacked_size(uint32_t ggml_type, uint32_t in_dim, uint32_t out_dim) {
  OgmLayout l;
  if (!ogm_layout_for(ggml_type, &l) || in_dim == 0 || in_dim % l.block_elems != 0) return 0;
  return n_tiles_for(l, in_dim, out_dim) * l.tile_bytes;
}

static int check_shape(uint32_t ggml_type, size_t row_bytes, uint32_t in_dim, uint32_t out_dim,
                       OgmLayout *l) {
  if (!ogm_layout_for(ggml_type, l)) return OGM_ERR_UNSUPPORTED;
  if (in_dim == 0 || out_dim == 0) return OGM_ERR_INVALID;
  if (in_dim % l->block_elems != 0) return OGM_ERR_UNSUPPORTED;
  // engine/loader.rs:1564-1570: row_bytes = in_dim / block_elems * block_bytes
  if (row_bytes != (size_t)(in_dim / l->block_elems) * l->block_bytes) return OGM_ERR_INVALID;
  return OGM_OK;
}

extern "C" int ogm_repack_host(uint32_t ggml_type, const void *raw, size_t row_bytes,
                               uint32_t in_dim, uint32_t out_dim, void *repacked) {
  OgmLayout l;
  int rc = check_shape(ggml_type, row_bytes, in_dim, out_dim, &l);
  if (rc != OGM_OK) return rc;
  if (!raw || !repacked) return OGM_ERR_INVALID;
  const uint8_t *src = (const uint8_t *)raw;
  uint8_t *dst = (uint8_t *)repacked;
  const OgmTiling t = ogm_tiling_for(in_dim / l.block_elems, out_dim);
  // Zero units: rows beyond out_dim (the last row block only) and, where a row's blocks do not fill its last
  // column tile, that tile of every row block.
  if (t.upr % t.C != 0)
    memset(dst, 0, (size_t)t.nrb * t.nct * l.tile_bytes);
  else if (out_dim % t.R != 0)
    memset(dst + (size_t)(t.nrb - 1) * t.nct * l.tile_bytes, 0, (size_t)t.nct * l.tile_bytes);
  for (uint32_t o = 0; o < out_dim; o++) {
    for (uint32_t blk = 0; blk < t.upr; blk++) {
      const uint8_t *b = src + (size_t)o * row_bytes + (size_t)blk * l.block_bytes;
      size_t tile_index;
      uint32_t lane;
      ogm_unit_place(t, o, blk, &tile_index, &lane);
      uint8_t *tile = dst + tile_index * l.tile_bytes;
      for (uint32_t p = 0; p < l.pieces; p++) {
        const uint32_t have = piece_bytes(l, p);   // 16, or what is left of the block
        uint8_t *dst_piece = tile + p * 1024 + lane * 16;
        memcpy(dst_piece, b + l.piece_off + p * 16, have);
        if (have < 16) memset(dst_piece + have, 0, 16 - have);
      }
      if (l.tail_bytes)
        memcpy(tile + l.pieces * 1024 + lane * l.tail_bytes, b + l.tail_off, l.tail_bytes);
    }
  }
  return OGM_OK;
}

extern "C" int ogm_unrepack_host(uint32_t ggml_type, const void *repacked, size_t row_bytes,
                                 uint32_t in_dim, uint32_t out_dim, void *raw) {
  OgmLayout l;
  int rc = check_shape(ggml_type, row_bytes, in_dim, out_dim, &l);
  if (rc != OGM_OK) return rc;
  if (!raw || !repacked) return OGM_ERR_INVALID;
  const uint8_t *src = (const uint8_t *)repacked;
  uint8_t *dst = (uint8_t *)raw;
  const OgmTiling t = ogm_tiling_for(in_dim / l.block_elems, out_dim);
  for (uint32_t o = 0; o < out_dim; o++) {
    for (uint32_t blk = 0; blk < t.upr; blk++) {
      uint8_t *b = dst + (size_t)o * row_bytes + (size_t)blk * l.block_bytes;
      size_t tile_index;
      uint32_t lane;
      ogm_unit_place(t, o, blk, &tile_index, &lane);
      const uint8_t *tile = src + tile_index * l.tile_bytes;
      for (uint32_t p = 0; p < l.pieces; p++)
        memcpy(b + l.piece_off + p * 16, tile + p * 1024 + lane * 16, piece_bytes(l, p));
      if (l.tail_bytes)
        memcpy(b + l.tail_off, tile + l.pieces * 1024 + lane * l.tail_bytes, l.tail_bytes);
    }
  }
  return OGM_OK;
}
