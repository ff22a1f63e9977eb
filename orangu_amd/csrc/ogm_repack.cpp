// Host-side repack of raw GGUF rows into the tile-planar layout, and its exact inverse.
// The layout itself is described in ogm_layout.h.  Input is QuantMatrix::raw_bytes()
// (engine/loader.rs:608-610): out_dim rows of row_bytes, rows contiguous.
#include <string.h>

#include "../../include/orangu_mi355x.h"
#include "ogm_layout.h"

extern "C" int ogm_supports_type(uint32_t ggml_type) {
  return ggml_type == OGM_Q8_0 || ggml_type == OGM_Q4_K || ggml_type == OGM_Q6_K;
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

static size_t n_tiles_for(const OgmLayout &l, uint32_t in_dim, uint32_t out_dim) {
  size_t units = (size_t)out_dim * (in_dim / l.block_elems);
  return (units + OGM_TILE_UNITS - 1) / OGM_TILE_UNITS;
}

extern "C" size_t ogm_repacked_size(uint32_t ggml_type, uint32_t in_dim, uint32_t out_dim) {
  OgmLayout l;
  if (!ogm_layout_for(ggml_type, &l) || in_dim % l.block_elems != 0) return 0;
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
  // Rows are contiguous and a row is a whole number of blocks, so the matrix is one flat run
  // of blocks.
  size_t units = (size_t)out_dim * (in_dim / l.block_elems);
  size_t tiles = n_tiles_for(l, in_dim, out_dim);
  size_t last_full = units / OGM_TILE_UNITS;
  if (last_full < tiles) memset(dst + last_full * l.tile_bytes, 0, l.tile_bytes);
  for (size_t u = 0; u < units; u++) {
    const uint8_t *b = src + u * l.block_bytes;
    uint8_t *tile = dst + (u / OGM_TILE_UNITS) * l.tile_bytes;
    size_t lane = u % OGM_TILE_UNITS;
    for (uint32_t p = 0; p < l.pieces; p++)
      memcpy(tile + p * 1024 + lane * 16, b + l.piece_off + p * 16, 16);
    if (l.tail_bytes)
      memcpy(tile + l.pieces * 1024 + lane * l.tail_bytes, b + l.tail_off, l.tail_bytes);
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
  size_t units = (size_t)out_dim * (in_dim / l.block_elems);
  for (size_t u = 0; u < units; u++) {
    uint8_t *b = dst + u * l.block_bytes;
    const uint8_t *tile = src + (u / OGM_TILE_UNITS) * l.tile_bytes;
    size_t lane = u % OGM_TILE_UNITS;
    for (uint32_t p = 0; p < l.pieces; p++)
      memcpy(b + l.piece_off + p * 16, tile + p * 1024 + lane * 16, 16);
    if (l.tail_bytes)
      memcpy(b + l.tail_off, tile + l.pieces * 1024 + lane * l.tail_bytes, l.tail_bytes);
  }
  return OGM_OK;
}
