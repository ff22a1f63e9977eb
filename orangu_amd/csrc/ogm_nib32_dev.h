// Device helper shared by the GEMV format and the GEMM kernel of the symmetric per-32 nibble types
// (Q4_0, Q5_0, IQ4_NL; unpack_block_q5_bits and unpack_block_iq4_nl, vecdot.rs:913-1039).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

// Four nibbles `n` (one per byte, 0..15) as four signed int8 weights.  KIND 0: Q4_0, n - 8;
// KIND 1: Q5_0, (n | fifth bit) - 16 with the four fifth bits in the low bits of h4; KIND 2: IQ4_NL,
// n indexes the sixteen levels -127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89,
// 113 (iq_grids.rs:5941-5943); KIND 3: Q5_1, n | fifth bit, unsigned 0..31 (unpack_block_q5_1, vecdot.rs:1032).
template <int KIND>
__device__ __forceinline__ uint32_t ogm_nib32_weights(uint32_t n, uint32_t h4) {
  if (KIND == 2) {
    // sixteen-entry byte table: two eight-entry v_perm lookups, chosen by bit 3 of the index
    const uint32_t sel = n & 0x07070707u;
    const uint32_t lo = __builtin_amdgcn_perm(0xF6EADDCFu, 0xBFAD9881u, sel);   // levels 0..7
    const uint32_t hi = __builtin_amdgcn_perm(0x71594535u, 0x26190D01u, sel);   // levels 8..15
    const uint32_t pick = ((n >> 3) & 0x01010101u) * 0xFFu;
    return (lo & ~pick) | (hi & pick);
  }
  if (KIND == 3) return n | (((h4 * 0x00204081u) & 0x01010101u) << 4);
  // v - bias per byte without borrows between bytes: set bit 7, subtract, flip bit 7 back
  const uint32_t v = KIND == 1 ? (n | (((h4 * 0x00204081u) & 0x01010101u) << 4)) : n;
  const uint32_t bias = KIND == 1 ? 0x10101010u : 0x08080808u;
  return ((v | 0x80808080u) - bias) ^ 0x80808080u;
}
