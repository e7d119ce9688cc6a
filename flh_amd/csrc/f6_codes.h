// The 6-bit (e3m2) encoding of int4 codes used by the operands of the 6-bit matrix instruction.
#pragma once
#include "lane_ops.h"

namespace flh {

constexpr int kF6BlockBytes = 96;   // encoded bytes of 128 codes of one row

// Eight int4 nibbles of one dword (two's complement; nibble j in bits 4 j) -> 48 bits of e3m2 codes, code j at
// bit 6 j.  A code is sign << 5 | {0, 12, 16, 18, 20, 21, 22, 23, 24}[magnitude]: a 16-entry byte table, looked up
// four nibbles at a time with two byte permutes (entries 0..7 and 8..15) and a bit select on the nibble's top bit.
__device__ __forceinline__ unsigned long long bf6_of_nibbles(unsigned w) {
  constexpr unsigned kPosLo = 0x12100C00u, kPosHi = 0x17161514u;   //  0 ..  7
  constexpr unsigned kNegLo = 0x35363738u, kNegHi = 0x2C303234u;   // -8 .. -1
  auto lut = [&](unsigned x) {                         // four nibbles, one per byte
    const unsigned sel = x & 0x07070707u;
    const unsigned pos = __builtin_amdgcn_perm(kPosHi, kPosLo, sel), neg = __builtin_amdgcn_perm(kNegHi, kNegLo, sel);
    const unsigned mask = ((x >> 3) & 0x01010101u) * 0xFFu;
    return (neg & mask) | (pos & ~mask);
  };
  const unsigned L = lut(w & 0x0F0F0F0Fu), H = lut((w >> 4) & 0x0F0F0F0Fu);   // codes 0,2,4,6 and 1,3,5,7
  // pairs p_i = code(2 i) | code(2 i + 1) << 6 in 16-bit lanes
  const unsigned X = (L & 0x00FF00FFu) | ((H & 0x00FF00FFu) << 6);           // p0, p2
  const unsigned Y = ((L >> 8) & 0x00FF00FFu) | (((H >> 8) & 0x00FF00FFu) << 6);   // p1, p3
  const unsigned long long p0 = X & 0xFFFu, p2 = X >> 16, p1 = Y & 0xFFFu, p3 = Y >> 16;
  return p0 | (p1 << 12) | (p2 << 24) | (p3 << 36);
}

// Store the eight codes of one lane (nibble dword w, chunk c16 = 0 .. 15 of a 128-code block) into the block's 96 bytes.
// A lane's codes are 48 bits; the four lanes of a hardware quad must own the chunks 4 p .. 4 p + 3 of one 24-byte piece
// with chunk index and quad position differing by a constant XOR (the lane labellings of the quantiser kernels do):
// three of them store eight bytes each after fetching their successor's bits from the lane whose chunk index is one
// higher -- the xor-1 resp. xor-3 partner.  Every lane of the wave must call it (cross-lane reads).
__device__ __forceinline__ void f6_store_chunk(unsigned w, int c16, uint8_t* block, bool valid) {
  const unsigned long long own = bf6_of_nibbles(w);
  const unsigned lo = (unsigned)own, hi = (unsigned)(own >> 32);
  constexpr int kQuadXor3 = 0x1B;                       // quad_perm:[3,2,1,0]
  const int role = c16 & 3;                             // position of this lane's 48 bits inside the 24-byte piece
  const unsigned x1lo = (unsigned)dpp_i<kDppQuadXor1>((int)lo), x1hi = (unsigned)dpp_i<kDppQuadXor1>((int)hi);
  const unsigned x3lo = (unsigned)dpp_i<kQuadXor3>((int)lo), x3hi = (unsigned)dpp_i<kQuadXor3>((int)hi);
  const unsigned nlo = role == 1 ? x3lo : x1lo, nhi = role == 1 ? x3hi : x1hi;
  const unsigned long long next = (unsigned long long)nlo | ((unsigned long long)nhi << 32);
  const unsigned long long word = role == 0 ? own | (next << 48) : role == 1 ? (own >> 16) | (next << 32)
                                                                            : (own >> 32) | (next << 16);
  if (valid && role < 3) {
    uint8_t* dst = block + 48 * ((c16 >> 2) & 1) + 24 * (c16 >> 3) + 8 * role;
    *(v2i*)dst = v2i{(int)(unsigned)word, (int)(unsigned)(word >> 32)};
  }
}

}  // namespace flh
