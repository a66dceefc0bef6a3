// Device layout of 4-bit codes (Q4_0 and W4_GROUP alike).
//
// A row of weights is cut into 16-byte chunks of 32 consecutive k.  A chunk is
// four 32-bit words; word t holds elements 8t .. 8t+7, and inside a word
// nibble p holds element
//         E[p] = { 0, 2, 4, 6, 1, 3, 5, 7 }[p]
// so that ((w >> 4s) & 0x000F000F) is the pair (element 2s, element 2s+1) in
// the low and high half-words: one shift and one and-or turn a word into four
// packed bf16 pairs in k order, which is what the bf16 dot and MFMA operands
// want.  The logical layouts (Q4_0's split-half blocks, W4_GROUP's even/odd
// bytes) are converted to this once at load time and stay the interchange.
#pragma once
#include <stdint.h>

namespace nq {

// 8 codes in element order -> one word
__device__ __forceinline__ uint32_t nib_pack8(const uint8_t* e) {
    return (uint32_t)(e[0] & 0xF) | ((uint32_t)(e[2] & 0xF) << 4) | ((uint32_t)(e[4] & 0xF) << 8) |
           ((uint32_t)(e[6] & 0xF) << 12) | ((uint32_t)(e[1] & 0xF) << 16) | ((uint32_t)(e[3] & 0xF) << 20) |
           ((uint32_t)(e[5] & 0xF) << 24) | ((uint32_t)(e[7] & 0xF) << 28);
}

// one word -> 8 codes in element order, as floats
__device__ __forceinline__ void nib_unpack8(uint32_t w, float* e) {
    e[0] = (float)(w & 0xF);
    e[2] = (float)((w >> 4) & 0xF);
    e[4] = (float)((w >> 8) & 0xF);
    e[6] = (float)((w >> 12) & 0xF);
    e[1] = (float)((w >> 16) & 0xF);
    e[3] = (float)((w >> 20) & 0xF);
    e[5] = (float)((w >> 24) & 0xF);
    e[7] = (float)(w >> 28);
}

}  // namespace nq
