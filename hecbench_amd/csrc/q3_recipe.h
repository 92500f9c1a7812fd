// Bit-field recipe shared by the GPTQ 3-bit matvec and GEMM kernels.
//
// A k-group of one weight column is a 96-bit string (three consecutive packed
// rows, word 0 lowest) holding 32 codes, code k at bits 3k..3k+2
// (layout of src/quant3MatMul-hip/kernels.h:42-86 in the HeCBench tree).
//
// The kernels never convert a code to a float.  An fp16 whose exponent field is
// zero is a subnormal of value mantissa * 2^-24, so a 3-bit code left in place at
// bit p (p <= 7) of an otherwise zero 16-bit half IS the fp16 number
// code * 2^(p-24).  One AND with a two-field mask therefore turns a 32-bit
// window of the string into two fp16 MFMA operands; the 2^p factor is folded into
// the activation that multiplies that slot.  Seven windows (three of them are the
// words themselves, four cost one funnel shift each) cover all 32 codes with
// exactly 16 registers: 20 VALU instructions per 32 weights.
#pragma once

#include <stdint.h>

namespace hq_q3 {

struct Field2 {
  int window;  // index into kWindowOffset
  int k_lo, p_lo;  // code index and bit position inside the low half
  int k_hi, p_hi;  // same for the high half (position relative to bit 16)
};

// Bit offset of each 32-bit window inside the 96-bit string.
constexpr int kWindowOffset[7] = {0, 4, 10, 32, 41, 64, 71};

constexpr Field2 kRecipe[16] = {
    {0, 0, 0, 6, 2},   {0, 1, 3, 7, 5},                      // word 0
    {1, 2, 2, 8, 4},   {1, 3, 5, 9, 7},                      // bits 4..35
    {2, 4, 2, 10, 4},  {2, 5, 5, 11, 7},                     // bits 10..41
    {3, 12, 4, 17, 3}, {3, 13, 7, 18, 6},                    // word 1
    {4, 14, 1, 19, 0}, {4, 15, 4, 20, 3}, {4, 16, 7, 21, 6}, // bits 41..72
    {5, 22, 2, 27, 1}, {5, 23, 5, 28, 4},                    // word 2
    {6, 24, 1, 29, 0}, {6, 25, 4, 30, 3}, {6, 26, 7, 31, 6}, // bits 71..95
};

constexpr uint32_t mask_of(int r) {
  return (7u << kRecipe[r].p_lo) | (7u << (16 + kRecipe[r].p_hi));
}

// Operand slot (0..31: register r, half h -> 2r+h) that carries code k.
constexpr int slot_of(int k) {
  for (int r = 0; r < 16; ++r) {
    if (kRecipe[r].k_lo == k) return 2 * r;
    if (kRecipe[r].k_hi == k) return 2 * r + 1;
  }
  return -1;
}
// Bit position of code k inside its half: the operand value is code * 2^(pos-24).
constexpr int pos_of(int k) {
  for (int r = 0; r < 16; ++r) {
    if (kRecipe[r].k_lo == k) return kRecipe[r].p_lo;
    if (kRecipe[r].k_hi == k) return kRecipe[r].p_hi;
  }
  return -1;
}

constexpr bool recipe_is_consistent() {
  for (int k = 0; k < 32; ++k) {
    int hits = 0;
    for (int r = 0; r < 16; ++r) {
      const Field2& f = kRecipe[r];
      const int off = kWindowOffset[f.window];
      if (f.k_lo == k) {
        ++hits;
        if (3 * k - off != f.p_lo || f.p_lo < 0 || f.p_lo > 7) return false;
      }
      if (f.k_hi == k) {
        ++hits;
        if (3 * k - off - 16 != f.p_hi || f.p_hi < 0 || f.p_hi > 7) return false;
      }
    }
    if (hits != 1) return false;
  }
  return true;
}
static_assert(recipe_is_consistent(), "every code must be covered once, inside the fp16 mantissa");

// Per-register facts packed for in-register lookup: entry r (16 bits) holds
// k_lo | k_hi << 5 | p_lo << 10 | p_hi << 13; four entries per 64-bit word.
constexpr uint64_t packed_entries(int word) {
  uint64_t v = 0;
  for (int i = 0; i < 4; ++i) {
    const Field2& f = kRecipe[4 * word + i];
    const uint64_t e = (uint64_t)f.k_lo | ((uint64_t)f.k_hi << 5) | ((uint64_t)f.p_lo << 10) |
                       ((uint64_t)f.p_hi << 13);
    v |= e << (16 * i);
  }
  return v;
}

struct SlotTable {
  uint8_t slot[32];
  uint8_t pos[32];
};
constexpr SlotTable make_slot_table() {
  SlotTable t{};
  for (int k = 0; k < 32; ++k) {
    t.slot[k] = (uint8_t)slot_of(k);
    t.pos[k] = (uint8_t)pos_of(k);
  }
  return t;
}

}  // namespace hq_q3
