// Internal helpers shared by the host and device translation units of libternary_spmm.
#pragma once
#include <cstdarg>
#include <cstdint>
#include <cstdio>

#include "ternary_spmm.h"

namespace tl {

// Stores a printf-formatted message in the calling thread's error slot and returns `code`.
int fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));

inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }
inline int64_t round_up(int64_t a, int64_t b) { return ceil_div(a, b) * b; }

// Descriptor word of one (column, tile): bits 0-7 number of +1 rows, bits 8-15
// number of -1 rows, bits 16-31 dword offset of the +1 run from the start of its (block, tile) chunk of the
// index stream (the -1 run follows the padded +1 run).
inline uint32_t make_desc(uint32_t n_pos, uint32_t n_neg, uint32_t dword_off)
{
    return (n_pos & 0xffu) | ((n_neg & 0xffu) << 8) | (dword_off << 16);
}

constexpr int kSentinel = 255;       // index byte that addresses the always-zero slot of a tile
constexpr int kTileSlots = 256;      // slots a staged tile occupies (tile_rows real rows + zeros)
constexpr int kMaxTileRows = 255;
// The single-row kernel lays the LDS images of consecutive tiles kTileSlots slots + this many bytes apart, so that
// equal slots of neighbouring tiles (the zero slot among them) fall on different LDS banks; the packer orders
// the rows of a run with that placement in mind.
constexpr int kSpmvImageSkew = 16;

}  // namespace tl
