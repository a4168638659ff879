// Where an element of the paged cache lies inside its (page, KV head) tile.
//
// A tile holds the keys, or the values, of `page_size` tokens of one KV head: page_size * head_size elements.
// Their order inside the tile is the order in which the MFMA attention kernel's lanes read them, so that every
// vector load of a wave covers whole contiguous kilobytes:
//
//   keys    element (token t, column d):  ((d / 16) * 2 + (d % 16) / 8) * page_size + t) * 8 + d % 8
//           -- for a block of 16 columns, the 16-byte pieces (8 columns) of all tokens lie side by side, first
//           those of the lower 8 columns, then those of the upper 8;
//   values  a page of 16 tokens: element (column d, token t), d in 32-column tiles of R = min(32, head - tile
//           start) columns:  tile * 512 + (((t % 8) / 4) * R + d % 32) * 8 + (t / 8) * 4 + t % 4
//           -- for each column the tokens {0..3, 8..11} form one 16-byte piece and {4..7, 12..15} the other,
//           which are the key slots one lane feeds to one MFMA;
//           a page of 32, 48, 64, ... tokens: its tokens in runs of 16, each run laid out as a page of 16 tokens,
//           one run after the other (16 * head elements each);
//           any other page size: d * page_size + t (column-major, only the general kernel reads it).
#pragma once
#include <stddef.h>

namespace atoma {

__host__ __device__ __forceinline__ size_t key_offset(int t, int d, int page_size) {
  return ((size_t)((d >> 4) * 2 + ((d >> 3) & 1)) * page_size + t) * 8 + (d & 7);
}

__host__ __device__ __forceinline__ size_t value_offset(int d, int t, int head_size, int page_size) {
  if (page_size & 15) return (size_t)d * page_size + t;
  const size_t run = (size_t)(t >> 4) * 16 * head_size;
  t &= 15;
  const int tile = d >> 5, c = d & 31;
  const int rows = head_size - tile * 32 < 32 ? head_size - tile * 32 : 32;
  return run + (size_t)tile * 512 + (size_t)(((t & 7) >> 2) * rows + c) * 8 + ((t >> 3) << 2) + (t & 3);
}

}  // namespace atoma
