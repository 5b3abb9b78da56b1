// Shared by the quantize / dequantize kernels of every model dtype: thread -> (row, word) mapping.
#pragma once
#include "gq_common.hpp"
#include "gq_internal.hpp"

namespace gq {

// Which (row, storage word) a thread owns: thread n of the grid owns word n of the row-major
// [rows, nw] array.  n / nw by a per-thread 64-bit division costs more instructions than the rest
// of a dequantize, so the quotient comes from a multiply-high with a constant made on the host
// (round-up method with one extra bit: q = (((n - h) >> 1) + h) >> shift, h = mulhi(n, magic),
// exact for every 32-bit n); arrays of 2^32 words or more keep the plain division.
struct WordGrid {
  uint32_t nw, magic, shift;
  uint32_t mode;  // 0: multiply-high, 1: nw is a power of two (shift only), 2: 64-bit division
};
__device__ __forceinline__ void locate_word(const WordGrid gr, int64_t nw, int64_t& row, int64_t& wd) {
  if (gr.mode == 2) {
    const int64_t idx = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    row = idx / nw;
    wd = idx - row * nw;
    return;
  }
  const uint32_t n = blockIdx.x * 256u + threadIdx.x;
  uint32_t q;
  if (gr.mode == 1) {
    q = n >> gr.shift;
  } else {
    const uint32_t h = __umulhi(n, gr.magic);
    q = (((n - h) >> 1) + h) >> gr.shift;
  }
  row = q;
  wd = n - q * gr.nw;
}
static inline WordGrid plan_words(int64_t rows, int64_t nw, unsigned& blocks) {
  WordGrid gr{static_cast<uint32_t>(nw), 0u, 0u, 0u};
  const int64_t total = rows * nw;
  const int64_t b = (total + 255) / 256;
  blocks = b < (int64_t(1) << 31) ? static_cast<unsigned>(b) : 0u;  // 0: more blocks than a grid holds
  if (total + 256 >= (int64_t(1) << 32)) {
    gr.mode = 2;
    return gr;
  }
  uint32_t log2 = 0;
  while ((int64_t(2) << log2) <= nw) ++log2;  // floor(log2(nw))
  gr.shift = log2;
  if ((nw & (nw - 1)) == 0) {
    gr.mode = 1;
    return gr;
  }
  const uint64_t num = uint64_t(1) << (32 + log2);
  uint64_t m = num / static_cast<uint64_t>(nw);
  const uint64_t rem = num % static_cast<uint64_t>(nw);
  m = 2 * m + (2 * rem >= static_cast<uint64_t>(nw) ? 1 : 0) + 1;
  gr.magic = static_cast<uint32_t>(m);  // the 33rd bit is the "+ n" of the formula
  return gr;
}

}  // namespace gq
