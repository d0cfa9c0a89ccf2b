// Chunk-slot arithmetic of the split-KV kernels, shared by device code and by the host entry point
// that exposes it to the tests.  A launch is sized from shapes alone (no host read of the page
// table), so every kernel instance recomputes its place from page_indptr with these functions.
#ifndef TVMKV_CSRC_SPLIT_PLAN_H_
#define TVMKV_CSRC_SPLIT_PLAN_H_

#include <cstdint>

#if defined(__HIPCC__)
#define TVMKV_HD __host__ __device__ __forceinline__
#else
#define TVMKV_HD inline
#endif

namespace tvmkv {

// Decode: sequence b owns the chunk slots [slot_begin(b), slot_begin(b) + ceil(npages_b / cp)), which
// always fit in front of slot_begin(b + 1); the grid has floor(nnz_pages / cp) + batch slots.
TVMKV_HD int slot_begin(const int32_t* page_indptr, int b, int cp) { return page_indptr[b] / cp + b; }

// Largest b in [0, batch) with slot_begin(b) <= slot.
TVMKV_HD int find_sequence(const int32_t* page_indptr, int batch, int cp, int slot) {
  int lo = 0, hi = batch - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (slot_begin(page_indptr, mid, cp) <= slot) {
      lo = mid;
    } else {
      hi = mid - 1;
    }
  }
  return lo;
}

}  // namespace tvmkv

#endif  // TVMKV_CSRC_SPLIT_PLAN_H_
