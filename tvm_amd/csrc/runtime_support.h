// Host-side support shared by the kernel launchers: tuning options (read from the environment once,
// changeable through tvmkv_set_option) and the scratch buffers of the split-KV kernels.
#ifndef TVMKV_CSRC_RUNTIME_SUPPORT_H_
#define TVMKV_CSRC_RUNTIME_SUPPORT_H_

#include <hip/hip_runtime_api.h>

#include <cstddef>
#include <cstdint>

namespace tvmkv {

enum Option {
  kOptDecodeChunkPages = 0,   // pages per split-KV chunk of the decode kernel, 0 = derived from the shapes
  kOptDecodeSeparateMerge,    // != 0: merge the chunks in a second launch instead of inside the kernel
  kOptDecodeWgsPerCu,         // > 0: cap the decode grid at this many workgroups per compute unit
  kOptMlaChunkTokens,         // lower bound of the tokens per split-KV chunk of the MLA kernel, 0 = 128
  kOptMlaSeparateMerge,       // unused (the MLA chunks are always merged in a second launch)
  kOptPrefillKvSplits,        // > 0: split the keys of every row tile of a paged prefill launch this many ways, 0 = derived
  kNumOptions
};
int64_t option(Option id);

// Scratch memory of a split-KV launch.  A buffer belongs to one (device, stream, user): launches on
// one stream are ordered and may share it, launches on different streams (two caches, two layers in
// flight) never do.  The first `counter_bytes` bytes hold arrival counters that are never reset:
// every launch gets a new `epoch`, a counter is a 64-bit word (epoch << 32 | arrivals), and a word
// left behind by an earlier launch -- also one that failed or was abandoned half way -- carries an
// older epoch and counts as zero.
struct ScratchLease {
  char* ptr;        // device memory, at least the requested size, 256-byte aligned
  uint32_t epoch;   // never 0
};
enum ScratchUser { kScratchDecode = 0, kScratchMla = 1, kScratchPrefill = 2 };
ScratchLease lease_scratch(ScratchUser user, hipStream_t stream, size_t bytes, size_t counter_bytes);

// Chunk-slot arithmetic of the decode split, on the host (the device functions of the same names in
// kernels_decode.hip compute the same values; the tests compare both against a direct enumeration).
int decode_pick_chunk_pages(int64_t nnz_pages, int h_kv, int batch);

}  // namespace tvmkv

#endif  // TVMKV_CSRC_RUNTIME_SUPPORT_H_
