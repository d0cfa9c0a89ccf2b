// Host-side support shared by the kernel launchers: tuning options (read from the environment once,
// changeable through tvmkv_set_option) and the scratch buffers of the split-KV kernels.
#ifndef TVMKV_CSRC_RUNTIME_SUPPORT_H_
#define TVMKV_CSRC_RUNTIME_SUPPORT_H_

#include <hip/hip_runtime_api.h>

#include <cstddef>
#include <cstdint>
#include <mutex>

struct tvmkv_rope_scaling;  // include/tvmkv.h

namespace tvmkv {

enum Option {
  kOptDecodeChunkPages = 0,   // pages per split-KV chunk of the decode kernel, 0 = derived from the shapes
  kOptDecodeSeparateMerge,    // != 0: merge the chunks in a second launch instead of inside the kernel
  kOptDecodeWgsPerCu,         // > 0: cap the decode grid at this many workgroups per compute unit
  kOptMlaChunkTokens,         // lower bound of the tokens per split-KV chunk of the MLA kernel, 0 = 128
  kOptMlaSeparateMerge,       // unused (the MLA chunks are always merged in a second launch)
  kOptPrefillKvSplits,        // > 0: split the keys of every row tile of a paged prefill launch this many ways, 0 = derived
  kOptNoFusedDecodeStep,      // != 0: the cache object runs a decode step as split+RoPE+append and decode, two launches
  kNumOptions
};
int64_t option(Option id);

// Scratch memory of a split-KV launch.  A buffer belongs to one (device, stream, user): launches on
// one stream are ordered and may share it, launches on different streams (two caches, two layers in
// flight) never do.  The first `counter_bytes` bytes hold arrival counters that are not reset between
// launches: every launch gets a new `epoch`, a counter is a 64-bit word (epoch << 32 | arrivals), and a
// word left behind by an earlier launch -- also one that failed or was abandoned half way -- carries an
// older epoch and counts as zero.  The epoch is the low half of a 64-bit launch count; when it wraps
// (2^32 launches on one buffer) the counters are cleared by a kernel in stream order and the epochs
// start over at 1.
// The lease keeps the pool locked until it is destroyed: hold it until the launch that uses the buffer
// has been enqueued, so that a second host thread on the same stream cannot free the buffer in between.
struct ScratchLease {
  char* ptr;        // device memory, at least the requested size, 256-byte aligned
  uint32_t epoch;   // never 0
  std::unique_lock<std::mutex> lock;
};
enum ScratchUser { kScratchDecode = 0, kScratchMla = 1, kScratchPrefill = 2, kScratchGeneric = 3 };
ScratchLease lease_scratch(ScratchUser user, hipStream_t stream, size_t bytes, size_t counter_bytes);
// Frees the buffers of (current device, stream) after synchronising the stream; a buffer whose address
// a graph under capture has recorded is kept until the process ends instead.
void release_scratch(hipStream_t stream);
// The epoch of the next launch from a 64-bit launch count (host arithmetic only).
uint32_t next_scratch_epoch(uint64_t* launches, bool* wrapped);
void zero_scratch_counters(char* ptr, size_t counter_bytes, hipStream_t stream);
// Test aid: sets the launch count of every pooled buffer (to run a launch across the epoch wrap).
void debug_set_scratch_launches(uint64_t launches);

// The table of an attention kernel's in-kernel RoPE for a frequency variant (NULL: the default
// frequencies): entries for all head_dim elements, see InlineRopeTable in kernels_common.cuh.  Host
// arithmetic only (defined next to the split-rotary kernel's tables in kernels_page.hip).
struct InlineRopeHost {
  float v[256];
  int inverse;
  int halves_differ;
  float magnitude;
};
InlineRopeHost inline_rope_table(const ::tvmkv_rope_scaling* scaling, int head_dim, double rope_theta);

// Chunk-slot arithmetic of the decode split, on the host (the device functions of the same names in
// kernels_decode.hip compute the same values; the tests compare both against a direct enumeration).
int decode_pick_chunk_pages(int64_t nnz_pages, int h_kv, int batch, int head_dim = 128);
// the same for launches whose work items carry 32 query heads (GQA groups above 16)
int decode_pick_chunk_pages_wide(int64_t nnz_pages, int h_kv, int batch, int head_blocks, int resident_items);

}  // namespace tvmkv

#endif  // TVMKV_CSRC_RUNTIME_SUPPORT_H_
