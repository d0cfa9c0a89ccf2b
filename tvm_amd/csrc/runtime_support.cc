// Tuning options and the scratch-buffer pool of the split-KV launchers (see runtime_support.h).
#include "runtime_support.h"

#include <hip/hip_runtime.h>

#include <algorithm>
#include <atomic>
#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>
#include <tuple>
#include <vector>

#include "common.h"

namespace tvmkv {

namespace {

struct OptionTable {
  std::atomic<int64_t> value[kNumOptions];
  OptionTable() {
    static const char* const env_names[] = {"TVMKV_DECODE_CHUNK_PAGES", "TVMKV_DECODE_SEPARATE_MERGE",
                                                       "TVMKV_DECODE_WGS_PER_CU", "TVMKV_MLA_CHUNK_TOKENS",
                                                       "TVMKV_MLA_SEPARATE_MERGE", "TVMKV_PREFILL_KV_SPLITS",
                                                       "TVMKV_NO_FUSED_DECODE_STEP"};
    static_assert(sizeof(env_names) / sizeof(env_names[0]) == kNumOptions, "one environment variable per option");
    for (int i = 0; i < kNumOptions; ++i) {
      const char* text = std::getenv(env_names[i]);  // once, when the library is loaded
      value[i].store(text != nullptr ? std::atoll(text) : 0, std::memory_order_relaxed);
    }
  }
};
OptionTable g_options;

const char* const kOptionNames[] = {"decode_chunk_pages", "decode_separate_merge", "decode_wgs_per_cu",
                                               "mla_chunk_tokens", "mla_separate_merge", "prefill_kv_splits",
                                               "no_fused_decode_step"};
static_assert(sizeof(kOptionNames) / sizeof(kOptionNames[0]) == kNumOptions, "one name per option");

struct Scratch {
  char* ptr = nullptr;
  size_t bytes = 0;
  size_t counter_bytes = 0;
  uint64_t launches = 0;       // launches served from this buffer; the epoch of a launch is its low half
  bool seen_in_capture = false;  // a graph under capture has recorded this buffer's address
};
std::mutex g_scratch_mutex;
std::map<std::tuple<int, hipStream_t, int>, Scratch> g_scratch;
// Buffers that a captured graph may still name after their entry has grown: kept until the process ends.
std::vector<char*> g_retired;

__global__ void zero_words_kernel(unsigned long long* words, size_t count) {
  for (size_t i = blockIdx.x * static_cast<size_t>(blockDim.x) + threadIdx.x; i < count;
       i += static_cast<size_t>(gridDim.x) * blockDim.x) {
    words[i] = 0ull;
  }
}

bool stream_is_capturing(hipStream_t stream) {
  hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
  if (stream != nullptr && hipStreamIsCapturing(stream, &capture) != hipSuccess) {
    (void)hipGetLastError();
    capture = hipStreamCaptureStatusNone;
  }
  return capture != hipStreamCaptureStatusNone;
}

}  // namespace

int64_t option(Option id) { return g_options.value[id].load(std::memory_order_relaxed); }

uint32_t next_scratch_epoch(uint64_t* launches, bool* wrapped) {
  ++*launches;
  *wrapped = false;
  if (static_cast<uint32_t>(*launches) == 0) {  // 2^32 launches: the epochs start over at 1
    ++*launches;
    *wrapped = true;
  }
  return static_cast<uint32_t>(*launches);
}

void zero_scratch_counters(char* ptr, size_t counter_bytes, hipStream_t stream) {
  if (counter_bytes == 0) return;
  const size_t words = counter_bytes / sizeof(unsigned long long);
  hipLaunchKernelGGL(zero_words_kernel, dim3(64), dim3(256), 0, stream, reinterpret_cast<unsigned long long*>(ptr), words);
  HIP_CHECK(hipGetLastError());
}

ScratchLease lease_scratch(ScratchUser user, hipStream_t stream, size_t bytes, size_t counter_bytes) {
  int dev = 0;
  HIP_CHECK(hipGetDevice(&dev));
  // held by the lease until the caller has enqueued its launch: a thread that grows (and frees) this
  // entry's buffer first synchronises the stream, and by then the launch is on it
  std::unique_lock<std::mutex> lock(g_scratch_mutex);
  Scratch& s = g_scratch[std::make_tuple(dev, stream, static_cast<int>(user))];
  const bool capturing = stream_is_capturing(stream);
  if (s.bytes < bytes || s.counter_bytes < counter_bytes) {
    // growing means hipMalloc and hipFree: neither belongs into a graph under capture
    KV_CHECK(!capturing)
        << "the stream is being captured into a graph and this call needs " << bytes << " bytes of scratch memory that "
        << "are not allocated yet: run the same call once on this stream before the capture starts, or use "
        << "tvmkv_batch_decode_paged_kv_noalloc";
    if (s.ptr != nullptr) {
      if (s.seen_in_capture) {
        // a captured graph holds this address in its kernel arguments and may be replayed at any time
        g_retired.push_back(s.ptr);
      } else {
        // launches still queued on this stream read the old buffer; nobody else ever does
        HIP_CHECK(hipStreamSynchronize(stream));
        HIP_CHECK(hipFree(s.ptr));
      }
      s = Scratch{};
    }
    const size_t want = bytes + bytes / 2;
    void* ptr = nullptr;
    HIP_CHECK(hipMalloc(&ptr, want));
    s.ptr = static_cast<char*>(ptr);
    s.bytes = want;
    s.counter_bytes = counter_bytes;
    s.launches = 0;
    zero_scratch_counters(s.ptr, counter_bytes, stream);  // a kernel, not a memset node
  }
  s.seen_in_capture = s.seen_in_capture || capturing;
  bool wrapped = false;
  const uint32_t epoch = next_scratch_epoch(&s.launches, &wrapped);
  // Every launch leaves its counters at (epoch, 0), and the kernels bring a word of an older epoch up to
  // their own with a maximum: after the wrap an abandoned launch's word would compare as newer, so the
  // counters start over from zero (a kernel in stream order; recorded into a graph it is harmless).
  if (wrapped) zero_scratch_counters(s.ptr, s.counter_bytes, stream);
  return ScratchLease{s.ptr, epoch, std::move(lock)};
}

void release_scratch(hipStream_t stream) {
  int dev = 0;
  HIP_CHECK(hipGetDevice(&dev));
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  KV_CHECK(!stream_is_capturing(stream)) << "tvmkv_release_scratch: the stream is being captured";
  bool synced = false;
  for (auto it = g_scratch.begin(); it != g_scratch.end();) {
    if (std::get<0>(it->first) != dev || std::get<1>(it->first) != stream) {
      ++it;
      continue;
    }
    if (it->second.ptr != nullptr) {
      if (it->second.seen_in_capture) {
        g_retired.push_back(it->second.ptr);
      } else {
        if (!synced) HIP_CHECK(hipStreamSynchronize(stream));
        synced = true;
        HIP_CHECK(hipFree(it->second.ptr));
      }
    }
    it = g_scratch.erase(it);
  }
}

void debug_set_scratch_launches(uint64_t launches) {
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  for (auto& entry : g_scratch) entry.second.launches = launches;
}

// Work items of a decode launch: every item pays ~2 us of fixed cost (locating its sequence, q, the
// cross-wave merge) and every chunk of a sequence is one more partial state for the merge, whose loads
// are round trips to memory.  Large launches (cfg 2: 147 k pages x kv heads) run best with ~2300 items =
// three rounds of 3 workgroups x 256 CUs; small ones with fewer and longer items (one sequence of 131 072
// tokens: 0.110 ms with 32-page chunks, 0.085 with 128; 64 sequences with one kv head: 0.140 ms with
// 8-page chunks, 0.073 with 64).  One step of the matrix-core decode kernel is 2 pages per wave, 8 per
// workgroup; chunks are multiples of 8 pages up to 128.  Two cases take longer chunks than that:
//  * more than 16 chunks per sequence while at least 768 items remain: the states of a sequence are
//    merged by one workgroup, a serial tail (8 sequences of 16-65 k tokens: 0.245 ms with 64 pages,
//    0.236 with 128);
//  * sequences that fit one 128-page chunk on average, enough of them to fill the chip without a split:
//    no partial states at all (256 sequences of 512-2048 tokens: 0.220 ms with 64 pages, 0.210 with 128).
// Chunks of 32, 64, 96 or 128 pages put the chunks of a sequence whose pages have consecutive ids -- a cache that
// was filled sequence by sequence hands them out that way -- at a distance in memory at which the workgroups of
// the sequence, which walk their chunks in step, keep meeting in the same memory channels.  Seen at head dim 128
// with 8 and 16 kv heads (pages of 64 and 128 KiB), not with 4 or fewer, and not at head dims 64 and 256.  Measured, 8 kv heads, us with permuted / consecutive
// page ids (chunk pages -> time):
//   64 x U[1024,8192] (cfg 2)      48: 195.8 / 196.3   56: 194.5 / 196.5   64: 197.8 / 205.1   80: 195.0 / 197.3
//   8 x U[32768,131072], 64 q      112: 435.1 / 438.8  120: 439.5 / 440.5  128: 436.8 / 478.9  64: 453.3 / 527.3
//   16 x U[8192,32768]             112: 200.9 / 202.6  64: 206.6 / 231.4   128: 206.6 / 221.6
//   4 x 32768                      88: 90.2 / 92.1     96: 92.5 / 101.3    104: 91.9 / 93.4
//   64 x U[1024,8192], 16 kv heads 56: 389.9 / 387.3   32: 390.7 / 425.5   64: 390.2 / 406.0
//   64 x U[1024,8192], 4 kv heads  56: 126.0 / 123.2   64: 120.5 / 118.2
//   head dim 256, 8 kv heads        48: 437 / 429       64: 421 / 417       80: 417 / 411       (no camping: the rule is left alone)
//   head dim 64, 8 kv heads         48: 115 / 111       64: 116 / 112       96: 112 / 110       (flat)
static bool camps(int chunk_pages, int h_kv, int head_dim) { return h_kv >= 8 && head_dim == 128 && chunk_pages % 32 == 0; }

int decode_pick_chunk_pages(int64_t nnz_pages, int h_kv, int batch, int head_dim) {
  const int64_t forced = option(kOptDecodeChunkPages);
  if (forced >= 8 && forced % 8 == 0) return static_cast<int>(forced);
  const int64_t work = nnz_pages * h_kv;
  const int64_t per_sequence = nnz_pages / std::max(batch, 1);
  if (work <= 65536) {
    // Small launches (up to 1 M cached tokens x kv heads): the shortest chunk, a multiple of 8 pages from 24 on,
    // whose grid fits the 3 workgroups x 256 compute units the chip holds at once -- every workgroup starts
    // at once and none runs alone at the end; one or two very long sequences take 128-page chunks instead when
    // that still leaves 384 items (more than 32 states per sequence cost more than the items lost).  Measured
    // (us, chunk pages -> time, * = this rule; the rule before in brackets):
    //   16 x U[100,4000] tokens, 8 kv heads   16: 29.8  24*: 26.1  32: 28.3  64: 32.1            [16]
    //   8 x U[2000,6000]                      16: 32.7  24*: 27.4  32: 30.3  64: 32.8            [16]
    //   4 x 32768                             64: 92.4  88: 87.5   96*: 88.7  128: 99.9          [64]
    //   64 x U[1024,8192], 16 q / 1 kv head   16: 49.7  24: 44.9   32*: 41.4  40: 37.6  64: 41.6 [16]
    //   64 x U[64,512]                        16: 23.4  32: 20.0   40*: 20.9  128: 19.4          [16]
    //   32 x U[100,2000]                      16: 34.6  32: 32.5   40*: 34.2  64: 36.2           [32]
    //   1 x 131072                            64: 102.3 120: 100.8 128*: 88.1                    [128]
    int cp = 128;
    for (int c = 24; c <= 128; c += 8) {
      if (camps(c, h_kv, head_dim)) continue;
      if ((nnz_pages / c + batch) * h_kv <= 768) {
        cp = c;
        break;
      }
    }
    if (per_sequence / cp > 32 && (nnz_pages / 128 + batch) * h_kv >= 384) cp = 128;
    return cp;
  }
  const int64_t items = std::min<int64_t>(std::max<int64_t>(work / 64, 768), 2304);
  const int64_t cp = work / items;
  int pow2 = 16;
  while (pow2 < 128 && pow2 * 3 / 2 <= cp) pow2 *= 2;  // nearest power of two
  const int64_t per_seq = nnz_pages / std::max(batch, 1);
  while (pow2 < 128 && per_seq / pow2 > 16 && work / (pow2 * 2) >= 768) pow2 *= 2;
  // one or two very long sequences: more than 32 states per sequence cost more than the items that the
  // longer chunk takes away (one sequence of 131 072 tokens, 8 kv heads: 0.103 ms with 64 pages, 0.089 with
  // 128; two of 65 536: 0.096 / 0.086; four of 32 768, 32 states each at 64 pages: 0.092 / 0.101)
  while (pow2 < 128 && per_seq / pow2 > 32 && work / (pow2 * 2) >= 384) pow2 *= 2;
  if (per_seq <= 96 && static_cast<int64_t>(batch) * h_kv >= 1536) return 128;
  // the neighbours of the powers of two that do not camp (see camps()); one or two sequences keep 128 pages
  // (64 states of a 131 072-token sequence merge in two rounds of 32)
  if (camps(pow2, h_kv, head_dim) && pow2 == 64) return 48;
  if (camps(pow2, h_kv, head_dim) && pow2 == 128 && batch > 2) return 112;
  return pow2;
}

// Work items of 32 query heads (GQA groups above 16): an item does twice the matrix and softmax work per
// K/V byte, two workgroups fit a compute unit, and every chunk of a sequence is a partial state of 32 (or
// 64, 128 ...) heads to merge (in a second kernel).  What decides such a launch is how its workgroups fill
// the chip: the shortest chunk (a multiple of 8 pages from 16 to 128) whose grid -- chunk slots x kv heads x
// head blocks -- still fits the workgroups the chip holds at once (resident_items = 2 per compute unit), or
// twice, three times that when no chunk size fits.  A grid just above a whole number of rounds runs its last
// workgroups alone; one well below leaves compute units with one workgroup where two would run.  Measured
// (us; 64 sequences of 1024-8192 tokens, 18 018 pages, unless noted; chunk pages -> time, * = this rule):
//   32 q / 1 kv   40: 54.2   48*: 42.4   56: 44.9   64: 47.9   96: 51.9   128: 60.7
//   64 / 1        48: 66.0   64: 72.5    80: 73.6   96*: 58.4  112: 60.4  128: 63.1
//   64 / 2        48: 79.8   64: 86.1    80: 86.3   96*: 70.3  112: 74.3  128: 80.3
//   128 / 4       40: 138.0  56: 136.1   64: 137.8  96*: 135.8 128: 148.2
//   8 sequences of 32k-128k tokens, 64 / 2     64: 180.5   96: 182.7   112*: 160.8   128: 166.9
//   16 sequences, 32 / 1                       16*: 23.1   24: 22.7    32: 24.2      64: 35.0
//   256 sequences of 512-2048 tokens, 32 / 1   64: 56.6    80: 58.8    88*           96: 63.3   (32, the rule before: 63.0)
int decode_pick_chunk_pages_wide(int64_t nnz_pages, int h_kv, int batch, int head_blocks, int resident_items) {
  const int64_t forced = option(kOptDecodeChunkPages);
  if (forced >= 8 && forced % 8 == 0) return static_cast<int>(forced);
  const int64_t per_slot = static_cast<int64_t>(h_kv) * head_blocks;
  const int64_t capacity = std::max(resident_items, 1);
  for (int rounds = 1; rounds <= 4; ++rounds) {
    for (int cp = 16; cp <= 128; cp += 8) {
      if ((nnz_pages / cp + batch) * per_slot <= capacity * rounds) return cp;
    }
  }
  return 128;
}

}  // namespace tvmkv

extern "C" {

int tvmkv_set_option(const char* name, int64_t value) {
  KV_API_BEGIN();
  KV_CHECK(name != nullptr) << "tvmkv_set_option: name is NULL";
  for (int i = 0; i < tvmkv::kNumOptions; ++i) {
    if (std::strcmp(name, tvmkv::kOptionNames[i]) == 0) {
      tvmkv::g_options.value[i].store(value, std::memory_order_relaxed);
      return TVMKV_OK;
    }
  }
  KV_CHECK(false) << "tvmkv_set_option: unknown option \"" << name << "\"";
  KV_API_END();
}

uint32_t tvmkv_debug_next_scratch_epoch(uint64_t* launches, int32_t* wrapped) {
  bool w = false;
  const uint32_t epoch = tvmkv::next_scratch_epoch(launches, &w);
  *wrapped = w ? 1 : 0;
  return epoch;
}

int tvmkv_release_scratch(void* stream) {
  KV_API_BEGIN();
  tvmkv::release_scratch(static_cast<hipStream_t>(stream));
  KV_API_END();
}

int tvmkv_get_option(const char* name, int64_t* value) {
  KV_API_BEGIN();
  KV_CHECK(name != nullptr && value != nullptr) << "tvmkv_get_option: NULL argument";
  for (int i = 0; i < tvmkv::kNumOptions; ++i) {
    if (std::strcmp(name, tvmkv::kOptionNames[i]) == 0) {
      *value = tvmkv::option(static_cast<tvmkv::Option>(i));
      return TVMKV_OK;
    }
  }
  KV_CHECK(false) << "tvmkv_get_option: unknown option \"" << name << "\"";
  KV_API_END();
}

}  // extern "C"
