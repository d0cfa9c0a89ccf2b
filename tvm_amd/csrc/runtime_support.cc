// Tuning options and the scratch-buffer pool of the split-KV launchers (see runtime_support.h).
#include "runtime_support.h"

#include <algorithm>
#include <atomic>
#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>
#include <tuple>

#include "common.h"

namespace tvmkv {

namespace {

struct OptionTable {
  std::atomic<int64_t> value[kNumOptions];
  OptionTable() {
    static const char* const env_names[] = {"TVMKV_DECODE_CHUNK_PAGES", "TVMKV_DECODE_SEPARATE_MERGE",
                                                       "TVMKV_DECODE_WGS_PER_CU", "TVMKV_MLA_CHUNK_TOKENS",
                                                       "TVMKV_MLA_SEPARATE_MERGE", "TVMKV_PREFILL_KV_SPLITS"};
    static_assert(sizeof(env_names) / sizeof(env_names[0]) == kNumOptions, "one environment variable per option");
    for (int i = 0; i < kNumOptions; ++i) {
      const char* text = std::getenv(env_names[i]);  // once, when the library is loaded
      value[i].store(text != nullptr ? std::atoll(text) : 0, std::memory_order_relaxed);
    }
  }
};
OptionTable g_options;

const char* const kOptionNames[] = {"decode_chunk_pages", "decode_separate_merge", "decode_wgs_per_cu",
                                               "mla_chunk_tokens", "mla_separate_merge", "prefill_kv_splits"};
static_assert(sizeof(kOptionNames) / sizeof(kOptionNames[0]) == kNumOptions, "one name per option");

struct Scratch {
  char* ptr = nullptr;
  size_t bytes = 0;
  size_t counter_bytes = 0;
  uint32_t epoch = 0;
};
std::mutex g_scratch_mutex;
std::map<std::tuple<int, hipStream_t, int>, Scratch> g_scratch;

}  // namespace

int64_t option(Option id) { return g_options.value[id].load(std::memory_order_relaxed); }

ScratchLease lease_scratch(ScratchUser user, hipStream_t stream, size_t bytes, size_t counter_bytes) {
  int dev = 0;
  HIP_CHECK(hipGetDevice(&dev));
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  Scratch& s = g_scratch[std::make_tuple(dev, stream, static_cast<int>(user))];
  if (s.bytes < bytes || s.counter_bytes < counter_bytes) {
    // growing means hipMalloc, hipFree and a memset: none of them belongs into a graph under capture
    hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
    if (stream != nullptr && hipStreamIsCapturing(stream, &capture) != hipSuccess) {
      (void)hipGetLastError();
      capture = hipStreamCaptureStatusNone;
    }
    KV_CHECK(capture == hipStreamCaptureStatusNone)
        << "the stream is being captured into a graph and this call needs " << bytes << " bytes of scratch memory that "
        << "are not allocated yet: run the same call once on this stream before the capture starts, or use "
        << "tvmkv_batch_decode_paged_kv_noalloc";
    if (s.ptr != nullptr) {
      // launches still queued on this stream read the old buffer; nobody else ever does
      HIP_CHECK(hipStreamSynchronize(stream));
      HIP_CHECK(hipFree(s.ptr));
      s = Scratch{};
    }
    const size_t want = bytes + bytes / 2;
    void* ptr = nullptr;
    HIP_CHECK(hipMalloc(&ptr, want));
    s.ptr = static_cast<char*>(ptr);
    s.bytes = want;
    s.counter_bytes = counter_bytes;
    s.epoch = 0;
    HIP_CHECK(hipMemsetAsync(s.ptr, 0, counter_bytes, stream));
  }
  if (++s.epoch == 0) {
    // 2^32 launches on this buffer: start the epochs over from clean counters
    HIP_CHECK(hipMemsetAsync(s.ptr, 0, s.counter_bytes, stream));
    s.epoch = 1;
  }
  return ScratchLease{s.ptr, s.epoch};
}

// Work items of a decode launch: every item pays ~2 us of fixed cost (locating its sequence, q, the
// cross-wave merge) and every chunk of a sequence is one more partial state for the merge, whose loads
// are round trips to memory.  Large launches (cfg 2: 147 k pages x kv heads) run best with ~2300 items =
// three rounds of 3 workgroups x 256 CUs; small ones with fewer and longer items (one sequence of 131 072
// tokens: 0.110 ms with 32-page chunks, 0.085 with 128; 64 sequences with one kv head: 0.140 ms with
// 8-page chunks, 0.073 with 64).  One step of the matrix-core decode kernel is 2 pages per wave, 8 per
// workgroup; chunks are powers of two from 16 to 128 pages.  Two cases take longer chunks than that:
//  * more than 16 chunks per sequence while at least 768 items remain: the states of a sequence are
//    merged by one workgroup, a serial tail (8 sequences of 16-65 k tokens: 0.245 ms with 64 pages,
//    0.236 with 128);
//  * sequences that fit one 128-page chunk on average, enough of them to fill the chip without a split:
//    no partial states at all (256 sequences of 512-2048 tokens: 0.220 ms with 64 pages, 0.210 with 128).
int decode_pick_chunk_pages(int64_t nnz_pages, int h_kv, int batch) {
  const int64_t forced = option(kOptDecodeChunkPages);
  if (forced >= 8 && forced % 8 == 0) return static_cast<int>(forced);
  const int64_t work = nnz_pages * h_kv;
  const int64_t items = std::min<int64_t>(std::max<int64_t>(work / 64, 768), 2304);
  const int64_t cp = work / items;
  int pow2 = 16;
  while (pow2 < 128 && pow2 * 3 / 2 <= cp) pow2 *= 2;  // nearest power of two
  const int64_t per_seq = nnz_pages / std::max(batch, 1);
  while (pow2 < 128 && per_seq / pow2 > 16 && work / (pow2 * 2) >= 768) pow2 *= 2;
  if (per_seq <= 96 && static_cast<int64_t>(batch) * h_kv >= 1536) pow2 = 128;
  return pow2;
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
