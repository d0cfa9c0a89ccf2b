// Random operation sequences against the host bookkeeping of the paged KV cache
// (tvm_amd/csrc/kv_bookkeeping.cc, block_pool.h), built for the HOST with AddressSanitizer and
// UndefinedBehaviorSanitizer by tests/test_host_sanitizers.py.  The driver keeps a small model of what
// it has done (live sequences and their lengths) so that most operations are valid, lets the
// library's own checks reject the rest, and after every step checks what must hold whatever the
// history: page ids inside the pool, no page handed out twice, the step's arrays inside the buffer.
// usage: fuzz_bookkeeping <seed> <operations> <sliding 0|1>
#include <cstdio>
#include <cstdlib>
#include <map>
#include <random>
#include <set>
#include <vector>

#include "../../tvm_amd/csrc/kv_bookkeeping.h"

namespace tvmkv {
void SetLastError(const std::string&) {}
}  // namespace tvmkv

using tvmkv::AuxSpan;
using tvmkv::KVBookkeeper;
using tvmkv::KVConfig;

static void Fail(const char* what, long a = 0, long b = 0) {
  std::fprintf(stderr, "invariant broken: %s (%ld, %ld)\n", what, a, b);
  std::abort();
}

int main(int argc, char** argv) {
  const unsigned seed = argc > 1 ? static_cast<unsigned>(std::atoi(argv[1])) : 1;
  const int operations = argc > 2 ? std::atoi(argv[2]) : 2000;
  const bool sliding = argc > 3 && std::atoi(argv[3]) != 0;
  std::mt19937 rng(seed);
  auto pick = [&](int lo, int hi) { return static_cast<int>(lo + rng() % static_cast<unsigned>(hi - lo + 1)); };

  KVConfig cfg;
  cfg.page_size = 16;
  cfg.num_total_pages = 96;
  cfg.reserved_num_seqs = 12;
  cfg.prefill_chunk_size = 256;
  cfg.support_sliding_window = sliding;
  cfg.rope_inline = sliding;
  KVBookkeeper book(cfg);
  std::vector<int32_t> buffer(static_cast<size_t>(book.RequiredCapacity()) + 64, -7);
  const size_t guard = 64;
  book.SetStepBuffer(buffer.data(), static_cast<int64_t>(buffer.size() - guard));

  std::map<int64_t, int> length;  // live sequences
  std::set<int64_t> windowed;
  int64_t next_id = 0;
  long steps = 0, rejected = 0;
  for (int op = 0; op < operations; ++op) {
    const int kind = pick(0, 99);
    try {
      if (kind < 12 || length.empty()) {
        if (static_cast<int>(length.size()) < 12) {
          book.AddSequence(next_id);
          length[next_id++] = 0;
        }
      } else if (kind < 20) {
        auto it = std::next(length.begin(), pick(0, static_cast<int>(length.size()) - 1));
        book.RemoveSequence(it->first);
        windowed.erase(it->first);
        length.erase(it);
      } else if (kind < 32) {
        auto it = std::next(length.begin(), pick(0, static_cast<int>(length.size()) - 1));
        if (static_cast<int>(length.size()) < 12) {
          const int64_t pos = pick(0, 9) == 0 ? -1 : pick(0, it->second);
          book.ForkSequence(it->first, next_id, pos);
          length[next_id++] = pos < 0 ? it->second : static_cast<int>(pos);
        }
      } else if (kind < 42) {
        auto it = std::next(length.begin(), pick(0, static_cast<int>(length.size()) - 1));
        const int n = pick(0, it->second + 1);  // one too many now and then: must be rejected
        book.PopN(it->first, n);
        it->second -= n;
      } else if (kind < 46 && sliding) {
        auto it = std::next(length.begin(), pick(0, static_cast<int>(length.size()) - 1));
        const int window = pick(8, 48), sink = pick(0, 6);
        book.EnableSlidingWindowForSeq(it->first, window, sink);
        windowed.insert(it->first);
      } else if (kind < 48) {
        book.Clear();
        length.clear();
        windowed.clear();
      } else if (kind < 60 && !sliding) {
        // a speculative step: every chosen sequence appends a random token tree, then (mostly) commits a path
        std::vector<int64_t> ids, lens, parents, leaves;
        for (auto& kv : length) {
          if (pick(0, 1) == 0) continue;
          const int n = pick(1, 9);
          ids.push_back(kv.first);
          lens.push_back(n);
          for (int i = 0; i < n; ++i) parents.push_back(i == 0 ? -1 : pick(pick(0, 3) == 0 ? -1 : 0, i - 1));
          leaves.push_back(pick(-1, n - 1));
        }
        if (ids.empty()) continue;
        book.BeginForward(ids.data(), lens.data(), static_cast<int64_t>(ids.size()), parents.data(),
                          static_cast<int64_t>(parents.size()));
        ++steps;
        for (size_t i = 0; i < ids.size(); ++i) length[ids[i]] += static_cast<int>(lens[i]);
        const tvmkv::StepLayout& s = book.step();
        for (size_t g = buffer.size() - guard; g < buffer.size(); ++g) {
          if (buffer[g] != -7) Fail("write behind the step buffer", static_cast<long>(g));
        }
        for (int d = 0; d < s.num_depths; ++d) {
          const AuxSpan& mask = s.tree_attn_mask[d];
          if (mask.present() && mask.offset + mask.size > s.used) Fail("tree mask beyond the used part", d);
        }
        if (pick(0, 9) != 0) {
          // the accepted path: walk up from the leaf to learn its length
          size_t at = 0;
          std::vector<int> accepted(ids.size(), 0);
          for (size_t i = 0; i < ids.size(); ++i) {
            for (int64_t node = leaves[i]; node >= 0; node = parents[at + static_cast<size_t>(node)]) ++accepted[i];
            at += static_cast<size_t>(lens[i]);
          }
          book.CommitAcceptedTokenTreeNodes(ids.data(), leaves.data(), static_cast<int>(ids.size()));
          for (size_t i = 0; i < ids.size(); ++i) length[ids[i]] += accepted[i] - static_cast<int>(lens[i]);
          const std::vector<int32_t>& indptr = book.commit_copy_length_indptr();
          for (size_t i = 1; i < indptr.size(); ++i) {
            if (indptr[i] < indptr[i - 1]) Fail("commit copy indptr not monotone", static_cast<long>(i));
          }
          if (!indptr.empty() && static_cast<size_t>(indptr.back()) > book.commit_copy_src_pos().size()) Fail("commit copy list short");
        }
      } else {
        // a forward step over a random subset, decode-like or prefill-like
        std::vector<int64_t> ids, lens;
        const bool decode = pick(0, 2) == 0;
        int64_t total = 0;
        for (auto& kv : length) {
          if (pick(0, 2) == 0) continue;
          const int64_t n = decode ? 1 : pick(1, 40);
          ids.push_back(kv.first);
          lens.push_back(n);
          total += n;
        }
        if (ids.empty()) continue;
        book.BeginForward(ids.data(), lens.data(), static_cast<int64_t>(ids.size()), nullptr, 0);
        ++steps;
        for (size_t i = 0; i < ids.size(); ++i) length[ids[i]] += static_cast<int>(lens[i]);
        // the step's arrays lie inside the buffer, and the guard words behind it are untouched
        const tvmkv::StepLayout& s = book.step();
        if (s.used < 0 || s.used > static_cast<int64_t>(buffer.size() - guard)) Fail("step.used", s.used);
        for (size_t g = buffer.size() - guard; g < buffer.size(); ++g) {
          if (buffer[g] != -7) Fail("write behind the step buffer", static_cast<long>(g));
        }
        // append slots: inside the pool, all different
        const AuxSpan& ap = s.append_position_map;
        if (!ap.present() || ap.size != total) Fail("append_position_map size", ap.size, total);
        std::set<int32_t> slots;
        for (int64_t i = 0; i < ap.size; ++i) {
          const int32_t slot = buffer[ap.offset + i];
          if (slot == -1 && sliding) continue;  // a token that slides out of its window at once is not stored
          if (slot < 0 || slot >= cfg.num_total_pages * cfg.page_size) Fail("append slot", slot);
          if (!slots.insert(slot).second) Fail("append slot handed out twice", slot);
        }
        // page tables: ids inside the pool; indptr monotone and consistent with the values
        for (int d = 0; d < s.num_depths; ++d) {
          const AuxSpan& ip = s.page_indptr[d];
          const AuxSpan& pv = s.page_indices[d];
          if (!ip.present()) Fail("page_indptr missing", d);
          for (int64_t i = 1; i < ip.size; ++i) {
            if (buffer[ip.offset + i] < buffer[ip.offset + i - 1]) Fail("page_indptr not monotone", d, i);
          }
          if (ip.size > 0 && buffer[ip.offset + ip.size - 1] != pv.size) Fail("page_indptr end", d, pv.size);
          for (int64_t i = 0; i < pv.size; ++i) {
            const int32_t page = buffer[pv.offset + i];
            if (page < 0 || page >= cfg.num_total_pages) Fail("page id", page);
          }
        }
      }
    } catch (const tvmkv::Error&) {
      // a rejected operation; pool exhaustion in the middle of a step leaves the object unusable, as
      // in the reference: start over
      ++rejected;
      book.Clear();
      length.clear();
      windowed.clear();
    }
    // pages in use + free pages = the pool
    const std::vector<int64_t> state = book.DumpState();
    (void)state;
    if (book.NumAvailablePages() < 0 || book.NumAvailablePages() > cfg.num_total_pages) Fail("free pages", book.NumAvailablePages());
    if (length.empty() && !book.Empty() && rejected == 0) Fail("cache not empty without sequences");
  }
  std::printf("seed %u: %d operations, %ld steps, %ld rejected\n", seed, operations, steps, rejected);

  // A long-running cache: forks inside pages and removals, over and over, without a Clear().  The page-id
  // arena must settle (every slice a fork or a removal gives back can serve a later request) and so must
  // the copy log.
  book.Clear();
  book.AddSequence(0);
  {
    const int64_t ids[1] = {0}, lens[1] = {200};
    book.BeginForward(ids, lens, 1, nullptr, 0);
  }
  int64_t child = 1, arena_after_warmup = 0;
  for (int cycle = 0; cycle < 20000; ++cycle) {
    const int live = pick(1, 4);
    for (int j = 0; j < live; ++j) book.ForkSequence(0, child + j, pick(1, 200));
    for (int j = 0; j < live; ++j) {
      const int64_t ids[1] = {child + j}, lens[1] = {static_cast<int64_t>(pick(1, 40))};
      book.BeginForward(ids, lens, 1, nullptr, 0);
    }
    for (int j = 0; j < live; ++j) book.RemoveSequence(child + j);
    child += live;
    if (cycle == 2000) arena_after_warmup = book.PageArenaInUse();
    if (cycle > 2000 && book.PageArenaInUse() > 2 * arena_after_warmup + 1024) {
      Fail("page-id arena keeps growing", book.PageArenaInUse(), arena_after_warmup);
    }
    book.TrimCopyLog(book.CopyLog().size());
    if (book.CopyLog().size() > KVBookkeeper::kCopyLogCap) Fail("copy log keeps growing", static_cast<long>(book.CopyLog().size()));
  }
  std::printf("churn: arena %ld entries after 2000 cycles, %ld after 20000\n", static_cast<long>(arena_after_warmup),
              static_cast<long>(book.PageArenaInUse()));
  return 0;
}
