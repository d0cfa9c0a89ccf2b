// Storage of the paged KV cache's host state: the stack of free pages, and the pool of blocks (the
// nodes of the prefix-sharing tree) as structure-of-arrays with every block's page ids in a slice
// of one flat arena.
//
// What the reference fixes is the ORDER in which pages and blocks are handed out and taken back
// (LIFO vectors, src/runtime/vm/paged_kv_cache.cc:1777-1798; page ids, append slots and the pool
// state are compared bit for bit) and the meaning of a block's fields
// (src/runtime/vm/attn_utils.h:101-152).  How they are stored is this library's own: a block's pages
// are a contiguous run of int32 in `arena_`, so flattening a step's page table is one memcpy per
// block, splitting off a shared prefix (fork) moves no data, and nothing is allocated per block.
#ifndef TVMKV_CSRC_BLOCK_POOL_H_
#define TVMKV_CSRC_BLOCK_POOL_H_

#include <cstdint>
#include <cstring>
#include <vector>

#include "common.h"

namespace tvmkv {

// Free pages: a stack that starts as [N-1, ..., 1, 0], so that pages come out as 0, 1, 2, ...
class PageStack {
 public:
  void Reset(int64_t num_pages) {
    ids_.resize(num_pages);
    for (int64_t i = 0; i < num_pages; ++i) ids_[i] = static_cast<int32_t>(num_pages - 1 - i);
  }
  bool Empty() const { return ids_.empty(); }
  int64_t Size() const { return static_cast<int64_t>(ids_.size()); }
  int32_t Pop() {
    KV_CHECK(!ids_.empty()) << "The KV cache is full. No page can be allocated.";
    const int32_t id = ids_.back();
    ids_.pop_back();
    return id;
  }
  void Push(int32_t id) { ids_.push_back(id); }
  const std::vector<int32_t>& Items() const { return ids_; }  // bottom first

 private:
  std::vector<int32_t> ids_;
};

class BlockPool {
 public:
  // scalar fields of block b (attn_utils.h:101-152)
  std::vector<int32_t> seq_length;     // tokens the block holds
  std::vector<int32_t> start_pos;      // position of its first token in the sequence
  std::vector<int32_t> sink_length;    // attention-sink tokens kept at its front (sliding window)
  std::vector<int32_t> window_offset;  // slot of the first window token inside its pages
  std::vector<int32_t> parent;         // -1 for a root
  std::vector<int32_t> refcount;       // sequences ending here + child blocks

  void Reset() {
    seq_length.clear();
    start_pos.clear();
    sink_length.clear();
    window_offset.clear();
    parent.clear();
    refcount.clear();
    slice_.clear();
    free_blocks_.clear();
    arena_.clear();
    bump_ = 0;
    for (auto& c : free_slices_) c.clear();
  }

  int32_t Size() const { return static_cast<int32_t>(slice_.size()); }
  int64_t NumFree() const { return static_cast<int64_t>(free_blocks_.size()); }
  const std::vector<int32_t>& FreeBlocks() const { return free_blocks_; }  // bottom first

  // A block with every field cleared: the most recently released one, else a new index.
  int32_t Acquire() {
    int32_t b;
    if (!free_blocks_.empty()) {
      b = free_blocks_.back();
      free_blocks_.pop_back();
    } else {
      b = Size();
      seq_length.push_back(0);
      start_pos.push_back(0);
      sink_length.push_back(0);
      window_offset.push_back(0);
      parent.push_back(-1);
      refcount.push_back(0);
      slice_.push_back(Slice{});
    }
    seq_length[b] = start_pos[b] = sink_length[b] = window_offset[b] = 0;
    parent[b] = -1;
    refcount[b] = 0;
    DropSlice(b);
    return b;
  }
  // The block's fields and page list stay readable until it is acquired again (state dumps show
  // released blocks as they were left); the caller has returned the pages it wants returned.
  void Release(int32_t b) { free_blocks_.push_back(b); }

  // ---- pages of a block -----------------------------------------------------------------------
  int32_t NumPages(int32_t b) const { return slice_[b].count; }
  const int32_t* Pages(int32_t b) const { return arena_.data() + slice_[b].offset; }
  int32_t Page(int32_t b, int32_t i) const { return arena_[slice_[b].offset + i]; }
  void SetPage(int32_t b, int32_t i, int32_t id) { arena_[slice_[b].offset + i] = id; }
  int32_t LastPage(int32_t b) const { return arena_[slice_[b].offset + slice_[b].count - 1]; }

  void PushPage(int32_t b, int32_t id) {
    Slice& s = slice_[b];
    if (s.count == s.capacity) Grow(b);
    arena_[slice_[b].offset + slice_[b].count++] = id;
  }
  int32_t PopPage(int32_t b) { return arena_[slice_[b].offset + --slice_[b].count]; }
  void ErasePage(int32_t b, int32_t i) {
    Slice& s = slice_[b];
    int32_t* base = arena_.data() + s.offset;
    std::memmove(base + i, base + i + 1, static_cast<size_t>(s.count - i - 1) * sizeof(int32_t));
    --s.count;
  }
  // The first n pages of `from` become the pages of `to` (which has none).  Where both parts keep at least
  // kMinSlice entries the slice is cut in two and no page id moves; otherwise a cut would leave a slice
  // that no later request can reuse (requests are for kMinSlice entries or more), so `to` gets a slice of
  // its own and the rest of `from` moves to the front of the old one.
  void SplitFront(int32_t from, int32_t n, int32_t to) {
    if (n >= kMinSlice && slice_[from].capacity - n >= kMinSlice) {
      Slice& f = slice_[from];
      slice_[to] = Slice{f.offset, n, n};
      f.offset += n;
      f.count -= n;
      f.capacity -= n;
      return;
    }
    int32_t want = kMinSlice;
    while (want < n) want *= 2;
    Slice fresh = Allocate(want);  // may move the arena: take addresses afterwards
    Slice& f = slice_[from];
    int32_t* base = arena_.data() + f.offset;
    std::memcpy(arena_.data() + fresh.offset, base, static_cast<size_t>(n) * sizeof(int32_t));
    std::memmove(base, base + n, static_cast<size_t>(f.count - n) * sizeof(int32_t));
    f.count -= n;
    fresh.count = n;
    slice_[to] = fresh;
  }
  // int32 entries of the arena handed out so far (free slices included): what a long-running cache holds
  int64_t ArenaInUse() const { return bump_; }

 private:
  struct Slice {
    int64_t offset = 0;
    int32_t count = 0;
    int32_t capacity = 0;
  };
  static int ClassOf(int32_t capacity) {  // floor(log2(capacity)), capacity >= 1
    int c = 0;
    while ((int64_t{2} << c) <= capacity) ++c;
    return c;
  }
  // Returns the block's slice to the free lists (a released block keeps it until then).
  void DropSlice(int32_t b) {
    Slice& s = slice_[b];
    if (s.capacity > 0) free_slices_[ClassOf(s.capacity)].push_back(Slice{s.offset, 0, s.capacity});
    s = Slice{};
  }
  Slice Allocate(int32_t capacity) {  // capacity is a power of two
    for (int c = ClassOf(capacity); c < kClasses; ++c) {
      if (!free_slices_[c].empty()) {
        Slice s = free_slices_[c].back();
        free_slices_[c].pop_back();
        return s;  // may be roomier than asked for
      }
    }
    if (bump_ + capacity > static_cast<int64_t>(arena_.size())) {
      arena_.resize(std::max<int64_t>(2 * static_cast<int64_t>(arena_.size()), bump_ + capacity + 1024));
    }
    Slice s{bump_, 0, capacity};
    bump_ += capacity;
    return s;
  }
  void Grow(int32_t b) {
    const Slice old = slice_[b];
    int32_t want = kMinSlice;
    while (want <= old.capacity) want *= 2;
    Slice fresh = Allocate(want);
    if (old.count > 0) {
      std::memcpy(arena_.data() + fresh.offset, arena_.data() + old.offset, static_cast<size_t>(old.count) * sizeof(int32_t));
    }
    fresh.count = old.count;
    if (old.capacity > 0) free_slices_[ClassOf(old.capacity)].push_back(Slice{old.offset, 0, old.capacity});
    slice_[b] = fresh;
  }

  static constexpr int kClasses = 32;
  static constexpr int32_t kMinSlice = 4;  // no slice is smaller: every free slice can serve some request
  std::vector<Slice> slice_;
  std::vector<int32_t> free_blocks_;
  std::vector<int32_t> arena_;
  int64_t bump_ = 0;
  std::vector<Slice> free_slices_[kClasses];
};

}  // namespace tvmkv

#endif  // TVMKV_CSRC_BLOCK_POOL_H_
