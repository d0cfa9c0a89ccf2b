// Host bookkeeping of the paged KV cache (see kv_bookkeeping.h).
#include "kv_bookkeeping.h"

#include <algorithm>
#include <cstring>
#include <map>

namespace tvmkv {

namespace {
inline int64_t AlignUp4(int64_t n) { return (n + 3) / 4 * 4; }  // arrays start on 16 bytes (attn_utils.h:1048-1052)
}  // namespace

KVBookkeeper::KVBookkeeper(const KVConfig& config) : cfg_(config) {
  KV_CHECK(cfg_.page_size > 0) << "page_size must be positive";
  Clear();
}

int64_t KVBookkeeper::RequiredCapacity() const {
  const int64_t r = cfg_.reserved_num_seqs, p = cfg_.num_total_pages, c = cfg_.prefill_chunk_size;
  // per depth: two page tables (the second is the layer-window view), five indptr-sized and six
  // batch-sized arrays, the token-tree labels; then the arrays that exist once
  return kMaxBlockDepth * (2 * p + 5 * (r + 1) + 6 * r + 2 * kTreeAttnMaxTreeSize * r + 16 * 4) + 2 * c + 2 * (r + 1) +
         8 * 4;
}

// ------------------------------------------------------------------------------------ sequences
int32_t KVBookkeeper::FindSeq(int64_t seq_id) const {
  auto it = seq_index_.find(seq_id);
  return it == seq_index_.end() ? -1 : it->second;
}

int32_t KVBookkeeper::RequireSeq(int64_t seq_id) const {
  const int32_t index = FindSeq(seq_id);
  KV_CHECK(index >= 0) << "The sequence \"" << seq_id << "\" cannot be found in KV cache.";
  return index;
}

// A sequence that ends at `last_block`: one more reference to that block, and its length is the sum
// of the blocks on the way up (attn_utils.h:180-199).
int32_t KVBookkeeper::NewSeq(int64_t seq_id, int32_t last_block) {
  int32_t index;
  if (!free_seq_slots_.empty()) {
    index = free_seq_slots_.back();
    free_seq_slots_.pop_back();
    seqs_[index] = SeqRecord{};
  } else {
    index = static_cast<int32_t>(seqs_.size());
    seqs_.emplace_back();
  }
  SeqRecord& seq = seqs_[index];
  seq.id = seq_id;
  seq.last_block = last_block;
  ++blocks_.refcount[last_block];
  for (int32_t b = last_block; b != -1; b = blocks_.parent[b]) seq.length += blocks_.seq_length[b];
  seq_index_.emplace(seq_id, index);
  return index;
}

void KVBookkeeper::DropSeq(int32_t index) {
  seq_index_.erase(seqs_[index].id);
  seqs_[index] = SeqRecord{};
  free_seq_slots_.push_back(index);
}

// ------------------------------------------------------------------------------------ verbs
// paged_kv_cache.cc:561-570
void KVBookkeeper::RequireUsable() const {
  KV_CHECK(!poisoned_) << "an earlier begin_forward failed after it had started to change the cache; the state of the "
                       << "page pool is undefined: call clear before using the cache again";
}

void KVBookkeeper::Clear() {
  poisoned_ = false;
  seqs_.clear();
  free_seq_slots_.clear();
  seq_index_.clear();
  pages_.Reset(cfg_.num_total_pages);
  blocks_.Reset();
  copy_log_.clear();
  began_forward_ = false;
  step_ = StepLayout{};
}

// :574-580
void KVBookkeeper::AddSequence(int64_t seq_id) {
  RequireUsable();
  KV_CHECK(FindSeq(seq_id) < 0) << "The sequence \"" << seq_id << "\" is already in the KV cache.";
  NewSeq(seq_id, blocks_.Acquire());
}

// :582-604: blocks that only this sequence holds give their pages back, leaf first
void KVBookkeeper::RemoveSequence(int64_t seq_id) {
  RequireUsable();
  const int32_t index = RequireSeq(seq_id);
  int32_t b = seqs_[index].last_block;
  KV_CHECK(blocks_.refcount[b] >= 1) << "block reference count underflow";
  for (; b != -1 && blocks_.refcount[b] == 1; b = blocks_.parent[b]) {
    const int32_t* ids = blocks_.Pages(b);
    for (int32_t i = 0, n = blocks_.NumPages(b); i < n; ++i) pages_.Push(ids[i]);
    blocks_.Release(b);
  }
  if (b != -1) {
    KV_CHECK(blocks_.refcount[b] > 1) << "block reference count underflow";
    --blocks_.refcount[b];
  }
  DropSeq(index);
}

// :606-719.  The child shares every block in front of the fork point.  A fork point inside a block cuts
// that block at the page boundary below it (the front part becomes a block both share); a fork
// point inside a page gives the child a page of its own whose first tokens are copied over.
void KVBookkeeper::ForkSequence(int64_t parent_seq_id, int64_t child_seq_id, int64_t fork_pos) {
  RequireUsable();
  const int32_t pi = FindSeq(parent_seq_id);
  KV_CHECK(pi >= 0) << "The parent sequence \"" << parent_seq_id << "\" cannot be found in KV cache.";
  KV_CHECK(FindSeq(child_seq_id) < 0) << "The child sequence \"" << child_seq_id << "\" is already in the KV cache.";
  KV_CHECK(fork_pos >= -1) << "The forked position should be non-negative, or -1 for last position as default.";
  KV_CHECK(fork_pos <= seqs_[pi].length) << "The forked position should not exceed the total length of parent sequence.";
  KV_CHECK(seqs_[pi].committed) << "The parent sequence's token tree computed in the last round of forward has not been "
                                   "committed with accepted nodes.";
  const int64_t ps = cfg_.page_size;
  if (fork_pos == -1) fork_pos = seqs_[pi].length;
  if (seqs_[pi].window != -1) {
    const SeqRecord& seq = seqs_[pi];
    const int32_t sink_size = seq.length - blocks_.seq_length[seq.last_block] + seq.last_block_sink;
    KV_CHECK(fork_pos <= sink_size) << "The parent sequence \"" << parent_seq_id
                                    << "\" is enabled with sliding window and thus only can be forked within sink size = "
                                    << sink_size << ". But the forked position = " << fork_pos << ".";
  }
  if (fork_pos == seqs_[pi].length && fork_pos % ps == 0 && blocks_.seq_length[seqs_[pi].last_block] > 0) {
    // a fork at a page-aligned end: the parent continues in an empty block of its own
    const int32_t tail = blocks_.Acquire();
    blocks_.start_pos[tail] = seqs_[pi].length;
    blocks_.parent[tail] = seqs_[pi].last_block;
    blocks_.refcount[tail] = 1;
    seqs_[pi].last_block = tail;
  }
  const int32_t child = blocks_.Acquire();

  // the parent's blocks, root first
  trace_.clear();
  for (int32_t b = seqs_[pi].last_block; b != -1; b = blocks_.parent[b]) trace_.push_back(b);
  int64_t offset = fork_pos;  // of the fork point inside the block under the cursor
  for (int64_t k = static_cast<int64_t>(trace_.size()) - 1; k >= 0; --k) {
    const int32_t b = trace_[k];
    if (k != 0) {  // not the parent's last block
      KV_CHECK(blocks_.seq_length[b] > 0) << "interior block is empty";
      KV_CHECK(blocks_.seq_length[b] % ps == 0) << "interior block is not page aligned";
      if (blocks_.seq_length[b] <= offset) {
        offset -= blocks_.seq_length[b];
        continue;
      }
    }
    const int32_t in_page = static_cast<int32_t>(offset % ps);
    const int32_t moved = static_cast<int32_t>(offset - in_page);
    const int32_t moved_pages = static_cast<int32_t>(moved / ps);
    if (moved_pages == 0) {
      const int32_t up = blocks_.parent[b];
      if (up != -1) ++blocks_.refcount[up];
      blocks_.parent[child] = up;
    } else {
      const int32_t shared = blocks_.Acquire();
      blocks_.parent[shared] = blocks_.parent[b];
      blocks_.parent[b] = shared;
      blocks_.parent[child] = shared;
      blocks_.refcount[shared] = 2;
      blocks_.SplitFront(b, moved_pages, shared);
      blocks_.start_pos[shared] = blocks_.start_pos[b];
      blocks_.start_pos[b] += moved;
      blocks_.seq_length[shared] = moved;
      blocks_.seq_length[b] -= moved;
      if (seqs_[pi].window != -1 && b == seqs_[pi].last_block) {
        KV_CHECK(moved <= seqs_[pi].last_block_sink) << "fork beyond the attention sink";
        seqs_[pi].last_block_sink -= moved;
      }
    }
    blocks_.start_pos[child] = static_cast<int32_t>(fork_pos - in_page);
    blocks_.seq_length[child] = in_page;
    if (in_page > 0) {
      const int32_t src_page = blocks_.Page(b, 0);
      const int32_t tgt_page = pages_.Pop();
      blocks_.PushPage(child, tgt_page);
      copy_log_.insert(copy_log_.end(), {src_page, tgt_page, in_page});
    }
    break;
  }
  NewSeq(child_seq_id, child);
}

// :772-801
void KVBookkeeper::EnableSlidingWindowForSeq(int64_t seq_id, int32_t sliding_window_size, int32_t attn_sink_size) {
  RequireUsable();
  KV_CHECK(cfg_.support_sliding_window || cfg_.support_layer_sliding_window)
      << "The KV cache does not support sliding window.";
  const int32_t index = RequireSeq(seq_id);
  KV_CHECK(attn_sink_size >= 0) << "The specified attention sink size is expected to be non negative";
  KV_CHECK(sliding_window_size > 0) << "The specified sliding window size should be positive.";
  KV_CHECK(attn_sink_size < sliding_window_size) << "The attn sink size should be less than the sliding window size.";
  SeqRecord& seq = seqs_[index];
  KV_CHECK(seq.window == -1) << "A sequence cannot be enabled twice for sliding window.";
  const int32_t prefix_length = seq.length - blocks_.seq_length[seq.last_block];
  KV_CHECK(prefix_length >= 0) << "negative prefix length";
  seq.last_block_sink = std::max(attn_sink_size - prefix_length, 0);
  seq.window = sliding_window_size;
}

// :803-862
void KVBookkeeper::PopN(int64_t seq_id, int32_t n) {
  RequireUsable();
  const int32_t index = RequireSeq(seq_id);
  KV_CHECK(n >= 0) << "The length of popping " << n << " cannot be negative.";
  KV_CHECK(n <= seqs_[index].length) << "The sequence only has length " << seqs_[index].length
                                     << ", while the length of pop is " << n
                                     << " which exceeds the whole sequence length.";
  if (n == 0) return;
  const int64_t ps = cfg_.page_size;
  SeqRecord& seq = seqs_[index];
  int32_t b = seq.last_block;
  KV_CHECK(blocks_.refcount[b] >= 1) << "block reference count underflow";
  while (b != -1 && blocks_.refcount[b] == 1) {
    const int32_t len = blocks_.seq_length[b];
    if (n > len) {  // the whole block goes
      n -= len;
      seq.length -= len;
      const int32_t* ids = blocks_.Pages(b);
      for (int32_t i = 0, cnt = blocks_.NumPages(b); i < cnt; ++i) pages_.Push(ids[i]);
      blocks_.Release(b);
      b = blocks_.parent[b];
      seq.last_block = b;
      continue;
    }
    const int64_t keep = (len - n + ps - 1) / ps;
    while (blocks_.NumPages(b) > keep) pages_.Push(blocks_.PopPage(b));
    seq.length -= n;
    blocks_.seq_length[b] -= n;
    n = 0;
    break;
  }
  if (n != 0) {
    // The pop reaches into a block that others share: a fork below the pop point under a temporary
    // id takes the place of the sequence.
    const int64_t temp_id = -1 - seq_id;
    KV_CHECK(FindSeq(temp_id) < 0) << "temporary sequence id is in use";
    ForkSequence(seq_id, temp_id, seqs_[index].length - n);
    RemoveSequence(seq_id);
    const int32_t moved = FindSeq(temp_id);
    seq_index_.erase(temp_id);
    seqs_[moved].id = seq_id;
    seq_index_.emplace(seq_id, moved);
  }
}

// :866-880
bool KVBookkeeper::Empty() const {
  return seq_index_.empty() && blocks_.NumFree() == blocks_.Size() && pages_.Size() == cfg_.num_total_pages;
}

int32_t KVBookkeeper::TotalSequenceLength() const {
  int32_t total = 0;
  for (const auto& entry : seq_index_) total += seqs_[entry.second].length;
  return total;
}

// ------------------------------------------------------------------------------------ windows
// attn_utils.h:289-303
int32_t KVBookkeeper::LayerWindowOffset(int64_t seq_length) const {
  if (seq_length <= cfg_.layer_sliding_window_size) return 0;
  return static_cast<int32_t>((seq_length - cfg_.layer_sliding_window_size) % cfg_.page_size);
}
int32_t KVBookkeeper::LayerWindowNumPages(int64_t seq_length) const {
  if (seq_length == 0) return 0;
  const int64_t window_length = std::min(seq_length, cfg_.layer_sliding_window_size);
  return static_cast<int32_t>((LayerWindowOffset(seq_length) + window_length + cfg_.page_size - 1) / cfg_.page_size);
}

// :1935-1992: tokens beyond the window leave the last block from behind the attention sink; pages they
// leave empty go back to the pool
void KVBookkeeper::SlideWindow(SeqRecord& seq) {
  if (seq.window == -1 || !cfg_.support_sliding_window) return;
  if (seq.length <= seq.window) return;
  const int32_t ps = static_cast<int32_t>(cfg_.page_size);
  const int32_t to_slide = seq.length - seq.window;
  const int32_t b = seq.last_block;
  if (seq.last_block_sink > 0 && blocks_.sink_length[b] == 0) {
    KV_CHECK(blocks_.window_offset[b] == 0) << "sliding window offset set before the sink";
    blocks_.sink_length[b] = seq.last_block_sink;
    blocks_.window_offset[b] = seq.last_block_sink;
  }
  // Only the last block slides.  The reference erases pages without looking (:1966-1972) and runs off
  // the end of the block's page list when a shared prefix alone is longer than the window; here
  // that is an error like any other.
  KV_CHECK(to_slide <= blocks_.seq_length[b] - blocks_.sink_length[b])
      << "The sliding window has to drop " << to_slide << " tokens, but the last block of the sequence holds only "
      << blocks_.seq_length[b] - blocks_.sink_length[b] << " behind its attention sink.";
  const int32_t sink_pages = (blocks_.sink_length[b] + ps - 1) / ps;
  int32_t first_page = (blocks_.window_offset[b] + to_slide) / ps;
  const int32_t first_slot = (blocks_.window_offset[b] + to_slide) % ps;
  for (; first_page > sink_pages; --first_page) {
    const int32_t id = blocks_.Page(b, sink_pages);
    if (id != kTempPageId) pages_.Push(id);
    blocks_.ErasePage(b, sink_pages);
  }
  KV_CHECK(first_page == sink_pages - 1 || first_page == sink_pages) << "sliding window left an unexpected first page";
  seq.length = seq.window;
  blocks_.seq_length[b] -= to_slide;
  blocks_.window_offset[b] = first_page * ps + first_slot;
  KV_CHECK(blocks_.seq_length[b] >= blocks_.sink_length[b]) << "block shorter than its attention sink";
  KV_CHECK(blocks_.window_offset[b] >= blocks_.sink_length[b]) << "sliding window overlaps the attention sink";
  KV_CHECK((blocks_.window_offset[b] + (blocks_.seq_length[b] - blocks_.sink_length[b]) + ps - 1) / ps ==
           blocks_.NumPages(b))
      << "page count does not match the slid window";
}

// :2004-2044
void KVBookkeeper::ReserveAppendLength(SeqRecord& seq, int64_t append_length) {
  const int32_t b = seq.last_block;
  const int64_t ps = cfg_.page_size;
  KV_CHECK(append_length > 0) << "Append with length 0 is not allowed.";
  KV_CHECK(blocks_.refcount[b] == 1) << "The block is " << blocks_.refcount[b] - 1
                                     << "-time referenced by other blocks, thus cannot accept new KV values.";
  const int64_t want = (blocks_.seq_length[b] - blocks_.sink_length[b] + blocks_.window_offset[b] + append_length + ps - 1) / ps;
  const bool may_borrow = seq.window != -1 && cfg_.support_sliding_window;
  for (int64_t have = blocks_.NumPages(b); have < want; ++have) {
    // a sliding sequence that finds the pool empty takes a placeholder: the slide below frees pages
    blocks_.PushPage(b, pages_.Empty() && may_borrow ? kTempPageId : pages_.Pop());
  }
  blocks_.seq_length[b] += static_cast<int32_t>(append_length);
  SlideWindow(seq);
  if (cfg_.support_sliding_window) {
    for (int32_t i = 0, n = blocks_.NumPages(b); i < n; ++i) {
      if (blocks_.Page(b, i) == kTempPageId) blocks_.SetPage(b, i, pages_.Pop());
    }
  }
}

// ------------------------------------------------------------------------------------ the step
int32_t* KVBookkeeper::Place(AuxSpan* span, int64_t size) {
  const int64_t at = AlignUp4(step_.used);
  KV_CHECK(at + size <= capacity_) << "auxiliary buffer overflow (" << at + size << " > " << capacity_
                                   << "): batch or append length beyond the configured limits";
  span->offset = at;
  span->size = size;
  step_.used = at + size;
  return buffer_ + at;
}

// :884-1212
void KVBookkeeper::BeginForward(const int64_t* seq_ids, const int64_t* append_lengths, int64_t batch_size,
                                const int64_t* token_tree_parent_ptr, int64_t n_tree) {
  if (cfg_.first_layer_is_mla) {
    KV_CHECK(token_tree_parent_ptr == nullptr) << "Tree attention is not supported yet for MLA";
  }
  RequireUsable();
  began_forward_ = false;  // until the step is complete
  // armed at the first change to a sequence, disarmed when the step is complete
  struct PoisonOnFailure {
    KVBookkeeper* book;
    bool armed = false;
    ~PoisonOnFailure() {
      if (armed) book->poisoned_ = true;
    }
  } guard{this};
  if (buffer_ == nullptr) {
    own_buffer_.resize(RequiredCapacity());
    buffer_ = own_buffer_.data();
    capacity_ = static_cast<int64_t>(own_buffer_.size());
  }
  const int32_t ps = static_cast<int32_t>(cfg_.page_size);
  const int64_t B = batch_size;
  cur_seq_ids_.assign(seq_ids, seq_ids + B);
  cur_append_lengths_.assign(append_lengths, append_lengths + B);
  cur_seq_index_.resize(B);
  last_block_len_before_.resize(2 * B);  // second half: k_ragged_rope_pos_offset until its place is known
  int32_t* k_ragged = last_block_len_before_.data() + B;
  step_ = StepLayout{};
  step_.is_decode_request = true;
  // what can be checked before anything changes is checked first: every id known, every length positive (the
  // reference finds these while it already bumps lengths, paged_kv_cache.cc:905-925; the messages are its own)
  for (int64_t i = 0; i < B; ++i) {
    RequireSeq(seq_ids[i]);
    KV_CHECK(append_lengths[i] > 0) << "Append with length 0 is not allowed.";
  }
  for (int64_t i = 0; i < B; ++i) {
    const int32_t index = RequireSeq(seq_ids[i]);
    SeqRecord& seq = seqs_[index];
    cur_seq_index_[i] = index;
    last_block_len_before_[i] = blocks_.seq_length[seq.last_block];
    k_ragged[i] = seq.length - (seq.committed ? 0 : static_cast<int32_t>(seq.tree_parent.size()));
    guard.armed = true;
    seq.length += static_cast<int32_t>(append_lengths[i]);
    if (append_lengths[i] != 1) step_.is_decode_request = false;
    step_.total_append_length += append_lengths[i];
  }
  KV_CHECK(B > 0) << "begin_forward needs at least one sequence";

  // ---- every sequence's blocks, leaf first; depth d of sequence i is trace_[end_i - 1 - d] ---------------
  trace_.clear();
  trace_begin_.resize(B + 1);
  int max_len = 0;
  for (int64_t i = 0; i < B; ++i) {
    trace_begin_[i] = static_cast<int32_t>(trace_.size());
    for (int32_t b = seqs_[cur_seq_index_[i]].last_block; b != -1; b = blocks_.parent[b]) trace_.push_back(b);
    max_len = std::max(max_len, static_cast<int>(trace_.size()) - trace_begin_[i]);
  }
  trace_begin_[B] = static_cast<int32_t>(trace_.size());
  const int num_depths = std::min(max_len, kMaxBlockDepth);
  step_.num_depths = num_depths;
  auto trace_len = [&](int64_t i) { return trace_begin_[i + 1] - trace_begin_[i]; };
  auto block_at = [&](int64_t i, int d) { return trace_[trace_begin_[i + 1] - 1 - d]; };  // d < trace_len(i)

  // ---- entries of every depth (attn_utils.h:243-332): consecutive sequences on one block share an
  // entry unless the decode kernel runs the depth or the depth is the last one ---------------------------
  for (int d = 0; d < num_depths; ++d) {
    std::vector<int32_t>& ids = depth_block_[d];
    ids.resize(B);
    for (int64_t i = 0; i < B; ++i) ids[i] = d < trace_len(i) ? block_at(i, d) : -1;
    int64_t pages_each = 0, pages_merged = 0;
    for (int64_t i = 0; i < B; ++i) {
      if (ids[i] == -1) continue;
      pages_each += blocks_.NumPages(ids[i]);
      if (i == 0 || ids[i] != ids[i - 1]) pages_merged += blocks_.NumPages(ids[i]);
    }
    const double ratio = pages_merged > 0 ? 1.0 * pages_each / pages_merged : 0.0;
    const bool decode = step_.is_decode_request && ratio < 32;
    step_.use_decode_kernel[d] = decode;
    const bool merge = !decode && d != kMaxBlockDepth - 1;
    entry_block_[d].clear();
    entry_qlen_[d].clear();
    entry_first_seq_[d].clear();
    for (int64_t i = 0; i < B; ++i) {
      if (merge && i > 0 && ids[i] == ids[i - 1]) {
        entry_qlen_[d].back() += static_cast<int32_t>(append_lengths[i]);
      } else {
        entry_block_[d].push_back(ids[i]);
        entry_qlen_[d].push_back(static_cast<int32_t>(append_lengths[i]));
        entry_first_seq_[d].push_back(static_cast<int32_t>(i));
      }
    }
  }
  if (num_depths == kMaxBlockDepth) {
    KV_CHECK(static_cast<int64_t>(entry_block_[num_depths - 1].size()) == B) << "blocks at the maximum depth must not coalesce";
  }

  step_.append_before_attn = !cfg_.support_sliding_window && step_.use_decode_kernel[num_depths - 1];
  for (int64_t i = 0; i < B; ++i) {
    if (!seqs_[cur_seq_index_[i]].committed) step_.append_before_attn = true;
  }

  if (token_tree_parent_ptr != nullptr) {
    KV_CHECK(!cfg_.support_sliding_window) << "Tree attention does not support sliding window.";
    KV_CHECK(!cfg_.rope_inline) << "Tree attention does not support inline RoPE mode.";
    BuildTreeMasks(token_tree_parent_ptr, n_tree);
  } else {
    for (int64_t i = 0; i < B; ++i) {
      SeqRecord& seq = seqs_[cur_seq_index_[i]];
      KV_CHECK(seq.committed) << "The input batch does not form a tree, in which case the sequences in the input "
                                 "batch are expected to have their accepted tokens token tree nodes committed. "
                                 "Please invoke CommitAcceptedTokenTreeNodes for sequence "
                              << seq_ids[i];
      seq.is_chain = true;
      seq.tree_parent.clear();
      seq.tree_depth.clear();
    }
    for (int d = 0; d < kMaxBlockDepth; ++d) step_.is_chain[d] = true;
  }

  if (step_.append_before_attn) {
    for (int64_t i = 0; i < B; ++i) ReserveAppendLength(seqs_[cur_seq_index_[i]], append_lengths[i]);
  }

  // ---- sizes, then places in the order of the reference's upload (:2388-2517), then the values ------------
  // blocks of sequence i behind the last depth are listed behind its block of that depth
  auto for_each_block_of_entry = [&](int d, int e, auto&& f) {
    const int32_t b = entry_block_[d][e];
    if (b == -1) return;
    f(b);
    if (d == kMaxBlockDepth - 1) {
      const int64_t i = entry_first_seq_[d][e];
      for (int k = kMaxBlockDepth; k < trace_len(i); ++k) f(block_at(i, k));
    }
  };
  int64_t n_entries[kMaxBlockDepth] = {0, 0}, n_pages[kMaxBlockDepth] = {0, 0}, n_pages_sw[kMaxBlockDepth] = {0, 0};
  int64_t n_absent[kMaxBlockDepth] = {0, 0};
  for (int d = 0; d < num_depths; ++d) {
    n_entries[d] = static_cast<int64_t>(entry_block_[d].size());
    for (int e = 0; e < n_entries[d]; ++e) {
      if (entry_block_[d][e] == -1) {
        ++n_absent[d];
        continue;
      }
      int64_t pages = 0, tokens = 0;
      for_each_block_of_entry(d, e, [&](int32_t b) {
        pages += blocks_.NumPages(b);
        tokens += blocks_.seq_length[b];
      });
      n_pages[d] += pages;
      n_pages_sw[d] += std::min<int64_t>(pages, LayerWindowNumPages(tokens));
    }
  }
  const bool layer_sw = cfg_.support_layer_sliding_window;
  int32_t* q_rope = Place(&step_.q_rope_position_map, step_.total_append_length);
  int32_t *qo_indptr[kMaxBlockDepth], *page_indptr[kMaxBlockDepth], *page_indices[kMaxBlockDepth];
  int32_t *page_indptr_sw[kMaxBlockDepth] = {nullptr, nullptr}, *page_indices_sw[kMaxBlockDepth] = {nullptr, nullptr};
  int32_t *rows[kMaxBlockDepth], *k_rope[kMaxBlockDepth], *k_rope_sw[kMaxBlockDepth] = {nullptr, nullptr};
  for (int d = 0; d < num_depths; ++d) qo_indptr[d] = Place(&step_.qo_indptr[d], n_entries[d] + 1);
  for (int d = 0; d < num_depths; ++d) page_indptr[d] = Place(&step_.page_indptr[d], n_entries[d] + 1);
  for (int d = 0; d < num_depths; ++d) page_indices[d] = Place(&step_.page_indices[d], n_pages[d]);
  if (layer_sw) {
    for (int d = 0; d < num_depths; ++d) page_indptr_sw[d] = Place(&step_.page_indptr_sw[d], n_entries[d] + 1);
    for (int d = 0; d < num_depths; ++d) page_indices_sw[d] = Place(&step_.page_indices_sw[d], n_pages_sw[d]);
  }
  for (int d = 0; d < num_depths; ++d) {
    // last_page_len, sliding_window_offset, sink_size back to back: one (3, n) array where a kernel wants all three
    AuxSpan three;
    rows[d] = Place(&three, 3 * n_entries[d]);
    step_.last_page_len[d] = AuxSpan{three.offset, n_entries[d]};
    step_.sliding_window_offset[d] = AuxSpan{three.offset + n_entries[d], n_entries[d]};
    step_.sink_size[d] = AuxSpan{three.offset + 2 * n_entries[d], n_entries[d]};
    step_.length_info[d] = cfg_.support_sliding_window ? three : step_.last_page_len[d];
    step_.layer_sw_length_info[d] = three;
  }
  for (int d = 0; d < num_depths; ++d) {
    k_rope[d] = Place(&step_.k_rope_pos_offset[d], n_entries[d]);
    if (layer_sw) k_rope_sw[d] = Place(&step_.k_rope_pos_offset_sw[d], n_entries[d]);
  }
  int32_t* append_indptr = Place(&step_.cur_append_lengths_indptr, B + 1);
  std::memcpy(Place(&step_.k_ragged_rope_pos_offset, B), k_ragged, static_cast<size_t>(B) * sizeof(int32_t));
  int32_t* append_map = Place(&step_.append_position_map, step_.total_append_length);
  for (int d = 0; d < num_depths; ++d) {
    if (step_.is_chain[d]) continue;
    std::memcpy(Place(&step_.tree_attn_mask[d], static_cast<int64_t>(tree_mask_[d].size())), tree_mask_[d].data(),
                tree_mask_[d].size() * sizeof(int32_t));
    std::memcpy(Place(&step_.tree_attn_mn_indptr[d], static_cast<int64_t>(tree_mn_indptr_[d].size())),
                tree_mn_indptr_[d].data(), tree_mn_indptr_[d].size() * sizeof(int32_t));
  }
  const int64_t uploaded = step_.used;
  if (!layer_sw) {
    // The layer-window view of the page tables is still part of the step's description (the reference
    // builds it whatever the layers are), but no kernel of this cache reads it: it sits behind the part
    // that is uploaded.  Without layer windows the reference only notes a position offset for absent
    // blocks.
    for (int d = 0; d < num_depths; ++d) page_indptr_sw[d] = Place(&step_.page_indptr_sw[d], n_entries[d] + 1);
    for (int d = 0; d < num_depths; ++d) page_indices_sw[d] = Place(&step_.page_indices_sw[d], n_pages_sw[d]);
    for (int d = 0; d < num_depths; ++d) k_rope_sw[d] = Place(&step_.k_rope_pos_offset_sw[d], n_absent[d]);
  }

  for (int d = 0; d < num_depths; ++d) {
    const int64_t n = n_entries[d];
    int32_t *last_len = rows[d], *win_off = rows[d] + n, *sink = rows[d] + 2 * n;
    int32_t* pages_out = page_indices[d];
    int32_t* pages_sw_out = page_indices_sw[d];
    int32_t* absent_out = layer_sw ? nullptr : k_rope_sw[d];
    qo_indptr[d][0] = page_indptr[d][0] = page_indptr_sw[d][0] = 0;
    for (int e = 0; e < n; ++e) {
      qo_indptr[d][e + 1] = qo_indptr[d][e] + entry_qlen_[d][e];
      const int32_t first = entry_block_[d][e];
      if (first == -1) {
        page_indptr[d][e + 1] = page_indptr[d][e];
        page_indptr_sw[d][e + 1] = page_indptr_sw[d][e];
        last_len[e] = win_off[e] = sink[e] = k_rope[d][e] = 0;
        if (layer_sw) {
          k_rope_sw[d][e] = 0;
        } else {
          *absent_out++ = 0;
        }
        continue;
      }
      int32_t* entry_pages = pages_out;
      int32_t tokens = 0, last_block = first;
      for_each_block_of_entry(d, e, [&](int32_t b) {
        const int32_t cnt = blocks_.NumPages(b);
        if (cnt > 0) std::memcpy(pages_out, blocks_.Pages(b), static_cast<size_t>(cnt) * sizeof(int32_t));
        pages_out += cnt;
        tokens += blocks_.seq_length[b];
        last_block = b;
      });
      const int32_t pages = static_cast<int32_t>(pages_out - entry_pages);
      page_indptr[d][e + 1] = page_indptr[d][e] + pages;
      const int32_t pages_sw = std::min(pages, LayerWindowNumPages(tokens));  // the newest pages
      std::memcpy(pages_sw_out, pages_out - pages_sw, static_cast<size_t>(pages_sw) * sizeof(int32_t));
      pages_sw_out += pages_sw;
      page_indptr_sw[d][e + 1] = page_indptr_sw[d][e] + pages_sw;
      last_len[e] = tokens == 0 ? 0 : (tokens - blocks_.sink_length[last_block] + blocks_.window_offset[last_block] - 1) % ps + 1;
      win_off[e] = layer_sw ? LayerWindowOffset(tokens) : blocks_.window_offset[last_block];
      sink[e] = blocks_.sink_length[last_block];
      k_rope[d][e] = blocks_.start_pos[first];
      if (layer_sw) {
        k_rope_sw[d][e] = static_cast<int32_t>(
            std::max<int64_t>(0, blocks_.start_pos[first] + tokens - cfg_.layer_sliding_window_size));
      }
    }
  }

  if (!step_.append_before_attn) {
    for (int64_t i = 0; i < B; ++i) ReserveAppendLength(seqs_[cur_seq_index_[i]], append_lengths[i]);
  }

  // ---- positions of the new tokens and the slots they are written to (:1150-1183) -----------------------
  int64_t cursor = 0;
  append_indptr[0] = 0;
  for (int64_t i = 0; i < B; ++i) {
    const SeqRecord& seq = seqs_[cur_seq_index_[i]];
    const int32_t b = seq.last_block;
    const int32_t len = static_cast<int32_t>(append_lengths[i]);
    const int32_t block_len = blocks_.seq_length[b], sink_len = blocks_.sink_length[b], off = blocks_.window_offset[b];
    const int32_t* ids = blocks_.Pages(b);
    const int32_t* depths = nullptr;
    if (!seq.tree_depth.empty()) {
      const int64_t offset_in_tree = static_cast<int64_t>(seq.tree_parent.size()) - len;
      KV_CHECK(offset_in_tree >= 0) << "token tree smaller than the append length";
      depths = seq.tree_depth.data() + offset_in_tree;
    }
    for (int32_t pos = 0; pos < len; ++pos) {
      q_rope[cursor] = k_ragged[i] + (depths != nullptr ? depths[pos] : pos);
      const int32_t before = last_block_len_before_[i] + pos;  // where the token falls if the sink is still filling
      const int32_t in_block = block_len - len + pos;
      int32_t slot_index;
      if (before < sink_len) {
        slot_index = before;
      } else if (in_block < sink_len) {
        slot_index = -1;  // slid out before it was ever written
      } else {
        slot_index = in_block - sink_len + off;
      }
      append_map[cursor] = slot_index < 0 ? -1 : ids[slot_index / ps] * ps + slot_index % ps;
      ++cursor;
    }
    append_indptr[i + 1] = static_cast<int32_t>(cursor);
  }
  step_.used = uploaded;  // what follows is host-side description only
  began_forward_ = true;
  guard.armed = false;
}

// :1800-1928: labels (pre-order number, end of the subtree's range) of every node of every tree
void KVBookkeeper::BuildTreeMasks(const int64_t* token_tree_parent_ptr, int64_t n_tree) {
  const int64_t B = static_cast<int64_t>(cur_seq_ids_.size());
  auto trace_len = [&](int64_t i) { return trace_begin_[i + 1] - trace_begin_[i]; };
  for (int d = 0; d < step_.num_depths; ++d) {
    std::vector<int32_t>& mn_indptr = tree_mn_indptr_[d];
    std::vector<int32_t>& mask = tree_mask_[d];
    mn_indptr.assign(1, 0);
    mask.clear();
    for (int k = 0; k < kMaxBlockDepth; ++k) step_.is_chain[k] = true;
    bool all_chains = true;
    int64_t offset = 0;
    in_depth_.assign(B, 0);
    for (int64_t i = 0; i < B; ++i) {
      SeqRecord& seq = seqs_[cur_seq_index_[i]];
      const int64_t len = cur_append_lengths_[i];
      // with the new tokens in the pages already, a tree is masked at the depth that holds them
      const bool here = !step_.append_before_attn || depth_block_[d][i] == seq.last_block ||
                        (d + 1 == kMaxBlockDepth && trace_len(i) > kMaxBlockDepth);
      in_depth_[i] = here;
      if (!here) {
        mn_indptr.push_back(mn_indptr.back());
        offset += len;
        continue;
      }
      KV_CHECK(static_cast<int64_t>(seq.tree_parent.size()) <= blocks_.seq_length[seq.last_block])
          << "The token tree size is larger than the sequence length of the last block.";
      KV_CHECK(offset + len <= n_tree) << "Invalid token tree size.";
      for (int64_t j = 0; j < len; ++j) seq.tree_parent.push_back(static_cast<int32_t>(token_tree_parent_ptr[offset + j]));
      offset += len;
      KV_CHECK(static_cast<int>(seq.tree_parent.size()) <= kTreeAttnMaxTreeSize)
          << "The tree size is " << len << " which exceeds the maximum tree size limit " << kTreeAttnMaxTreeSize;
      mn_indptr.push_back(mn_indptr.back() + static_cast<int32_t>(seq.tree_parent.size()));
    }
    KV_CHECK(n_tree == offset) << "Invalid token tree size. The sum of \"append_lengths\" is " << offset
                               << " while there are " << n_tree << " elements in \"token_tree_parent_ptr\".";
    for (int64_t i = 0; i < B; ++i) {
      if (!in_depth_[i]) continue;
      SeqRecord& seq = seqs_[cur_seq_index_[i]];
      const int32_t size = static_cast<int32_t>(seq.tree_parent.size());
      seq.is_chain = true;
      seq.committed = false;
      seq.tree_depth.assign(size, 0);
      for (int32_t n = 0; n < size; ++n) {
        const int32_t up = seq.tree_parent[n];
        KV_CHECK(up < n) << "Invalid token tree. The parent of node " << n << " in tree " << i << " is " << up
                         << ", which is not smaller than " << n;
        KV_CHECK(up >= -1) << "Invalid token tree. The parent of node " << n << " in tree " << i << " is " << up;
        if (up != n - 1) {
          seq.is_chain = false;
          all_chains = false;
        }
        seq.tree_depth[n] = up == -1 ? 0 : seq.tree_depth[up] + 1;
      }
      // A depth-first walk that visits children in index order numbers a node's subtree contiguously:
      // the label of node n is [first, first + size of its subtree).  Parents come before children in
      // the array, so subtree sizes add up in one backward pass and the first numbers follow in one
      // forward pass (next_first[p]: the number the next child of p will take).
      subtree_.assign(size, 1);
      for (int32_t n = size - 1; n >= 0; --n) {
        if (seq.tree_parent[n] != -1) subtree_[seq.tree_parent[n]] += subtree_[n];
      }
      next_first_.assign(size, 0);
      int32_t next_root = 0;
      for (int32_t n = 0; n < size; ++n) {
        const int32_t up = seq.tree_parent[n];
        int32_t& next = up == -1 ? next_root : next_first_[up];
        const int32_t first = next;
        next += subtree_[n];
        next_first_[n] = first + 1;
        mask.push_back(first);
        mask.push_back(first + subtree_[n]);
      }
    }
    step_.is_chain[d] = all_chains;
    if (!step_.append_before_attn) break;
  }
}

// :1566-1659
bool KVBookkeeper::CommitAcceptedTokenTreeNodes(const int64_t* seq_ids, const int64_t* leaf_indices, int num) {
  RequireUsable();
  // The reference takes the batch of the last step for granted (its only caller is its own VM); here the
  // call comes through a C ABI: a different batch would index the step's arrays out of range or pop the
  // wrong sequences, so it is refused before anything changes.
  KV_CHECK(num >= 0 && static_cast<size_t>(num) == cur_seq_ids_.size())
      << "commit_accepted_token_tree_nodes: " << num << " sequences, the last step had " << cur_seq_ids_.size();
  for (int i = 0; i < num; ++i) {
    KV_CHECK(seq_ids[i] == cur_seq_ids_[i])
        << "commit_accepted_token_tree_nodes: sequence " << seq_ids[i] << " at position " << i
        << ", the last step had sequence " << cur_seq_ids_[i] << " there";
  }
  bool is_chain = true;
  for (int i = 0; i < num; ++i) {
    const SeqRecord& seq = seqs_[RequireSeq(seq_ids[i])];
    is_chain = seq.is_chain;
    KV_CHECK(leaf_indices[i] == -1 || !seq.committed)
        << "The accepted nodes of sequence " << seq_ids[i] << " are already committed.";
    KV_CHECK(leaf_indices[i] >= -1) << "Invalid tree index " << leaf_indices[i] << " which is less than -1";
    KV_CHECK(leaf_indices[i] < static_cast<int64_t>(seq.tree_parent.size()))
        << "Invalid tree index " << leaf_indices[i] << " which is larger than or equals to the append length "
        << seq.tree_parent.size() << " of the sequence";
  }
  bool copies = false;
  if (!is_chain) {
    commit_length_indptr_.assign(1, 0);
    commit_src_.clear();
    commit_dst_.clear();
    const int32_t* append_map = buffer_ + step_.append_position_map.offset;
    const int32_t* append_indptr = buffer_ + step_.cur_append_lengths_indptr.offset;
    for (int i = 0; i < num; ++i) {
      const SeqRecord& seq = seqs_[FindSeq(seq_ids[i])];
      if (leaf_indices[i] != -1) {
        // the accepted path, root first: its k-th node moves to the k-th new slot of the sequence;
        // a head of the path that already sits there stays
        path_.clear();
        for (int32_t node = static_cast<int32_t>(leaf_indices[i]); node != -1; node = seq.tree_parent[node]) path_.push_back(node);
        KV_CHECK(static_cast<int>(path_.size()) == seq.tree_depth[leaf_indices[i]] + 1) << "token tree depth mismatch";
        std::reverse(path_.begin(), path_.end());
        size_t k = 0;
        while (k < path_.size() && path_[k] == static_cast<int32_t>(k)) ++k;
        for (; k < path_.size(); ++k) {
          commit_src_.push_back(append_map[append_indptr[i] + path_[k]]);
          commit_dst_.push_back(append_map[append_indptr[i] + static_cast<int32_t>(k)]);
        }
      }
      commit_length_indptr_.push_back(static_cast<int32_t>(commit_src_.size()));
    }
    copies = !commit_src_.empty();
  }
  for (int i = 0; i < num; ++i) {
    const SeqRecord& seq = seqs_[FindSeq(seq_ids[i])];
    const int64_t keep = leaf_indices[i] != -1 ? seq.tree_depth[leaf_indices[i]] + 1 : 0;
    PopN(cur_seq_ids_[i], static_cast<int32_t>(cur_append_lengths_[i] - keep));
    SeqRecord& after = seqs_[FindSeq(cur_seq_ids_[i])];  // a pop into a shared block re-creates the record
    after.committed = true;
    after.tree_parent.clear();
    after.tree_depth.clear();
  }
  return copies;
}

// ------------------------------------------------------------------------------------ introspection
std::vector<int32_t> KVBookkeeper::PositionMapOf(int64_t seq_id, int64_t start_pos, int64_t end_pos) const {
  const SeqRecord& seq = seqs_[RequireSeq(seq_id)];
  KV_CHECK(start_pos >= 0) << "DebugGetKV does not accept negative start_pos " << start_pos;
  KV_CHECK(end_pos <= seq.length) << "DebugGetKV does not accept out-of-range end_pos";
  KV_CHECK(start_pos < end_pos) << "DebugGetKV does not accept \"start_pos >= end_pos\"";
  const int32_t ps = static_cast<int32_t>(cfg_.page_size);
  std::vector<int32_t> chain;
  for (int32_t b = seq.last_block; b != -1; b = blocks_.parent[b]) chain.push_back(b);
  std::vector<int32_t> map;
  map.reserve(seq.length);
  for (auto it = chain.rbegin(); it != chain.rend(); ++it) {
    const int32_t b = *it;
    for (int32_t i = 0; i < blocks_.seq_length[b]; ++i) {
      const int32_t at = i < blocks_.sink_length[b] ? i : i - blocks_.sink_length[b] + blocks_.window_offset[b];
      map.push_back(blocks_.Page(b, at / ps) * ps + at % ps);
    }
  }
  return std::vector<int32_t>(map.begin() + start_pos, map.begin() + end_pos);
}

std::vector<int64_t> KVBookkeeper::DumpState() const {
  std::vector<int64_t> out;
  out.push_back(pages_.Size());
  out.insert(out.end(), pages_.Items().begin(), pages_.Items().end());
  out.push_back(blocks_.NumFree());
  out.insert(out.end(), blocks_.FreeBlocks().begin(), blocks_.FreeBlocks().end());
  out.push_back(blocks_.Size());
  for (int32_t b = 0; b < blocks_.Size(); ++b) {
    out.push_back(blocks_.NumPages(b));
    for (int32_t i = 0; i < blocks_.NumPages(b); ++i) out.push_back(blocks_.Page(b, i));
    out.insert(out.end(), {blocks_.seq_length[b], blocks_.start_pos[b], blocks_.sink_length[b], blocks_.window_offset[b],
                           blocks_.parent[b], blocks_.refcount[b]});
  }
  std::map<int64_t, int32_t> ordered(seq_index_.begin(), seq_index_.end());
  out.push_back(static_cast<int64_t>(ordered.size()));
  for (const auto& entry : ordered) {
    const SeqRecord& seq = seqs_[entry.second];
    out.insert(out.end(), {entry.first, seq.last_block, seq.length, seq.window, seq.last_block_sink});
  }
  return out;
}

AuxSpan KVBookkeeper::FindAux(const std::string& name, int depth) const {
  struct PerDepth {
    const char* name;
    const AuxSpan (StepLayout::*spans)[kMaxBlockDepth];
  };
  static const PerDepth per_depth[] = {
      {"qo_indptr", &StepLayout::qo_indptr},
      {"page_indptr", &StepLayout::page_indptr},
      {"page_indices", &StepLayout::page_indices},
      {"page_indptr_sliding_window", &StepLayout::page_indptr_sw},
      {"page_indices_sliding_window", &StepLayout::page_indices_sw},
      {"last_page_len", &StepLayout::last_page_len},
      {"sliding_window_offset", &StepLayout::sliding_window_offset},
      {"sink_size", &StepLayout::sink_size},
      {"k_rope_pos_offset", &StepLayout::k_rope_pos_offset},
      {"k_rope_pos_offset_sliding_window", &StepLayout::k_rope_pos_offset_sw},
      {"tree_attn_mask", &StepLayout::tree_attn_mask},
      {"tree_attn_mn_indptr", &StepLayout::tree_attn_mn_indptr}};
  for (const PerDepth& entry : per_depth) {
    if (name == entry.name) {
      KV_CHECK(depth >= 0 && depth < kMaxBlockDepth) << "depth " << depth << " out of range";
      const AuxSpan span = (step_.*(entry.spans))[depth];
      return span.present() ? span : AuxSpan{0, 0};
    }
  }
  const AuxSpan* global = nullptr;
  if (name == "q_rope_position_map") global = &step_.q_rope_position_map;
  if (name == "append_position_map") global = &step_.append_position_map;
  if (name == "cur_append_lengths_indptr") global = &step_.cur_append_lengths_indptr;
  if (name == "k_ragged_rope_pos_offset") global = &step_.k_ragged_rope_pos_offset;
  KV_CHECK(global != nullptr) << "unknown auxiliary array \"" << name << "\"";
  return global->present() ? *global : AuxSpan{0, 0};
}

}  // namespace tvmkv
