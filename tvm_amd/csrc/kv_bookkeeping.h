// Host bookkeeping of the paged KV cache: sequences, the prefix-sharing block tree, the page pool and
// the per-step auxiliary arrays.  No device code: the cache object (paged_kv_cache.cc) owns one of
// these and the device resources, and a host-only cache is just this class.
//
// Behaviour (verbs, order of checks, error texts, the order in which pages and blocks are handed out,
// every integer of the auxiliary arrays) follows the reference's PagedAttentionKVCacheObj
// (src/runtime/vm/paged_kv_cache.cc:561-1212, :1566-1659, :1800-2044) and src/runtime/vm/attn_utils.h.
// The representation is this library's own: blocks are structure-of-arrays with their page ids in
// slices of one arena (block_pool.h), sequences are records in a dense table, and a step's auxiliary
// arrays are laid out and written once, in place, in the buffer that is uploaded (no per-step
// containers, no second copy into a staging area).
#ifndef TVMKV_CSRC_KV_BOOKKEEPING_H_
#define TVMKV_CSRC_KV_BOOKKEEPING_H_

#include <algorithm>
#include <cstddef>
#include <cstdint>
#include <string>
#include <unordered_map>
#include <vector>

#include "block_pool.h"

namespace tvmkv {

constexpr int kMaxBlockDepth = 2;          // kPagedKVCacheMaxBlockDepth (attn_utils.h:50)
constexpr int kTreeAttnMaxTreeSize = 256;  // attn_utils.h:52
constexpr int32_t kTempPageId = -1;        // kPagedKVCacheTempPageId (attn_utils.h:58)

// One auxiliary array of the step: `size` int32 at element `offset` of the step's buffer.
struct AuxSpan {
  int64_t offset = -1;  // -1: not part of this step
  int64_t size = 0;
  bool present() const { return offset >= 0; }
};

// Everything attention needs to know about the current step, by depth where it applies.
struct StepLayout {
  int num_depths = 0;
  bool append_before_attn = false;
  bool is_decode_request = false;
  bool use_decode_kernel[kMaxBlockDepth] = {false, false};
  bool is_chain[kMaxBlockDepth] = {true, true};
  int64_t total_append_length = 0;
  int64_t used = 0;  // int32 elements of the buffer in use (what has to be uploaded)
  AuxSpan q_rope_position_map, append_position_map, cur_append_lengths_indptr, k_ragged_rope_pos_offset;
  AuxSpan qo_indptr[kMaxBlockDepth], page_indptr[kMaxBlockDepth], page_indices[kMaxBlockDepth];
  AuxSpan page_indptr_sw[kMaxBlockDepth], page_indices_sw[kMaxBlockDepth];
  AuxSpan last_page_len[kMaxBlockDepth], sliding_window_offset[kMaxBlockDepth], sink_size[kMaxBlockDepth];
  AuxSpan length_info[kMaxBlockDepth];           // last_page_len alone, or the three rows above back to back
  AuxSpan layer_sw_length_info[kMaxBlockDepth];  // the three rows again, for layers with their own window
  AuxSpan k_rope_pos_offset[kMaxBlockDepth], k_rope_pos_offset_sw[kMaxBlockDepth];
  AuxSpan tree_attn_mask[kMaxBlockDepth], tree_attn_mn_indptr[kMaxBlockDepth];
};

struct KVConfig {
  int64_t page_size = 16;
  int64_t num_total_pages = 0;
  int64_t reserved_num_seqs = 0;
  int64_t prefill_chunk_size = 0;
  int64_t layer_sliding_window_size = 1024;
  bool support_sliding_window = false;        // per-sequence windows with attention sinks
  bool support_layer_sliding_window = false;  // some layers attend to a fixed window
  bool rope_inline = false;
  bool first_layer_is_mla = false;
};

class KVBookkeeper {
 public:
  explicit KVBookkeeper(const KVConfig& config);

  // The buffer the next BeginForward writes the auxiliary arrays into (at least capacity int32).
  // The device layer alternates between two pinned buffers; a host-only cache keeps one of its own.
  void SetStepBuffer(int32_t* buffer, int64_t capacity) {
    buffer_ = buffer;
    capacity_ = capacity;
  }
  int64_t RequiredCapacity() const;  // what a step can need at most with this configuration

  // ---- verbs --------------------------------------------------------------------------------------
  void Clear();
  void AddSequence(int64_t seq_id);
  void RemoveSequence(int64_t seq_id);
  void ForkSequence(int64_t parent_seq_id, int64_t child_seq_id, int64_t fork_pos);
  void EnableSlidingWindowForSeq(int64_t seq_id, int32_t sliding_window_size, int32_t attn_sink_size);
  void PopN(int64_t seq_id, int32_t n);
  bool Empty() const;
  int32_t NumAvailablePages() const { return static_cast<int32_t>(pages_.Size()); }
  int32_t TotalSequenceLength() const;
  void BeginForward(const int64_t* seq_ids, const int64_t* append_lengths, int64_t batch_size,
                    const int64_t* token_tree_parent_ptr, int64_t n_tree);
  // Pops the rejected tokens of every sequence of the last step; fills the compaction copy list (empty
  // when every tree was a chain).  Returns true when there is something to copy.
  bool CommitAcceptedTokenTreeNodes(const int64_t* seq_ids, const int64_t* leaf_indices, int num);

  // ---- what the device layer and the introspection calls read -----------------------------------
  bool began_forward() const { return began_forward_; }
  const StepLayout& step() const { return step_; }
  const int32_t* step_buffer() const { return buffer_; }
  int64_t batch_size() const { return static_cast<int64_t>(cur_seq_ids_.size()); }
  // Slot ids of the cached tokens [start_pos, end_pos) of a sequence (DebugGetKV, :1698-1710).
  std::vector<int32_t> PositionMapOf(int64_t seq_id, int64_t start_pos, int64_t end_pos) const;
  const std::vector<int32_t>& commit_copy_length_indptr() const { return commit_length_indptr_; }
  const std::vector<int32_t>& commit_copy_src_pos() const { return commit_src_; }
  const std::vector<int32_t>& commit_copy_dst_pos() const { return commit_dst_; }
  // (src page, target page, tokens) of every partial-page copy a fork has asked for since Clear
  int64_t PageArenaInUse() const { return blocks_.ArenaInUse(); }
  const std::vector<int64_t>& CopyLog() const { return copy_log_; }
  // The log only grows between two Clear() calls; once it holds more than kCopyLogCap numbers, the oldest
  // of its first `consumed` numbers are dropped down to kCopyLogKeep.  Returns how many were dropped.
  static constexpr size_t kCopyLogCap = 3 * 8192, kCopyLogKeep = 3 * 1024;
  size_t TrimCopyLog(size_t consumed) {
    if (copy_log_.size() <= kCopyLogCap) return 0;
    const size_t drop = std::min(consumed, copy_log_.size() - kCopyLogKeep) / 3 * 3;
    copy_log_.erase(copy_log_.begin(), copy_log_.begin() + static_cast<std::ptrdiff_t>(drop));
    return drop;
  }
  std::vector<int64_t> DumpState() const;
  AuxSpan FindAux(const std::string& name, int depth) const;

 private:
  struct SeqRecord {
    int64_t id = 0;
    int32_t last_block = -1;
    int32_t length = 0;
    int32_t window = -1;          // sliding-window size, -1 = none
    int32_t last_block_sink = 0;  // attention-sink tokens that fall into the last block
    bool is_chain = true;
    bool committed = true;        // the token tree of the last step has been committed
    std::vector<int32_t> tree_parent, tree_depth;
  };

  int32_t FindSeq(int64_t seq_id) const;     // index into seqs_, -1 if absent
  int32_t RequireSeq(int64_t seq_id) const;  // throws the reference's "cannot be found" text
  int32_t NewSeq(int64_t seq_id, int32_t last_block);
  void DropSeq(int32_t index);
  int32_t LayerWindowOffset(int64_t seq_length) const;
  int32_t LayerWindowNumPages(int64_t seq_length) const;
  void ReserveAppendLength(SeqRecord& seq, int64_t append_length);
  void SlideWindow(SeqRecord& seq);
  void BuildTreeMasks(const int64_t* token_tree_parent_ptr, int64_t n_tree);
  int32_t* Place(AuxSpan* span, int64_t size);  // next 16-byte aligned run of the step buffer

  KVConfig cfg_;
  PageStack pages_;
  BlockPool blocks_;
  std::vector<SeqRecord> seqs_;        // dense; free entries are recycled
  std::vector<int32_t> free_seq_slots_;
  std::unordered_map<int64_t, int32_t> seq_index_;
  std::vector<int64_t> copy_log_;

  // ---- current step -----------------------------------------------------------------------------
  bool began_forward_ = false;
  // A begin_forward that fails after it has started to change sequences (the pool runs out, a sliding window
  // meets a shared prefix, the step buffer overflows) leaves lengths bumped and pages half reserved, as in the
  // reference (paged_kv_cache.cc:919 bumps seq_length before it reserves).  There the failure aborts the
  // program; here it comes back as an error code, so the object refuses every verb but Clear() afterwards
  // instead of handing out slots of a state nobody defined.
  bool poisoned_ = false;
  void RequireUsable() const;
  StepLayout step_;
  int32_t* buffer_ = nullptr;
  int64_t capacity_ = 0;
  std::vector<int32_t> own_buffer_;  // used until SetStepBuffer is called
  std::vector<int64_t> cur_seq_ids_, cur_append_lengths_;
  std::vector<int32_t> cur_seq_index_;
  // scratch of BeginForward, kept between calls so that a step allocates nothing
  std::vector<int32_t> trace_, trace_begin_, last_block_len_before_;
  std::vector<int32_t> depth_block_[kMaxBlockDepth];
  std::vector<int32_t> entry_block_[kMaxBlockDepth], entry_qlen_[kMaxBlockDepth], entry_first_seq_[kMaxBlockDepth];
  std::vector<int32_t> commit_length_indptr_, commit_src_, commit_dst_;
  std::vector<int32_t> tree_mask_[kMaxBlockDepth], tree_mn_indptr_[kMaxBlockDepth];
  std::vector<int32_t> subtree_, next_first_, path_;
  std::vector<char> in_depth_;
};

}  // namespace tvmkv

#endif  // TVMKV_CSRC_KV_BOOKKEEPING_H_
