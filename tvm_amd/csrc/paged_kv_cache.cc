// Host side of the paged KV cache: page pool, prefix-sharing block tree, per-step auxiliary
// arrays and the orchestration of the HIP kernels.  Behaviour (verbs, check order, error
// texts, page/block allocation order) follows the reference's PagedAttentionKVCacheObj
// (src/runtime/vm/paged_kv_cache.cc) and its helpers (src/runtime/vm/attn_utils.h); the
// device layer underneath is this library's own: one merged, double-buffered auxiliary
// buffer uploaded with a single copy per step on a private copy stream, and launchers from
// include/tvmkv.h for every kernel.
#include <algorithm>
#include <cstring>
#include <functional>
#include <map>
#include <memory>
#include <numeric>
#include <unordered_map>
#include <vector>

#include "common.h"

namespace tvmkv {

namespace {
thread_local std::string g_last_error;
}
void SetLastError(const std::string& msg) { g_last_error = msg; }

constexpr int kMaxBlockDepth = 2;     // kPagedKVCacheMaxBlockDepth (attn_utils.h:50)
constexpr int kTreeAttnMaxTreeSize = 256;  // attn_utils.h:52
constexpr int32_t kTempPageId = -1;   // kPagedKVCacheTempPageId (attn_utils.h:58)

// attn_utils.h:101-152
struct Block {
  std::vector<int32_t> page_ids;
  int32_t seq_length = 0;
  int32_t start_pos = 0;
  int32_t sink_length = 0;
  int32_t sliding_window_offset = 0;
  int32_t index;
  int32_t parent_idx = -1;
  int external_ref_cnt = 0;
  explicit Block(int32_t index) : index(index) {}
  void Reset() {
    page_ids.clear();
    seq_length = start_pos = sink_length = sliding_window_offset = 0;
    parent_idx = -1;
    external_ref_cnt = 0;
  }
};

// attn_utils.h:165-230
struct Sequence {
  int32_t last_block_idx;
  int32_t seq_length = 0;
  int sliding_window_size = -1;
  int last_block_attn_sink_size = 0;
  bool is_chain = true;
  std::vector<int32_t> token_tree_parent_ptr;
  std::vector<int32_t> token_tree_node_depths;
  bool accepted_indices_committed = true;

  Sequence(std::vector<Block>* pool, int32_t last_block_idx) : last_block_idx(last_block_idx) {
    ++pool->at(last_block_idx).external_ref_cnt;
    int32_t ptr = last_block_idx;
    while (true) {
      const Block& block = pool->at(ptr);
      seq_length += block.seq_length;
      if (block.parent_idx == -1) break;
      ptr = block.parent_idx;
    }
  }

  std::vector<int32_t> GetBlockTrace(const std::vector<Block>& pool) const {
    std::vector<int32_t> trace;
    for (int32_t ptr = last_block_idx; ptr != -1; ptr = pool[ptr].parent_idx) trace.push_back(ptr);
    std::reverse(trace.begin(), trace.end());
    return trace;
  }
};

using I32Vec = std::vector<int32_t>;

// One array of the merged device buffer.
struct AuxView {
  int32_t* ptr = nullptr;
  int64_t size = 0;
};

class PagedKVCache {
 public:
  PagedKVCache(const int64_t* cache_config, int n_config, int64_t layer_begin, int64_t layer_end,
               int64_t num_qo_heads, int64_t num_kv_heads, int64_t qk_head_dim, int64_t v_head_dim,
               std::vector<int64_t> attn_kinds, bool enable_kv_transfer, int rope_mode,
               double rope_scale, double rope_theta, int dtype_bits, int device_id)
      : page_size_(cache_config[3]),
        num_layers_(layer_end - layer_begin),
        layer_id_begin_offset_(layer_begin),
        layer_id_end_offset_(layer_end),
        num_qo_heads_(num_qo_heads),
        num_kv_heads_(num_kv_heads),
        qk_head_dim_(qk_head_dim),
        v_head_dim_(v_head_dim),
        prefill_chunk_size_(cache_config[2]),
        attn_kinds_(std::move(attn_kinds)),
        rotary_scale_(rope_scale),
        rotary_theta_(rope_theta),
        reserved_num_seqs_(cache_config[0]),
        device_(device_id) {
    // paged_kv_cache.cc:2606-2619
    int64_t total_token_capacity = cache_config[1];
    bool support_sliding_window = cache_config[4] != 0;
    layer_sliding_window_size_ = n_config == 6 ? cache_config[5] : 1024;
    KV_CHECK(page_size_ > 0) << "page_size must be positive";
    num_total_pages_ = (total_token_capacity + page_size_ - 1) / page_size_ + 1;
    if (support_sliding_window) num_total_pages_ += reserved_num_seqs_ * 2;
    // paged_kv_cache.cc:335-344
    bool has_layer_sliding =
        std::find(attn_kinds_.begin(), attn_kinds_.end(), TVMKV_ATTN_MHA_SLIDING) != attn_kinds_.end();
    support_sliding_window_ = has_layer_sliding ? false : support_sliding_window;
    support_layer_sliding_window_ = has_layer_sliding;
    rope_mode_ = (support_sliding_window && rope_mode != TVMKV_ROPE_NONE) ? TVMKV_ROPE_INLINE : rope_mode;
    KV_CHECK(layer_sliding_window_size_ > 0) << "Per-layer sliding window size must be positive.";
    bool has_mla = std::find(attn_kinds_.begin(), attn_kinds_.end(), TVMKV_ATTN_MLA) != attn_kinds_.end();
    if (has_mla) {
      KV_CHECK(!support_sliding_window_) << "Sliding window not supported yet for MLA";
      KV_CHECK(!enable_kv_transfer) << "KV transfer not supported yet for MLA";
    }
    KV_UNSUPPORTED(enable_kv_transfer)
        << "KV transfer (disaggregation) needs a second device and is not built in this library";
    KV_UNSUPPORTED(dtype_bits != 16) << "only fp16 KV storage is built (got " << dtype_bits << " bits)";
    KV_CHECK(static_cast<int64_t>(attn_kinds_.size()) >= layer_end)
        << "attn_kinds must cover every layer id up to " << layer_end;
    for (int64_t kind : attn_kinds_) {
      KV_UNSUPPORTED(kind != TVMKV_ATTN_MHA && kind != TVMKV_ATTN_MLA && kind != TVMKV_ATTN_MHA_SLIDING)
          << "attention kind " << kind << " is not supported";
    }
    for (int d = 0; d < kMaxBlockDepth; ++d) is_chain_on_depths_[d] = true;
    ResetPool();
    if (device_ >= 0) InitDevice();
  }

  ~PagedKVCache() { ReleaseDevice(); }

  // ---------------------------------------------------------------- pool verbs
  // paged_kv_cache.cc:561-570
  void Clear() {
    ResetPool();
    dirty_aux_data_device_ = false;
  }

  // :574-580
  void AddSequence(int64_t seq_id) {
    KV_CHECK(seq_map_.find(seq_id) == seq_map_.end())
        << "The sequence \"" << seq_id << "\" is already in the KV cache.";
    int32_t block_idx = GetFreeBlock();
    seq_map_.insert({seq_id, Sequence(&global_block_pool_, block_idx)});
    dirty_aux_data_device_ = true;
  }

  // :582-604
  void RemoveSequence(int64_t seq_id) {
    auto it = seq_map_.find(seq_id);
    KV_CHECK(it != seq_map_.end()) << "The sequence \"" << seq_id << "\" cannot be found in KV cache.";
    int32_t block_idx = it->second.last_block_idx;
    KV_CHECK(global_block_pool_[block_idx].external_ref_cnt >= 1) << "block reference count underflow";
    while (block_idx != -1 && global_block_pool_[block_idx].external_ref_cnt == 1) {
      for (int32_t page_id : global_block_pool_[block_idx].page_ids) free_page_ids_.push_back(page_id);
      free_block_idx_.push_back(block_idx);
      block_idx = global_block_pool_[block_idx].parent_idx;
    }
    if (block_idx != -1) {
      KV_CHECK(global_block_pool_[block_idx].external_ref_cnt > 1) << "block reference count underflow";
      --global_block_pool_[block_idx].external_ref_cnt;
    }
    seq_map_.erase(it);
    dirty_aux_data_device_ = true;
  }

  // :606-719
  void ForkSequence(int64_t parent_seq_id, int64_t child_seq_id, int64_t fork_pos) {
    auto parent_it = seq_map_.find(parent_seq_id);
    KV_CHECK(parent_it != seq_map_.end())
        << "The parent sequence \"" << parent_seq_id << "\" cannot be found in KV cache.";
    KV_CHECK(seq_map_.find(child_seq_id) == seq_map_.end())
        << "The child sequence \"" << child_seq_id << "\" is already in the KV cache.";
    KV_CHECK(fork_pos >= -1)
        << "The forked position should be non-negative, or -1 for last position as default.";
    KV_CHECK(fork_pos <= parent_it->second.seq_length)
        << "The forked position should not exceed the total length of parent sequence.";
    KV_CHECK(parent_it->second.accepted_indices_committed)
        << "The parent sequence's token tree computed in the last round of forward has not been "
           "committed with accepted nodes.";
    std::vector<Block>& pool = global_block_pool_;
    if (fork_pos == -1) fork_pos = parent_it->second.seq_length;

    if (parent_it->second.sliding_window_size != -1) {
      const Sequence& seq = parent_it->second;
      int32_t sink_size = seq.seq_length - pool[seq.last_block_idx].seq_length + seq.last_block_attn_sink_size;
      KV_CHECK(fork_pos <= sink_size)
          << "The parent sequence \"" << parent_seq_id
          << "\" is enabled with sliding window and thus only can be forked within sink size = "
          << sink_size << ". But the forked position = " << fork_pos << ".";
    }

    if (fork_pos == parent_it->second.seq_length && fork_pos % page_size_ == 0 &&
        pool[parent_it->second.last_block_idx].seq_length > 0) {
      // Give the parent an empty tail block so that it can keep decoding after the fork.
      int32_t new_block_idx = GetFreeBlock();
      pool[new_block_idx].start_pos = parent_it->second.seq_length;
      pool[new_block_idx].parent_idx = parent_it->second.last_block_idx;
      pool[new_block_idx].external_ref_cnt = 1;
      parent_it->second.last_block_idx = new_block_idx;
    }

    int32_t child_block_idx = GetFreeBlock();
    std::vector<int32_t> trace = parent_it->second.GetBlockTrace(pool);
    int64_t in_block_offset = fork_pos;
    for (int32_t forked_block_idx : trace) {
      if (forked_block_idx != trace.back()) {
        KV_CHECK(pool[forked_block_idx].seq_length > 0) << "interior block is empty";
        KV_CHECK(pool[forked_block_idx].seq_length % page_size_ == 0) << "interior block is not page aligned";
        if (pool[forked_block_idx].seq_length <= in_block_offset) {
          in_block_offset -= pool[forked_block_idx].seq_length;
          continue;
        }
      }
      int32_t in_page_offset = in_block_offset % page_size_;
      int32_t moved_offset = in_block_offset - in_page_offset;
      int32_t moved_pages = moved_offset / page_size_;
      if (moved_pages == 0) {
        int32_t parent_block_idx = pool[forked_block_idx].parent_idx;
        if (parent_block_idx != -1) ++pool[parent_block_idx].external_ref_cnt;
        pool[child_block_idx].parent_idx = parent_block_idx;
      } else {
        int32_t parent_block_idx = GetFreeBlock();
        pool[parent_block_idx].parent_idx = pool[forked_block_idx].parent_idx;
        pool[forked_block_idx].parent_idx = parent_block_idx;
        pool[child_block_idx].parent_idx = parent_block_idx;
        pool[parent_block_idx].external_ref_cnt = 2;

        auto first_page = pool[forked_block_idx].page_ids.begin();
        auto last_page = pool[forked_block_idx].page_ids.begin() + moved_pages;
        pool[parent_block_idx].page_ids = {first_page, last_page};
        pool[forked_block_idx].page_ids.erase(first_page, last_page);

        pool[parent_block_idx].start_pos = pool[forked_block_idx].start_pos;
        pool[forked_block_idx].start_pos += moved_offset;
        pool[parent_block_idx].seq_length = moved_offset;
        pool[forked_block_idx].seq_length -= moved_offset;

        if (parent_it->second.sliding_window_size != -1 &&
            forked_block_idx == parent_it->second.last_block_idx) {
          KV_CHECK(moved_offset <= parent_it->second.last_block_attn_sink_size) << "fork beyond the attention sink";
          parent_it->second.last_block_attn_sink_size -= moved_offset;
        }
      }
      pool[child_block_idx].start_pos = fork_pos - in_page_offset;
      pool[child_block_idx].seq_length = in_page_offset;

      if (in_page_offset > 0) {
        int32_t src_page_id = pool[forked_block_idx].page_ids[0];
        int32_t tgt_page_id = GetFreePage();
        pool[child_block_idx].page_ids.push_back(tgt_page_id);
        CopySinglePage(src_page_id, tgt_page_id, in_page_offset);
      }
      break;
    }
    seq_map_.insert({child_seq_id, Sequence(&pool, child_block_idx)});
    dirty_aux_data_device_ = true;
  }

  // :772-801
  void EnableSlidingWindowForSeq(int64_t seq_id, int32_t sliding_window_size, int32_t attn_sink_size) {
    KV_CHECK(support_sliding_window_ || support_layer_sliding_window_)
        << "The KV cache does not support sliding window.";
    auto it = seq_map_.find(seq_id);
    KV_CHECK(it != seq_map_.end()) << "The sequence \"" << seq_id << "\" cannot be found in KV cache.";
    KV_CHECK(attn_sink_size >= 0) << "The specified attention sink size is expected to be non negative";
    KV_CHECK(sliding_window_size > 0) << "The specified sliding window size should be positive.";
    KV_CHECK(attn_sink_size < sliding_window_size)
        << "The attn sink size should be less than the sliding window size.";
    KV_CHECK(it->second.sliding_window_size == -1) << "A sequence cannot be enabled twice for sliding window.";
    const Block& last_block = global_block_pool_[it->second.last_block_idx];
    int32_t prefix_length = it->second.seq_length - last_block.seq_length;
    KV_CHECK(prefix_length >= 0) << "negative prefix length";
    it->second.last_block_attn_sink_size = std::max(attn_sink_size - prefix_length, 0);
    it->second.sliding_window_size = sliding_window_size;
  }

  // :803-862
  void PopN(int64_t seq_id, int32_t n) {
    auto it = seq_map_.find(seq_id);
    KV_CHECK(it != seq_map_.end()) << "The sequence \"" << seq_id << "\" cannot be found in KV cache.";
    KV_CHECK(n >= 0) << "The length of popping " << n << " cannot be negative.";
    KV_CHECK(n <= it->second.seq_length)
        << "The sequence only has length " << it->second.seq_length
        << ", while the length of pop is " << n << " which exceeds the whole sequence length.";
    if (n == 0) return;
    std::vector<Block>& pool = global_block_pool_;
    int32_t block_idx = it->second.last_block_idx;
    KV_CHECK(pool[block_idx].external_ref_cnt >= 1) << "block reference count underflow";
    while (block_idx != -1 && pool[block_idx].external_ref_cnt == 1) {
      if (n > pool[block_idx].seq_length) {
        n -= pool[block_idx].seq_length;
        it->second.seq_length -= pool[block_idx].seq_length;
        for (int32_t page_id : pool[block_idx].page_ids) free_page_ids_.push_back(page_id);
        free_block_idx_.push_back(block_idx);
        block_idx = pool[block_idx].parent_idx;
        it->second.last_block_idx = block_idx;
        continue;
      }
      int64_t cur_npage = pool[block_idx].page_ids.size();
      int64_t tgt_npage = (pool[block_idx].seq_length - n + page_size_ - 1) / page_size_;
      while (cur_npage > tgt_npage) {
        free_page_ids_.push_back(pool[block_idx].page_ids.back());
        pool[block_idx].page_ids.pop_back();
        --cur_npage;
      }
      it->second.seq_length -= n;
      pool[block_idx].seq_length -= n;
      n = 0;
      break;
    }
    if (n) {
      // The pop reaches into a shared block: re-fork below the pop point under a temporary id.
      int64_t temp_seq_id = -1 - seq_id;
      KV_CHECK(seq_map_.find(temp_seq_id) == seq_map_.end()) << "temporary sequence id is in use";
      ForkSequence(seq_id, temp_seq_id, it->second.seq_length - n);
      RemoveSequence(seq_id);
      auto temp_it = seq_map_.find(temp_seq_id);
      Sequence moved = temp_it->second;
      seq_map_.erase(temp_it);
      seq_map_.insert({seq_id, moved});
    }
    dirty_aux_data_device_ = true;
  }

  // :866-880
  bool Empty() const {
    return seq_map_.empty() && free_block_idx_.size() == global_block_pool_.size() &&
           free_page_ids_.size() == static_cast<size_t>(num_total_pages_);
  }
  int32_t GetNumAvailablePages() const { return free_page_ids_.size(); }
  int32_t GetTotalSequenceLength() const {
    int32_t total = 0;
    for (const auto& it : seq_map_) total += it.second.seq_length;
    return total;
  }

  // ---------------------------------------------------------------- BeginForward (:884-1212)
  void BeginForward(const int64_t* seq_ids, const int64_t* append_lengths, int64_t batch_size,
                    const int64_t* token_tree_parent_ptr, int64_t n_tree) {
    if (attn_kinds_[0] == TVMKV_ATTN_MLA) {
      KV_CHECK(token_tree_parent_ptr == nullptr) << "Tree attention is not supported yet for MLA";
    }
    cur_batch_size_ = batch_size;
    cur_seq_ids_.assign(seq_ids, seq_ids + batch_size);
    cur_append_lengths_.assign(append_lengths, append_lengths + batch_size);
    std::vector<Block>& pool = global_block_pool_;

    std::vector<Sequence*> sequences;
    std::vector<int32_t> last_block_length_before_append;
    is_decode_request_ = true;
    sequences.reserve(batch_size);
    last_block_length_before_append.reserve(batch_size);
    k_ragged_rope_pos_offset_.clear();
    for (int64_t i = 0; i < batch_size; ++i) {
      auto it = seq_map_.find(seq_ids[i]);
      KV_CHECK(it != seq_map_.end()) << "The sequence \"" << seq_ids[i] << "\" cannot be found in KV cache.";
      sequences.push_back(&it->second);
      last_block_length_before_append.push_back(pool[it->second.last_block_idx].seq_length);
      int k_rope_offset = it->second.seq_length;
      if (!it->second.accepted_indices_committed) {
        k_rope_offset -= static_cast<int>(it->second.token_tree_parent_ptr.size());
      }
      k_ragged_rope_pos_offset_.push_back(k_rope_offset);
      it->second.seq_length += append_lengths[i];
      if (append_lengths[i] != 1) is_decode_request_ = false;
    }
    KV_CHECK(batch_size > 0) << "begin_forward needs at least one sequence";

    std::vector<I32Vec> block_ids_on_depths, trailing_blocks;
    GetBlockIdsOnDepth(sequences, &block_ids_on_depths, &trailing_blocks);
    num_depths_ = std::min(static_cast<int>(block_ids_on_depths.size()), kMaxBlockDepth);

    std::vector<std::vector<std::pair<int32_t, int32_t>>> chunked_block_ids_arr;
    use_decode_kernel_.clear();
    for (int d = 0; d < num_depths_; ++d) {
      bool use_decode_kernel = false;
      chunked_block_ids_arr.push_back(GetChunkedBlockIds(
          block_ids_on_depths[d], /*enable_coalesce=*/d != kMaxBlockDepth - 1, &use_decode_kernel));
      use_decode_kernel_.push_back(use_decode_kernel);
    }
    if (num_depths_ == kMaxBlockDepth) {
      KV_CHECK(static_cast<int64_t>(chunked_block_ids_arr[num_depths_ - 1].size()) == cur_batch_size_)
          << "blocks at the maximum depth must not coalesce";
    }

    append_before_attn_ = !support_sliding_window_ && use_decode_kernel_.back();
    bool has_previous_tree = std::any_of(sequences.begin(), sequences.end(), [](const Sequence* s) {
      return !s->accepted_indices_committed;
    });
    if (has_previous_tree) append_before_attn_ = true;

    if (token_tree_parent_ptr != nullptr) {
      KV_CHECK(!support_sliding_window_) << "Tree attention does not support sliding window.";
      KV_CHECK(rope_mode_ != TVMKV_ROPE_INLINE) << "Tree attention does not support inline RoPE mode.";
      ConstructTokenTreeMask(sequences, token_tree_parent_ptr, n_tree, block_ids_on_depths, trailing_blocks);
    } else {
      for (int64_t i = 0; i < cur_batch_size_; ++i) {
        Sequence* sequence = sequences[i];
        KV_CHECK(sequence->accepted_indices_committed)
            << "The input batch does not form a tree, in which case the sequences in the input "
               "batch are expected to have their accepted tokens token tree nodes committed. "
               "Please invoke CommitAcceptedTokenTreeNodes for sequence "
            << seq_ids[i];
        sequence->is_chain = true;
        sequence->token_tree_parent_ptr.clear();
        sequence->token_tree_node_depths.clear();
      }
      for (int d = 0; d < kMaxBlockDepth; ++d) is_chain_on_depths_[d] = true;
    }

    if (append_before_attn_) {
      for (int64_t i = 0; i < cur_batch_size_; ++i) ReserveAppendLengthInSeq(sequences[i], append_lengths[i]);
    }

    for (int d = 0; d < num_depths_; ++d) {
      I32Vec& qo_indptr_h = qo_indptr_[d];
      I32Vec& page_indptr_h = page_indptr_[d];
      I32Vec& page_indices_h = page_indices_[d];
      I32Vec& page_indptr_sw_h = page_indptr_sw_[d];
      I32Vec& page_indices_sw_h = page_indices_sw_[d];
      I32Vec& last_page_len_h = last_page_len_[d];
      I32Vec& sw_offset_h = sliding_window_offset_[d];
      I32Vec& sink_size_h = sink_size_[d];
      I32Vec& k_rope_h = k_rope_pos_offset_[d];
      I32Vec& k_rope_sw_h = k_rope_pos_offset_sw_[d];
      qo_indptr_h.assign(1, 0);
      page_indptr_h.assign(1, 0);
      page_indptr_sw_h.assign(1, 0);
      page_indices_h.clear();
      page_indices_sw_h.clear();
      last_page_len_h.clear();
      sw_offset_h.clear();
      sink_size_h.clear();
      k_rope_h.clear();
      k_rope_sw_h.clear();
      auto push_sliding_pages = [&](int32_t num_layer_sliding_pages) {
        page_indptr_sw_h.push_back(page_indptr_sw_h.back() + num_layer_sliding_pages);
        for (int64_t i = static_cast<int64_t>(page_indices_h.size()) - num_layer_sliding_pages;
             i < static_cast<int64_t>(page_indices_h.size()); ++i) {
          page_indices_sw_h.push_back(page_indices_h[i]);
        }
      };
      for (int i = 0; i < static_cast<int>(chunked_block_ids_arr[d].size()); ++i) {
        const auto& [block_id, chunk_append_length] = chunked_block_ids_arr[d][i];
        qo_indptr_h.push_back(qo_indptr_h.back() + chunk_append_length);
        if (block_id == -1) {
          page_indptr_h.push_back(page_indptr_h.back());
          page_indptr_sw_h.push_back(page_indptr_sw_h.back());
          last_page_len_h.push_back(0);
          sw_offset_h.push_back(0);
          sink_size_h.push_back(0);
          k_rope_h.push_back(0);
          k_rope_sw_h.push_back(0);
          continue;
        }
        const Block& block = pool[block_id];
        if (d < kMaxBlockDepth - 1) {
          page_indptr_h.push_back(page_indptr_h.back() + block.page_ids.size());
          for (int32_t page_id : block.page_ids) page_indices_h.push_back(page_id);
          push_sliding_pages(std::min(static_cast<int32_t>(block.page_ids.size()),
                                      GetLayerSlidingWindowNumPages(block.seq_length)));
          last_page_len_h.push_back(
              block.seq_length == 0
                  ? 0
                  : (block.seq_length - block.sink_length + block.sliding_window_offset - 1) % page_size_ + 1);
          sw_offset_h.push_back(support_layer_sliding_window_ ? GetLayerSlidingWindowOffset(block.seq_length)
                                                              : block.sliding_window_offset);
          sink_size_h.push_back(block.sink_length);
          k_rope_h.push_back(block.start_pos);
          if (support_layer_sliding_window_) {
            k_rope_sw_h.push_back(static_cast<int32_t>(std::max<int64_t>(
                0, block.start_pos + block.seq_length - layer_sliding_window_size_)));
          }
        } else {
          // Maximum depth: the blocks beyond it are concatenated behind this one.
          int32_t num_pages = static_cast<int32_t>(block.page_ids.size());
          int32_t total_seq_length = block.seq_length;
          int32_t last_block_id = block_id;
          for (int32_t page_id : block.page_ids) page_indices_h.push_back(page_id);
          for (int32_t id : trailing_blocks[i]) {
            const Block& trailing = pool[id];
            for (int32_t page_id : trailing.page_ids) page_indices_h.push_back(page_id);
            num_pages += trailing.page_ids.size();
            total_seq_length += trailing.seq_length;
            last_block_id = id;
          }
          page_indptr_h.push_back(page_indptr_h.back() + num_pages);
          push_sliding_pages(std::min(num_pages, GetLayerSlidingWindowNumPages(total_seq_length)));
          const Block& last_block = pool[last_block_id];
          last_page_len_h.push_back(
              total_seq_length == 0
                  ? 0
                  : (total_seq_length - last_block.sink_length + last_block.sliding_window_offset - 1) % page_size_ + 1);
          sw_offset_h.push_back(support_layer_sliding_window_ ? GetLayerSlidingWindowOffset(total_seq_length)
                                                              : last_block.sliding_window_offset);
          sink_size_h.push_back(last_block.sink_length);
          k_rope_h.push_back(block.start_pos);
          if (support_layer_sliding_window_) {
            k_rope_sw_h.push_back(static_cast<int32_t>(std::max<int64_t>(
                0, block.start_pos + total_seq_length - layer_sliding_window_size_)));
          }
        }
      }
    }

    if (!append_before_attn_) {
      for (int64_t i = 0; i < cur_batch_size_; ++i) ReserveAppendLengthInSeq(sequences[i], append_lengths[i]);
    }

    q_rope_position_map_.clear();
    append_position_map_.clear();
    for (int64_t i = 0; i < cur_batch_size_; ++i) {
      int64_t append_length = append_lengths[i];
      const Block& block = pool[sequences[i]->last_block_idx];
      for (int64_t pos = 0; pos < append_length; ++pos) {
        if (sequences[i]->token_tree_node_depths.empty()) {
          q_rope_position_map_.push_back(k_ragged_rope_pos_offset_[i] + pos);
        } else {
          int64_t offset_in_tree = static_cast<int64_t>(sequences[i]->token_tree_parent_ptr.size()) - append_length;
          KV_CHECK(offset_in_tree >= 0) << "token tree smaller than the append length";
          q_rope_position_map_.push_back(k_ragged_rope_pos_offset_[i] +
                                         sequences[i]->token_tree_node_depths[offset_in_tree + pos]);
        }
        int32_t pos_in_block = block.seq_length - append_length + pos;
        if (last_block_length_before_append[i] + pos < block.sink_length) {
          int32_t offset_in_block = last_block_length_before_append[i] + pos;
          append_position_map_.push_back(block.page_ids[offset_in_block / page_size_] * page_size_ +
                                         offset_in_block % page_size_);
        } else if (pos_in_block < block.sink_length) {
          append_position_map_.push_back(-1);
        } else {
          int32_t offset_in_block = pos_in_block - block.sink_length + block.sliding_window_offset;
          append_position_map_.push_back(block.page_ids[offset_in_block / page_size_] * page_size_ +
                                         offset_in_block % page_size_);
        }
      }
    }
    // The reference builds this indptr lazily in SyncAuxArrayToDevice (:2378-2384).
    cur_append_lengths_indptr_.assign(1, 0);
    for (int64_t i = 0; i < cur_batch_size_; ++i) {
      cur_append_lengths_indptr_.push_back(cur_append_lengths_indptr_.back() + cur_append_lengths_[i]);
    }
    began_forward_ = true;
  }

  void EndForward() {}

  // :1566-1659
  void CommitAcceptedTokenTreeNodes(const int64_t* seq_ids, const int64_t* leaf_indices, int num) {
    std::vector<Sequence*> sequences;
    sequences.reserve(num);
    bool is_chain = true;
    for (int i = 0; i < num; ++i) {
      auto it = seq_map_.find(seq_ids[i]);
      KV_CHECK(it != seq_map_.end()) << "The sequence \"" << seq_ids[i] << "\" cannot be found in KV cache.";
      sequences.push_back(&it->second);
      is_chain = it->second.is_chain;
      KV_CHECK(leaf_indices[i] == -1 || !it->second.accepted_indices_committed)
          << "The accepted nodes of sequence " << seq_ids[i] << " are already committed.";
      KV_CHECK(leaf_indices[i] >= -1) << "Invalid tree index " << leaf_indices[i] << " which is less than -1";
      KV_CHECK(leaf_indices[i] < static_cast<int64_t>(it->second.token_tree_parent_ptr.size()))
          << "Invalid tree index " << leaf_indices[i]
          << " which is larger than or equals to the append length "
          << it->second.token_tree_parent_ptr.size() << " of the sequence";
    }
    if (!is_chain) {
      commit_copy_length_indptr_.assign(1, 0);
      commit_copy_src_pos_.clear();
      commit_copy_dst_pos_.clear();
      for (int i = 0; i < num; ++i) {
        if (leaf_indices[i] == -1) {
          commit_copy_length_indptr_.push_back(commit_copy_length_indptr_.back());
          continue;
        }
        std::vector<int32_t> path_on_tree;
        int node = leaf_indices[i];
        while (node != -1) {
          path_on_tree.push_back(node);
          node = sequences[i]->token_tree_parent_ptr[node];
        }
        KV_CHECK(static_cast<int>(path_on_tree.size()) == sequences[i]->token_tree_node_depths[leaf_indices[i]] + 1)
            << "token tree depth mismatch";
        std::vector<int32_t> copy_dst_pos_in_seq(path_on_tree.size());
        std::iota(copy_dst_pos_in_seq.rbegin(), copy_dst_pos_in_seq.rend(), 0);
        while (!path_on_tree.empty() && path_on_tree.back() == copy_dst_pos_in_seq.back()) {
          path_on_tree.pop_back();
          copy_dst_pos_in_seq.pop_back();
        }
        std::reverse(path_on_tree.begin(), path_on_tree.end());
        std::reverse(copy_dst_pos_in_seq.begin(), copy_dst_pos_in_seq.end());
        for (int p = 0; p < static_cast<int>(path_on_tree.size()); ++p) {
          commit_copy_src_pos_.push_back(append_position_map_[cur_append_lengths_indptr_[i] + path_on_tree[p]]);
          commit_copy_dst_pos_.push_back(append_position_map_[cur_append_lengths_indptr_[i] + copy_dst_pos_in_seq[p]]);
        }
        commit_copy_length_indptr_.push_back(commit_copy_length_indptr_.back() + path_on_tree.size());
      }
      CompactKVCopy();
    }
    for (int i = 0; i < num; ++i) {
      int64_t length_to_pop =
          cur_append_lengths_[i] -
          (leaf_indices[i] != -1 ? (sequences[i]->token_tree_node_depths[leaf_indices[i]] + 1) : 0);
      PopN(cur_seq_ids_[i], length_to_pop);
      // PopN may have re-created the map entry: look the sequence up again before touching it.
      Sequence& seq = seq_map_.at(cur_seq_ids_[i]);
      seq.accepted_indices_committed = true;
      seq.token_tree_parent_ptr.clear();
      seq.token_tree_node_depths.clear();
    }
  }

  // ---------------------------------------------------------------- attention (device)
  // :1303-1402
  void AttentionWithFusedQKV(int64_t layer_id, const void* qkv, int64_t qkv_rows, void* out,
                             int64_t out_rows, double sm_scale) {
    RequireDevice();
    int64_t local_layer_id = CheckLayer(layer_id);
    KV_CHECK(attn_kinds_[layer_id] == TVMKV_ATTN_MHA || attn_kinds_[layer_id] == TVMKV_ATTN_MHA_SLIDING)
        << "attention_with_fused_qkv needs an MHA layer";
    KV_CHECK(out_rows == qkv_rows) << "qkv and output must have the same number of rows";
    int64_t total_seq_length = TotalAppendLength();
    KV_CHECK(total_seq_length <= qkv_rows)
        << "qkv has " << qkv_rows << " rows, fewer than the batch appends (" << total_seq_length << ")";
    KV_CHECK(total_seq_length <= prefill_chunk_size_)
        << "the batch appends " << total_seq_length << " tokens, more than prefill_chunk_size "
        << prefill_chunk_size_;
    ComputeStreamWaitForCopyStream();
    KV_CHECK(!dirty_aux_data_device_) << "auxiliary data is not synchronised";

    // A chunked-prefill step of a plain cache in two launches: k is rotated and the new k / v rows go
    // into their page slots (part 2 without q, part 3), then one pass over the cached and the new
    // tokens that reads the queries from qkv and rotates them itself (parts 2 and 5).
    if (OnePassPrefillApplies(layer_id)) {
      Launch(tvmkv_fused_rope_append(qkv, q_rope_position_map_view_.ptr, /*q=*/nullptr, temp_k_, temp_v_,
                                     rope_mode_ == TVMKV_ROPE_NORMAL, pages_[local_layer_id],
                                     append_position_map_view_.ptr, total_seq_length, num_qo_heads_, num_kv_heads_,
                                     qk_head_dim_, num_total_pages_, page_size_, rotary_scale_, rotary_theta_,
                                     compute_stream_));
      Launch(tvmkv_batch_prefill_cached_and_new_kv_fused_q(
          qkv, q_rope_position_map_view_.ptr, rope_mode_ == TVMKV_ROPE_NORMAL, rotary_scale_, rotary_theta_,
          cur_append_length_indptr_view_.ptr, temp_k_, temp_v_, pages_[local_layer_id], page_indptr_view_[0].ptr,
          page_indices_view_[0].ptr, length_info_view_[0].ptr, out, merged_lse_, sm_scale, cur_batch_size_,
          total_seq_length, page_indices_view_[0].size, num_total_pages_, num_qo_heads_, num_kv_heads_, qk_head_dim_,
          page_size_, compute_stream_));
      RecordComputeEvent();
      return;
    }
    // Part 2: split fused qkv, RoPE on q/k.  Part 3 with it, in one launch, when the new k / v rows may
    // go into their page slots before attention: always when the reference appends first, and in a
    // cache without sliding windows also when the reference appends afterwards (:1396-1401) -- there
    // the step's page tables cover only the tokens cached before it, the new slots lie on pages
    // that were free or beyond their sequence's cached tokens, and no kernel of the step reads them.
    // A sliding-window cache frees pages while it reserves the step's slots and hands them out again
    // in the same step (:1935-1992, :2004-2044): a new token's slot can be one that the step's page
    // table of another sequence still attends to, so there the rows are written after attention.
    const bool append_early = append_before_attn_ || !support_sliding_window_;
    if (append_early) {
      Launch(tvmkv_fused_rope_append(qkv, q_rope_position_map_view_.ptr, temp_q_, temp_k_, temp_v_,
                                     rope_mode_ == TVMKV_ROPE_NORMAL, pages_[local_layer_id],
                                     append_position_map_view_.ptr, total_seq_length, num_qo_heads_, num_kv_heads_,
                                     qk_head_dim_, num_total_pages_, page_size_, rotary_scale_, rotary_theta_,
                                     compute_stream_));
    } else {
      Launch(tvmkv_fused_rope(qkv, q_rope_position_map_view_.ptr, temp_q_, temp_k_, temp_v_,
                              rope_mode_ == TVMKV_ROPE_NORMAL, total_seq_length, num_qo_heads_, num_kv_heads_,
                              qk_head_dim_, rotary_scale_, rotary_theta_, compute_stream_));
    }
    // Part 5: attention.
    AttentionInternal(layer_id, temp_q_, temp_k_, temp_v_, out, total_seq_length, sm_scale);
    // Part 6: append after attention (:1396-1401).
    if (!append_early) {
      Launch(tvmkv_kv_cache_transpose_append(pages_[local_layer_id], temp_k_, temp_v_, append_position_map_view_.ptr,
                                             total_seq_length, num_total_pages_, num_kv_heads_, page_size_,
                                             qk_head_dim_, compute_stream_));
    }
    RecordComputeEvent();
  }

  // :1487-1525: attention of this step's queries against the K/V of another layer (the new tokens'
  // rows are handed in; nothing is appended).
  void AttentionWithSharedKV(int64_t source_layer_id, const void* q, const void* k, const void* v, void* o,
                             int64_t rows, double sm_scale) {
    RequireDevice();
    CheckLayer(source_layer_id);
    KV_CHECK(attn_kinds_[source_layer_id] == TVMKV_ATTN_MHA || attn_kinds_[source_layer_id] == TVMKV_ATTN_MHA_SLIDING)
        << "Querying K/V from another logical layer is only supported for MHA caches.";
    int64_t total_seq_length = TotalAppendLength();
    KV_CHECK(rows == total_seq_length)
        << "attention_with_shared_kv expects " << total_seq_length << " rows, got " << rows;
    ComputeStreamWaitForCopyStream();
    KV_CHECK(!dirty_aux_data_device_) << "auxiliary data is not synchronised";
    AttentionInternal(source_layer_id, q, k, v, o, total_seq_length, sm_scale);
    RecordComputeEvent();
  }

  // :1404-1445
  void SelfAttention(int64_t layer_id, const void* q, const void* k, const void* v, void* o, float* lse,
                     int64_t rows, int k_heads, int qk_dim, int v_dim, double sm_scale) {
    RequireDevice();
    CheckLayer(layer_id);
    int64_t total_seq_length = TotalAppendLength();
    KV_CHECK(rows == total_seq_length) << "self_attention expects " << total_seq_length << " rows, got " << rows;
    ComputeStreamWaitForCopyStream();
    KV_CHECK(!dirty_aux_data_device_) << "auxiliary data is not synchronised";
    if (!is_chain_on_depths_[0]) {
      KV_CHECK(attn_kinds_[layer_id] == TVMKV_ATTN_MHA) << "Tree attn not able for MLA for now.";
      KV_CHECK(k_heads == num_kv_heads_ && qk_dim == qk_head_dim_ && v_dim == v_head_dim_)
          << "self_attention: k/v shapes do not match the cache";
      MHASelfAttnInternal(q, k, v, o, lse, total_seq_length, sm_scale);
      RecordComputeEvent();
      return;
    }
    int rotary = attn_kinds_[layer_id] == TVMKV_ATTN_MHA ? (rope_mode_ == TVMKV_ROPE_INLINE) : 0;
    Launch(tvmkv_batch_prefill_ragged_kv(q, cur_append_length_indptr_view_.ptr, k, v,
                                         cur_append_length_indptr_view_.ptr, q_rope_position_map_view_.ptr,
                                         k_ragged_rope_pos_offset_view_.ptr, o, lse, /*causal=*/1, rotary,
                                         rotary_scale_, rotary_theta_, sm_scale, cur_batch_size_,
                                         total_seq_length, num_qo_heads_, k_heads, qk_dim, v_dim,
                                         compute_stream_));
    RecordComputeEvent();
  }

  // :1447-1485
  void CrossAttention(int64_t layer_id, const void* q, void* o, float* lse, int64_t rows, double sm_scale) {
    RequireDevice();
    int64_t local_layer_id = CheckLayer(layer_id);
    int64_t total_seq_length = TotalAppendLength();
    KV_CHECK(rows == total_seq_length) << "cross_attention expects " << total_seq_length << " rows, got " << rows;
    ComputeStreamWaitForCopyStream();
    KV_CHECK(!dirty_aux_data_device_) << "auxiliary data is not synchronised";
    if (attn_kinds_[layer_id] == TVMKV_ATTN_MHA) {
      MHACrossAttnInternal(local_layer_id, q, o, lse, total_seq_length, sm_scale, /*is_first_kernel=*/true,
                           /*causal=*/false);
    } else {
      MLACrossAttnInternal(local_layer_id, q, o, lse, total_seq_length, sm_scale);
    }
    RecordComputeEvent();
  }

  // :1527-1551
  void AppendMLAKV(int64_t layer_id, const void* kv, int64_t rows) {
    RequireDevice();
    int64_t local_layer_id = CheckLayer(layer_id);
    KV_CHECK(attn_kinds_[layer_id] == TVMKV_ATTN_MLA) << "append_mla_kv needs an MLA layer";
    int64_t total_seq_length = TotalAppendLength();
    KV_CHECK(rows <= total_seq_length) << "kv has more rows than the batch appends";
    ComputeStreamWaitForCopyStream();
    KV_CHECK(!dirty_aux_data_device_) << "auxiliary data is not synchronised";
    Launch(tvmkv_kv_cache_transpose_append_mla(pages_[local_layer_id], kv, append_position_map_view_.ptr, rows,
                                               num_total_pages_, page_size_, qk_head_dim_, compute_stream_));
    RecordComputeEvent();
  }

  // :1553-1559
  void MergeAttnOutputInplace(void* o_self, float* lse_self, const void* o_cross, const float* lse_cross,
                              int64_t rows, int heads, int dim) {
    RequireDevice();
    Launch(tvmkv_merge_state_inplace(o_self, lse_self, o_cross, lse_cross, rows, heads, dim, compute_stream_));
  }

  // :1661-1667
  AuxView GetQueryPositions() {
    RequireDevice();
    ComputeStreamWaitForCopyStream();
    KV_CHECK(!dirty_aux_data_device_) << "auxiliary data is not synchronised";
    return q_rope_position_map_view_;
  }

  // Slot ids of every cached token of a sequence (:1698-1710).
  I32Vec PositionMapOf(int64_t seq_id, int64_t start_pos, int64_t end_pos) {
    auto it = seq_map_.find(seq_id);
    KV_CHECK(it != seq_map_.end()) << "The sequence \"" << seq_id << "\" cannot be found in KV cache.";
    const Sequence& seq = it->second;
    KV_CHECK(start_pos >= 0) << "DebugGetKV does not accept negative start_pos " << start_pos;
    KV_CHECK(end_pos <= seq.seq_length) << "DebugGetKV does not accept out-of-range end_pos";
    KV_CHECK(start_pos < end_pos) << "DebugGetKV does not accept \"start_pos >= end_pos\"";
    I32Vec map;
    map.reserve(seq.seq_length);
    for (int32_t block_id : seq.GetBlockTrace(global_block_pool_)) {
      const Block& block = global_block_pool_[block_id];
      for (int i = 0; i < block.seq_length; ++i) {
        int32_t offset = i < block.sink_length ? i : i - block.sink_length + block.sliding_window_offset;
        map.push_back(block.page_ids[offset / page_size_] * page_size_ + offset % page_size_);
      }
    }
    return I32Vec(map.begin() + start_pos, map.begin() + end_pos);
  }

  // :1669-1766
  void DebugGetKV(int64_t seq_id, int64_t start_pos, int64_t end_pos, void* k_data, void* v_data, bool mla) {
    RequireDevice();
    I32Vec map = PositionMapOf(seq_id, start_pos, end_pos);
    HIP_CHECK(hipSetDevice(device_));
    int32_t* map_dev = nullptr;
    HIP_CHECK(hipMalloc(&map_dev, map.size() * sizeof(int32_t)));
    try {
      HIP_CHECK(hipMemcpyAsync(map_dev, map.data(), map.size() * sizeof(int32_t), hipMemcpyHostToDevice,
                               compute_stream_));
      for (int64_t layer = 0; layer < num_layers_; ++layer) {
        int64_t kind = attn_kinds_[layer + layer_id_begin_offset_];
        if (mla) {
          KV_CHECK(kind == TVMKV_ATTN_MLA) << "Only MLA is supported for DebugGetKVMLA";
          Launch(tvmkv_kv_cache_debug_get_kv_mla(pages_[layer], map_dev, k_data, layer, map.size(),
                                                 num_total_pages_, page_size_, qk_head_dim_, compute_stream_));
        } else {
          KV_CHECK(kind == TVMKV_ATTN_MHA) << "Only MHA is supported for DebugGetKV";
          Launch(tvmkv_kv_cache_debug_get_kv(pages_[layer], map_dev, k_data, v_data, layer, map.size(),
                                             num_total_pages_, num_kv_heads_, page_size_, qk_head_dim_,
                                             compute_stream_));
        }
      }
      HIP_CHECK(hipStreamSynchronize(compute_stream_));
    } catch (...) {
      (void)hipFree(map_dev);
      throw;
    }
    HIP_CHECK(hipFree(map_dev));
  }

  // ---------------------------------------------------------------- introspection
  const I32Vec* GetAux(const std::string& name, int depth) {
    static const std::map<std::string, int> per_depth = {
        {"qo_indptr", 0}, {"page_indptr", 1}, {"page_indices", 2}, {"page_indptr_sliding_window", 3},
        {"page_indices_sliding_window", 4}, {"last_page_len", 5}, {"sliding_window_offset", 6},
        {"sink_size", 7}, {"k_rope_pos_offset", 8}, {"k_rope_pos_offset_sliding_window", 9},
        {"tree_attn_mask", 10}, {"tree_attn_mn_indptr", 11}};
    auto it = per_depth.find(name);
    if (it != per_depth.end()) {
      KV_CHECK(depth >= 0 && depth < kMaxBlockDepth) << "depth " << depth << " out of range";
      I32Vec* arrays[] = {qo_indptr_, page_indptr_, page_indices_, page_indptr_sw_, page_indices_sw_,
                          last_page_len_, sliding_window_offset_, sink_size_, k_rope_pos_offset_,
                          k_rope_pos_offset_sw_, tree_attn_mask_, tree_attn_mn_indptr_};
      return &arrays[it->second][depth];
    }
    if (name == "q_rope_position_map") return &q_rope_position_map_;
    if (name == "append_position_map") return &append_position_map_;
    if (name == "cur_append_lengths_indptr") return &cur_append_lengths_indptr_;
    if (name == "k_ragged_rope_pos_offset") return &k_ragged_rope_pos_offset_;
    if (name == "commit_copy_length_indptr") return &commit_copy_length_indptr_;
    if (name == "commit_copy_src_pos") return &commit_copy_src_pos_;
    if (name == "commit_copy_dst_pos") return &commit_copy_dst_pos_;
    KV_CHECK(false) << "unknown auxiliary array \"" << name << "\"";
    return nullptr;
  }

  void GetFlags(int64_t* flags, int n) const {
    int64_t all[9] = {num_depths_,
                      append_before_attn_,
                      is_decode_request_,
                      use_decode_kernel_.size() > 0 ? use_decode_kernel_[0] : 0,
                      use_decode_kernel_.size() > 1 ? use_decode_kernel_[1] : 0,
                      is_chain_on_depths_[0],
                      is_chain_on_depths_[1],
                      num_total_pages_,
                      rope_mode_};
    for (int i = 0; i < n && i < 9; ++i) flags[i] = all[i];
  }

  std::vector<int64_t> DumpState() const {
    std::vector<int64_t> out;
    out.push_back(free_page_ids_.size());
    out.insert(out.end(), free_page_ids_.begin(), free_page_ids_.end());
    out.push_back(free_block_idx_.size());
    out.insert(out.end(), free_block_idx_.begin(), free_block_idx_.end());
    out.push_back(global_block_pool_.size());
    for (const Block& b : global_block_pool_) {
      out.push_back(b.page_ids.size());
      out.insert(out.end(), b.page_ids.begin(), b.page_ids.end());
      out.insert(out.end(), {b.seq_length, b.start_pos, b.sink_length, b.sliding_window_offset, b.parent_idx,
                             b.external_ref_cnt});
    }
    std::map<int64_t, const Sequence*> ordered;
    for (const auto& it : seq_map_) ordered[it.first] = &it.second;
    out.push_back(ordered.size());
    for (const auto& it : ordered) {
      out.insert(out.end(), {it.first, it.second->last_block_idx, it.second->seq_length,
                             it.second->sliding_window_size, it.second->last_block_attn_sink_size});
    }
    return out;
  }

  const std::vector<int64_t>& CopyLog() const { return copy_log_; }
  void* Pages(int64_t local_layer, int64_t* bytes) {
    RequireDevice();
    KV_CHECK(local_layer >= 0 && local_layer < num_layers_) << "layer " << local_layer << " out of range";
    *bytes = PageBytes(local_layer);
    return pages_[local_layer];
  }
  void SetStream(hipStream_t stream) { compute_stream_ = stream; }

  std::vector<int64_t> scratch_i64_;  // storage behind pointers returned through the C ABI

 private:
  // ---------------------------------------------------------------- pool helpers
  void ResetPool() {
    seq_map_.clear();
    free_page_ids_.clear();
    for (int64_t page_id = num_total_pages_ - 1; page_id >= 0; --page_id) free_page_ids_.push_back(page_id);
    global_block_pool_.clear();
    free_block_idx_.clear();
    copy_log_.clear();
    began_forward_ = false;
  }

  // :1777-1783
  int32_t GetFreePage() {
    KV_CHECK(!free_page_ids_.empty()) << "The KV cache is full. No page can be allocated.";
    int32_t page_id = free_page_ids_.back();
    free_page_ids_.pop_back();
    return page_id;
  }

  // :1786-1798
  int32_t GetFreeBlock() {
    if (!free_block_idx_.empty()) {
      int32_t block_idx = free_block_idx_.back();
      free_block_idx_.pop_back();
      global_block_pool_[block_idx].Reset();
      return block_idx;
    }
    int32_t block_idx = global_block_pool_.size();
    global_block_pool_.push_back(Block(block_idx));
    return block_idx;
  }

  // attn_utils.h:243-279
  void GetBlockIdsOnDepth(const std::vector<Sequence*>& sequences, std::vector<I32Vec>* block_ids_on_depths,
                          std::vector<I32Vec>* trailing_block_traces) const {
    int64_t num_depths = 0;
    std::vector<I32Vec> seq_block_traces;
    for (const Sequence* seq : sequences) {
      I32Vec trace = seq->GetBlockTrace(global_block_pool_);
      if (static_cast<int>(trace.size()) <= kMaxBlockDepth) {
        num_depths = std::max<int64_t>(num_depths, trace.size());
        seq_block_traces.push_back(std::move(trace));
        trailing_block_traces->push_back({});
      } else {
        seq_block_traces.emplace_back(trace.begin(), trace.begin() + kMaxBlockDepth);
        trailing_block_traces->emplace_back(trace.begin() + kMaxBlockDepth, trace.end());
        num_depths = std::max<int64_t>(num_depths, kMaxBlockDepth);
      }
    }
    for (int d = 0; d < num_depths; ++d) {
      I32Vec block_ids;
      for (const I32Vec& trace : seq_block_traces) {
        block_ids.push_back(d < static_cast<int>(trace.size()) ? trace[d] : -1);
      }
      block_ids_on_depths->push_back(std::move(block_ids));
    }
  }

  // attn_utils.h:293-332
  std::vector<std::pair<int32_t, int32_t>> GetChunkedBlockIds(const I32Vec& block_ids, bool enable_coalesce,
                                                              bool* use_decode_kernel_out) const {
    const std::vector<Block>& pool = global_block_pool_;
    std::vector<std::pair<int32_t, int32_t>> uncoalesced, coalesced;
    int cur_block_id = block_ids[0];
    int chunk_append_length = cur_append_lengths_[0];
    int page_counter_coalesced = 0;
    int page_counter_uncoalesced = block_ids[0] != -1 ? pool[block_ids[0]].page_ids.size() : 0;
    for (int i = 1; i < static_cast<int>(block_ids.size()); ++i) {
      if (block_ids[i] != -1) page_counter_uncoalesced += pool[block_ids[i]].page_ids.size();
      uncoalesced.emplace_back(block_ids[i - 1], cur_append_lengths_[i - 1]);
      if (block_ids[i] == cur_block_id) {
        chunk_append_length += cur_append_lengths_[i];
      } else {
        coalesced.emplace_back(cur_block_id, chunk_append_length);
        if (cur_block_id != -1) page_counter_coalesced += pool[cur_block_id].page_ids.size();
        cur_block_id = block_ids[i];
        chunk_append_length = cur_append_lengths_[i];
      }
    }
    uncoalesced.emplace_back(block_ids.back(), cur_append_lengths_.back());
    coalesced.emplace_back(cur_block_id, chunk_append_length);
    if (cur_block_id != -1) page_counter_coalesced += pool[cur_block_id].page_ids.size();
    double coalesce_ratio =
        page_counter_coalesced > 0 ? 1.0 * page_counter_uncoalesced / page_counter_coalesced : 0.0;
    bool use_decode_kernel = is_decode_request_ && coalesce_ratio < 32;
    *use_decode_kernel_out = use_decode_kernel;
    return (use_decode_kernel || !enable_coalesce) ? uncoalesced : coalesced;
  }

  // :289-303
  int32_t GetLayerSlidingWindowOffset(int64_t seq_length) const {
    if (seq_length <= layer_sliding_window_size_) return 0;
    return static_cast<int32_t>((seq_length - layer_sliding_window_size_) % page_size_);
  }
  int32_t GetLayerSlidingWindowNumPages(int64_t seq_length) const {
    if (seq_length == 0) return 0;
    int64_t window_length = std::min(seq_length, layer_sliding_window_size_);
    return static_cast<int32_t>((GetLayerSlidingWindowOffset(seq_length) + window_length + page_size_ - 1) /
                                page_size_);
  }

  // :1800-1928
  void ConstructTokenTreeMask(const std::vector<Sequence*>& sequences, const int64_t* token_tree_parent_ptr,
                              int64_t n_tree, const std::vector<I32Vec>& block_ids_on_depths,
                              const std::vector<I32Vec>& trailing_blocks) {
    auto check_for_sequence = [&](int seq_i, int depth) -> bool {
      if (!append_before_attn_) return true;
      return block_ids_on_depths[depth][seq_i] == sequences[seq_i]->last_block_idx ||
             (depth + 1 == kMaxBlockDepth && !trailing_blocks[seq_i].empty());
    };
    for (int d = 0; d < num_depths_; ++d) {
      I32Vec& mn_indptr = tree_attn_mn_indptr_[d];
      I32Vec& mask = tree_attn_mask_[d];
      std::vector<bool> seq_in_current_depth(cur_batch_size_, false);
      mn_indptr.assign(1, 0);
      mask.clear();
      for (int k = 0; k < kMaxBlockDepth; ++k) is_chain_on_depths_[k] = true;
      bool is_chain = true;
      int64_t offset = 0;
      for (int64_t i = 0; i < cur_batch_size_; ++i) {
        int64_t append_length = cur_append_lengths_[i];
        seq_in_current_depth[i] = check_for_sequence(i, d);
        if (!seq_in_current_depth[i]) {
          mn_indptr.push_back(mn_indptr.back());
          offset += append_length;
          continue;
        }
        KV_CHECK(static_cast<int64_t>(sequences[i]->token_tree_parent_ptr.size()) <=
                 global_block_pool_[sequences[i]->last_block_idx].seq_length)
            << "The token tree size is larger than the sequence length of the last block.";
        KV_CHECK(offset + append_length <= n_tree) << "Invalid token tree size.";
        for (int64_t j = 0; j < append_length; ++j) {
          sequences[i]->token_tree_parent_ptr.push_back(token_tree_parent_ptr[offset + j]);
        }
        offset += append_length;
        KV_CHECK(static_cast<int>(sequences[i]->token_tree_parent_ptr.size()) <= kTreeAttnMaxTreeSize)
            << "The tree size is " << append_length << " which exceeds the maximum tree size limit "
            << kTreeAttnMaxTreeSize;
        mn_indptr.push_back(mn_indptr.back() + sequences[i]->token_tree_parent_ptr.size());
      }
      KV_CHECK(n_tree == offset) << "Invalid token tree size. The sum of \"append_lengths\" is " << offset
                                 << " while there are " << n_tree << " elements in \"token_tree_parent_ptr\".";
      for (int64_t i = 0; i < cur_batch_size_; ++i) {
        if (!seq_in_current_depth[i]) continue;
        Sequence* seq = sequences[i];
        int64_t tree_size = seq->token_tree_parent_ptr.size();
        std::vector<int32_t> depth;
        depth.reserve(tree_size);
        seq->is_chain = true;
        seq->accepted_indices_committed = false;
        std::unordered_map<int, std::vector<int>> tree_parent_to_children;
        std::vector<int> tree_roots;
        for (int n = 0; n < tree_size; ++n) {
          int32_t parent = seq->token_tree_parent_ptr[n];
          KV_CHECK(parent < n) << "Invalid token tree. The parent of node " << n << " in tree " << i << " is "
                               << parent << ", which is not smaller than " << n;
          KV_CHECK(parent >= -1) << "Invalid token tree. The parent of node " << n << " in tree " << i
                                 << " is " << parent;
          if (parent != n - 1) {
            seq->is_chain = false;
            is_chain = false;
          }
          tree_parent_to_children[parent].push_back(n);
          if (parent != -1) {
            depth.push_back(depth[parent] + 1);
          } else {
            depth.push_back(0);
            tree_roots.push_back(n);
          }
        }
        std::vector<std::pair<int, int>> tree_order(tree_size);
        int order = 0;
        std::function<int(int)> tree_dfs = [&](int node) -> int {
          tree_order[node].first = order++;
          int upper_bound = tree_order[node].first + 1;
          for (int child : tree_parent_to_children[node]) upper_bound = std::max(upper_bound, tree_dfs(child));
          tree_order[node].second = upper_bound;
          return upper_bound;
        };
        for (int root : tree_roots) tree_dfs(root);
        for (int n = 0; n < tree_size; ++n) {
          mask.push_back(tree_order[n].first);
          mask.push_back(tree_order[n].second);
        }
        seq->token_tree_node_depths = std::move(depth);
      }
      is_chain_on_depths_[d] = is_chain;
      if (!append_before_attn_) break;
    }
  }

  // :1935-1992
  void SlideWindowForSequence(Sequence* seq) {
    if (seq->sliding_window_size == -1 || !support_sliding_window_) return;
    if (seq->seq_length <= seq->sliding_window_size) return;
    int32_t length_to_slide = seq->seq_length - seq->sliding_window_size;
    Block& block = global_block_pool_[seq->last_block_idx];
    if (seq->last_block_attn_sink_size > 0 && block.sink_length == 0) {
      KV_CHECK(block.sliding_window_offset == 0) << "sliding window offset set before the sink";
      block.sink_length = seq->last_block_attn_sink_size;
      block.sliding_window_offset = seq->last_block_attn_sink_size;
    }
    int32_t num_sink_pages = (block.sink_length + page_size_ - 1) / page_size_;
    int32_t page_idx_after_sliding = (block.sliding_window_offset + length_to_slide) / page_size_;
    int32_t page_start_offset_after_sliding = (block.sliding_window_offset + length_to_slide) % page_size_;
    while (page_idx_after_sliding > num_sink_pages) {
      if (block.page_ids[num_sink_pages] != kTempPageId) free_page_ids_.push_back(block.page_ids[num_sink_pages]);
      block.page_ids.erase(block.page_ids.begin() + num_sink_pages);
      --page_idx_after_sliding;
    }
    KV_CHECK(page_idx_after_sliding == num_sink_pages - 1 || page_idx_after_sliding == num_sink_pages)
        << "sliding window left an unexpected first page";
    seq->seq_length = seq->sliding_window_size;
    block.seq_length -= length_to_slide;
    block.sliding_window_offset = page_idx_after_sliding * page_size_ + page_start_offset_after_sliding;
    KV_CHECK(block.seq_length >= block.sink_length) << "block shorter than its attention sink";
    KV_CHECK(block.sliding_window_offset >= block.sink_length) << "sliding window overlaps the attention sink";
    KV_CHECK((block.sliding_window_offset + (block.seq_length - block.sink_length) + page_size_ - 1) / page_size_ ==
             static_cast<int64_t>(block.page_ids.size()))
        << "page count does not match the slid window";
  }

  // :2004-2044
  void ReserveAppendLengthInSeq(Sequence* seq, int64_t append_length) {
    Block& block = global_block_pool_[seq->last_block_idx];
    KV_CHECK(append_length > 0) << "Append with length 0 is not allowed.";
    KV_CHECK(block.external_ref_cnt == 1)
        << "The block is " << block.external_ref_cnt - 1
        << "-time referenced by other blocks, thus cannot accept new KV values.";
    int64_t cur_npage = block.page_ids.size();
    int64_t tgt_npage =
        (block.seq_length - block.sink_length + block.sliding_window_offset + append_length + page_size_ - 1) /
        page_size_;
    for (int64_t page_idx = cur_npage; page_idx < tgt_npage; ++page_idx) {
      if (free_page_ids_.empty() && seq->sliding_window_size != -1 && support_sliding_window_) {
        block.page_ids.push_back(kTempPageId);
      } else {
        block.page_ids.push_back(GetFreePage());
      }
    }
    block.seq_length += append_length;
    SlideWindowForSequence(seq);
    if (support_sliding_window_) {
      for (int i = 0; i < static_cast<int>(block.page_ids.size()); ++i) {
        if (block.page_ids[i] == kTempPageId) block.page_ids[i] = GetFreePage();
      }
    }
    dirty_aux_data_device_ = true;
  }

  // ---------------------------------------------------------------- device layer
  void RequireDevice() const {
    if (device_ < 0) throw Error(TVMKV_ENODEVICE, "this cache was created host-only (device_id = -1)");
  }
  static void Launch(int rc) {
    if (rc != TVMKV_OK) throw Error(rc, tvmkv_last_error());
  }
  int64_t CheckLayer(int64_t layer_id) const {
    int64_t local_layer_id = layer_id - layer_id_begin_offset_;
    KV_CHECK(local_layer_id >= 0 && local_layer_id < num_layers_) << "layer id " << layer_id << " out of range";
    return local_layer_id;
  }
  int64_t TotalAppendLength() const {
    KV_CHECK(began_forward_) << "begin_forward has not been called";
    return std::accumulate(cur_append_lengths_.begin(), cur_append_lengths_.end(), int64_t{0});
  }
  int64_t PageBytes(int64_t local_layer) const {
    int64_t kind = attn_kinds_[local_layer + layer_id_begin_offset_];
    // GetKVCacheShape, attn_utils.h:74-87
    if (kind == TVMKV_ATTN_MLA) return num_total_pages_ * page_size_ * qk_head_dim_ * 2;
    return num_total_pages_ * 2 * num_kv_heads_ * page_size_ * qk_head_dim_ * 2;
  }

  void InitDevice() {
    int count = 0;
    HIP_CHECK(hipGetDeviceCount(&count));
    KV_CHECK(device_ < count) << "device " << device_ << " does not exist (" << count << " visible)";
    HIP_CHECK(hipSetDevice(device_));
    try {
      pages_.assign(num_layers_, nullptr);
      for (int64_t l = 0; l < num_layers_; ++l) HIP_CHECK(hipMalloc(&pages_[l], PageBytes(l)));
      bool has_mha = false;
      for (int64_t kind : attn_kinds_) has_mha |= (kind != TVMKV_ATTN_MLA);
      if (has_mha) {
        HIP_CHECK(hipMalloc(&temp_q_, prefill_chunk_size_ * num_qo_heads_ * qk_head_dim_ * 2));
        HIP_CHECK(hipMalloc(&temp_k_, prefill_chunk_size_ * num_kv_heads_ * qk_head_dim_ * 2));
        HIP_CHECK(hipMalloc(&temp_v_, prefill_chunk_size_ * num_kv_heads_ * v_head_dim_ * 2));
      }
      HIP_CHECK(hipMalloc(&temp_out_, prefill_chunk_size_ * num_qo_heads_ * v_head_dim_ * 2));
      HIP_CHECK(hipMalloc(&temp_lse_, prefill_chunk_size_ * num_qo_heads_ * sizeof(float)));
      HIP_CHECK(hipMalloc(&merged_lse_, prefill_chunk_size_ * num_qo_heads_ * sizeof(float)));
      // Capacity of the merged auxiliary buffer: every array of SyncAuxArrayToDevice at its
      // maximum size, each start rounded up to 16 bytes.
      int64_t r = reserved_num_seqs_, p = num_total_pages_, c = prefill_chunk_size_;
      aux_capacity_ = kMaxBlockDepth * (4 * (r + 1) + 2 * p + 8 * r + kTreeAttnMaxTreeSize * 2 * r) + 3 * c +
                      2 * (r + 1) + 4 * 64;
      for (int i = 0; i < 2; ++i) {
        HIP_CHECK(hipMalloc(&aux_device_[i], aux_capacity_ * sizeof(int32_t)));
        HIP_CHECK(hipHostMalloc(&aux_staging_[i], aux_capacity_ * sizeof(int32_t), hipHostMallocDefault));
        HIP_CHECK(hipEventCreateWithFlags(&aux_copied_[i], hipEventDisableTiming));
      HIP_CHECK(hipEventCreateWithFlags(&aux_consumed_[i], hipEventDisableTiming));
      }
      // token-tree commit: copy_length_indptr + (2, copies) positions (attn_utils.h:1010-1021)
      commit_capacity_ = (r + 1 + 3) / 4 * 4 + 2 * std::min<int64_t>(kTreeAttnMaxTreeSize * r, c) + 4;
      HIP_CHECK(hipMalloc(&commit_device_, commit_capacity_ * sizeof(int32_t)));
      HIP_CHECK(hipHostMalloc(&commit_staging_, commit_capacity_ * sizeof(int32_t), hipHostMallocDefault));
      HIP_CHECK(hipEventCreateWithFlags(&commit_copied_, hipEventDisableTiming));
      HIP_CHECK(hipStreamCreateWithFlags(&copy_stream_, hipStreamNonBlocking));
      HIP_CHECK(hipEventCreateWithFlags(&compute_done_, hipEventDisableTiming));
    } catch (...) {
      ReleaseDevice();
      throw;
    }
  }

  void ReleaseDevice() {
    if (device_ < 0) return;
    (void)hipSetDevice(device_);
    for (void* p : pages_) (void)hipFree(p);
    pages_.clear();
    for (void** p : {&temp_q_, &temp_k_, &temp_v_, &temp_out_}) {
      (void)hipFree(*p);
      *p = nullptr;
    }
    (void)hipFree(temp_lse_);
    (void)hipFree(merged_lse_);
    temp_lse_ = merged_lse_ = nullptr;
    for (int i = 0; i < 2; ++i) {
      (void)hipFree(aux_device_[i]);
      if (aux_staging_[i]) (void)hipHostFree(aux_staging_[i]);
      if (aux_copied_[i]) (void)hipEventDestroy(aux_copied_[i]);
      if (aux_consumed_[i]) (void)hipEventDestroy(aux_consumed_[i]);
      aux_device_[i] = aux_staging_[i] = nullptr;
      aux_copied_[i] = aux_consumed_[i] = nullptr;
      aux_consumed_recorded_[i] = false;
    }
    (void)hipFree(commit_device_);
    if (commit_staging_) (void)hipHostFree(commit_staging_);
    if (commit_copied_) (void)hipEventDestroy(commit_copied_);
    commit_device_ = commit_staging_ = nullptr;
    commit_copied_ = nullptr;
    commit_staging_used_ = false;
    if (copy_stream_) (void)hipStreamDestroy(copy_stream_);
    if (compute_done_) (void)hipEventDestroy(compute_done_);
    copy_stream_ = nullptr;
    compute_done_ = nullptr;
  }

  void RecordComputeEvent() {
    HIP_CHECK(hipEventRecord(compute_done_, compute_stream_));
    compute_event_recorded_ = true;
    // the kernels enqueued so far are the last readers of the auxiliary buffer in use
    HIP_CHECK(hipEventRecord(aux_consumed_[aux_slot_], compute_stream_));
    aux_consumed_recorded_[aux_slot_] = true;
  }

  // :721-734.  The copy runs on the copy stream, after everything enqueued on the compute
  // stream so far (the source page may have been written by the previous step's append).
  void CopySinglePage(int32_t src_page_id, int32_t tgt_page_id, int64_t copy_length) {
    copy_log_.insert(copy_log_.end(), {src_page_id, tgt_page_id, copy_length});
    if (device_ < 0) return;
    HIP_CHECK(hipSetDevice(device_));
    if (compute_event_recorded_) HIP_CHECK(hipStreamWaitEvent(copy_stream_, compute_done_, 0));
    for (int64_t layer = 0; layer < num_layers_; ++layer) {
      if (attn_kinds_[layer + layer_id_begin_offset_] == TVMKV_ATTN_MLA) {
        Launch(tvmkv_copy_single_page_mla(pages_[layer], src_page_id, tgt_page_id, copy_length, num_total_pages_,
                                          page_size_, qk_head_dim_, copy_stream_));
      } else {
        Launch(tvmkv_copy_single_page(pages_[layer], src_page_id, tgt_page_id, copy_length, num_total_pages_,
                                      num_kv_heads_, page_size_, qk_head_dim_, copy_stream_));
      }
    }
    copy_stream_has_work_ = true;
  }

  // :736-770
  void CompactKVCopy() {
    int total_copy_length = commit_copy_length_indptr_.back();
    KV_CHECK(total_copy_length >= 0) << "negative copy length";
    if (total_copy_length == 0 || device_ < 0) return;
    HIP_CHECK(hipSetDevice(device_));
    // one upload: [copy_length_indptr (batch + 1), padded to 16 bytes | src positions | dst positions]
    const int64_t n_indptr = static_cast<int64_t>(commit_copy_length_indptr_.size());
    const int64_t pos_begin = (n_indptr + 3) / 4 * 4;
    KV_CHECK(pos_begin + 2 * static_cast<int64_t>(total_copy_length) <= commit_capacity_)
        << "token-tree commit copies " << total_copy_length << " slots, more than the cache was sized for";
    // the staging buffer is reused: wait until the previous commit's upload has read it
    if (commit_staging_used_) HIP_CHECK(hipEventSynchronize(commit_copied_));
    int32_t* staging = static_cast<int32_t*>(commit_staging_);
    std::memcpy(staging, commit_copy_length_indptr_.data(), n_indptr * sizeof(int32_t));
    std::memcpy(staging + pos_begin, commit_copy_src_pos_.data(), total_copy_length * sizeof(int32_t));
    std::memcpy(staging + pos_begin + total_copy_length, commit_copy_dst_pos_.data(),
                total_copy_length * sizeof(int32_t));
    int32_t* device = static_cast<int32_t*>(commit_device_);
    // after the attention kernels of the step that computed on these slots
    if (compute_event_recorded_) HIP_CHECK(hipStreamWaitEvent(copy_stream_, compute_done_, 0));
    HIP_CHECK(hipMemcpyAsync(device, staging, (pos_begin + 2 * total_copy_length) * sizeof(int32_t),
                             hipMemcpyHostToDevice, copy_stream_));
    HIP_CHECK(hipEventRecord(commit_copied_, copy_stream_));
    commit_staging_used_ = true;
    for (int64_t layer = 0; layer < num_layers_; ++layer) {
      Launch(tvmkv_compact_kv_copy(pages_[layer], device, device + pos_begin, cur_batch_size_, total_copy_length,
                                   num_total_pages_, num_kv_heads_, page_size_, qk_head_dim_, copy_stream_));
    }
    // The next BeginForward's first kernel waits for the copy stream (paged_kv_cache.cc:767-769).
    copy_stream_has_work_ = true;
  }

  // A chunked-prefill step of a plain cache (one depth, no sliding window, no inline RoPE, no token
  // tree) can run as one pass over the cached and the new tokens.
  bool OnePassPrefillApplies(int64_t layer_id) const {
    return !append_before_attn_ && num_depths_ == 1 && is_chain_on_depths_[0] && !use_decode_kernel_[0] &&
           page_indices_view_[0].size > 0 && !support_sliding_window_ && attn_kinds_[layer_id] == TVMKV_ATTN_MHA &&
           rope_mode_ != TVMKV_ROPE_INLINE && qk_head_dim_ == v_head_dim_ &&
           (qk_head_dim_ == 64 || qk_head_dim_ == 128);
  }

  // :2161-2180
  void AttentionInternal(int64_t layer_id, const void* q, const void* k, const void* v, void* output,
                         int64_t total_seq_length, double sm_scale) {
    int64_t local_layer_id = layer_id - layer_id_begin_offset_;
    // A chunked-prefill step of a plain cache (one depth, no sliding window, no inline RoPE, no
    // token tree): self-attention over the new tokens, attention over the cached ones and their
    // merge (:2169-2177, :2285-2292) in one pass over both key sets.
    if (OnePassPrefillApplies(layer_id)) {
      Launch(tvmkv_batch_prefill_cached_and_new_kv(q, cur_append_length_indptr_view_.ptr, k, v, pages_[local_layer_id],
                                                   page_indptr_view_[0].ptr, page_indices_view_[0].ptr,
                                                   length_info_view_[0].ptr, output, merged_lse_, sm_scale,
                                                   cur_batch_size_, total_seq_length, page_indices_view_[0].size,
                                                   num_total_pages_, num_qo_heads_, num_kv_heads_, qk_head_dim_,
                                                   page_size_, compute_stream_));
      return;
    }
    bool is_first_kernel = true;
    if (!append_before_attn_) {
      is_first_kernel = false;
      MHASelfAttnInternal(q, k, v, output, merged_lse_, total_seq_length, sm_scale);
    }
    bool self_attn_computed = !is_first_kernel;
    bool cross_attn_computed = MHACrossAttnInternal(
        local_layer_id, q, output, merged_lse_, total_seq_length, sm_scale, is_first_kernel,
        /*causal=*/!append_before_attn_ && attn_kinds_[layer_id] == TVMKV_ATTN_MHA_SLIDING);
    KV_CHECK(self_attn_computed || cross_attn_computed)
        << "Both self-attention and cross-attention are not computed.";
  }

  // :2182-2203
  void MHASelfAttnInternal(const void* q, const void* k, const void* v, void* o, float* lse, int64_t total_seq_length,
                           double sm_scale) {
    if (is_chain_on_depths_[0]) {
      Launch(tvmkv_batch_prefill_ragged_kv(q, cur_append_length_indptr_view_.ptr, k, v,
                                           cur_append_length_indptr_view_.ptr, q_rope_position_map_view_.ptr,
                                           k_ragged_rope_pos_offset_view_.ptr, o, lse, /*causal=*/1,
                                           rope_mode_ == TVMKV_ROPE_INLINE, rotary_scale_, rotary_theta_, sm_scale,
                                           cur_batch_size_, total_seq_length, num_qo_heads_, num_kv_heads_,
                                           qk_head_dim_, v_head_dim_, compute_stream_));
    } else {
      // the batch forms token trees
      KV_CHECK(tree_attn_mask_view_[0].ptr != nullptr && tree_attn_mn_indptr_view_[0].ptr != nullptr)
          << "token-tree mask is not on the device";
      KV_CHECK(qk_head_dim_ == v_head_dim_) << "tree attention needs equal qk and v head dims";
      Launch(tvmkv_batch_tree_attn(q, cur_append_length_indptr_view_.ptr, k, v, cur_append_length_indptr_view_.ptr,
                                   q_rope_position_map_view_.ptr, tree_attn_mn_indptr_view_[0].ptr,
                                   tree_attn_mask_view_[0].ptr, o, lse, rope_mode_ == TVMKV_ROPE_INLINE,
                                   rotary_scale_, rotary_theta_, sm_scale, cur_batch_size_, total_seq_length,
                                   num_qo_heads_, num_kv_heads_, qk_head_dim_, compute_stream_));
    }
  }

  // :2216-2299
  bool MHACrossAttnInternal(int64_t local_layer_id, const void* q, void* o, float* lse, int64_t total_seq_length,
                            double sm_scale, bool is_first_kernel, bool causal) {
    KV_CHECK(num_depths_ >= 1) << "The number of effective depths must be greater or equal to 1.";
    bool sliding_layer = attn_kinds_[local_layer_id + layer_id_begin_offset_] == TVMKV_ATTN_MHA_SLIDING;
    int sliding_window = (support_sliding_window_ || sliding_layer) ? 1 : 0;
    bool cross_attn_computed = false;
    for (int d = 0; d < num_depths_; ++d) {
      if (page_indices_view_[d].size == 0) continue;
      void* attn_output = is_first_kernel ? o : temp_out_;
      float* attn_lse = is_first_kernel ? lse : temp_lse_;
      const AuxView& page_indptr = sliding_layer ? page_indptr_sw_view_[d] : page_indptr_view_[d];
      const AuxView& page_indices = sliding_layer ? page_indices_sw_view_[d] : page_indices_view_[d];
      const AuxView& length_info = sliding_layer ? layer_sw_length_info_view_[d] : length_info_view_[d];
      const AuxView& k_rope_pos = sliding_layer ? k_rope_pos_offset_sw_view_[d] : k_rope_pos_offset_view_[d];
      double rotary_theta = sliding_layer ? 10000 : rotary_theta_;
      double rotary_scale = sliding_layer ? 1 : rotary_scale_;
      int rotary_mode = rope_mode_ == TVMKV_ROPE_INLINE;
      if (append_before_attn_ && !is_chain_on_depths_[d]) {
        KV_CHECK(tree_attn_mask_view_[d].ptr != nullptr && tree_attn_mn_indptr_view_[d].ptr != nullptr)
            << "token-tree mask is not on the device";
        Launch(tvmkv_tree_attn_paged_kv(q, qo_indptr_view_[d].ptr, pages_[local_layer_id], page_indptr.ptr,
                                        page_indices.ptr, length_info.ptr, k_rope_pos.ptr,
                                        q_rope_position_map_view_.ptr, attn_output, attn_lse, rotary_mode,
                                        rotary_scale, rotary_theta, sm_scale, tree_attn_mn_indptr_view_[d].ptr,
                                        tree_attn_mask_view_[d].ptr, qo_indptr_view_[d].size - 1, total_seq_length,
                                        page_indices.size, num_total_pages_, num_qo_heads_, num_kv_heads_,
                                        qk_head_dim_, page_size_, sliding_window, compute_stream_));
      } else if (use_decode_kernel_[d]) {
        Launch(tvmkv_batch_decode_paged_kv(q, pages_[local_layer_id], page_indptr.ptr, page_indices.ptr,
                                           length_info.ptr, k_rope_pos.ptr, q_rope_position_map_view_.ptr,
                                           attn_output, attn_lse, rotary_mode, rotary_scale, rotary_theta, sm_scale,
                                           qo_indptr_view_[d].size - 1, page_indices.size, num_total_pages_,
                                           num_qo_heads_, num_kv_heads_, qk_head_dim_, page_size_, sliding_window,
                                           compute_stream_));
      } else if (!is_first_kernel) {
        // The prefill kernel merges its state into (o, lse) in its epilogue: one launch for the
        // kernel and the merge of :2285-2292, and no temporary output.
        Launch(tvmkv_batch_prefill_paged_kv_merge(q, qo_indptr_view_[d].ptr, pages_[local_layer_id], page_indptr.ptr,
                                                  page_indices.ptr, length_info.ptr, k_rope_pos.ptr,
                                                  q_rope_position_map_view_.ptr, o, lse, causal, rotary_mode,
                                                  rotary_scale, rotary_theta, sm_scale, qo_indptr_view_[d].size - 1,
                                                  total_seq_length, page_indices.size, num_total_pages_,
                                                  num_qo_heads_, num_kv_heads_, qk_head_dim_, page_size_,
                                                  sliding_window, layer_sliding_window_size_, compute_stream_));
        cross_attn_computed = true;
        continue;
      } else {
        Launch(tvmkv_batch_prefill_paged_kv(q, qo_indptr_view_[d].ptr, pages_[local_layer_id], page_indptr.ptr,
                                            page_indices.ptr, length_info.ptr, k_rope_pos.ptr,
                                            q_rope_position_map_view_.ptr, attn_output, attn_lse, causal,
                                            rotary_mode, rotary_scale, rotary_theta, sm_scale,
                                            qo_indptr_view_[d].size - 1, total_seq_length, page_indices.size,
                                            num_total_pages_, num_qo_heads_, num_kv_heads_, qk_head_dim_, page_size_,
                                            sliding_window, layer_sliding_window_size_, compute_stream_));
      }
      if (!is_first_kernel) {
        Launch(tvmkv_merge_state_inplace(o, lse, temp_out_, temp_lse_, total_seq_length, num_qo_heads_, v_head_dim_,
                                         compute_stream_));
      } else {
        is_first_kernel = false;
      }
      cross_attn_computed = true;
    }
    return cross_attn_computed;
  }

  // :2302-2335
  bool MLACrossAttnInternal(int64_t local_layer_id, const void* q, void* o, float* lse, int64_t total_seq_length,
                            double sm_scale) {
    KV_CHECK(num_depths_ >= 1) << "The number of effective depths must be greater or equal to 1.";
    bool is_first_kernel = true;
    for (int d = 0; d < num_depths_; ++d) {
      if (page_indices_view_[d].size == 0) continue;
      void* attn_output = is_first_kernel ? o : temp_out_;
      float* attn_lse = is_first_kernel ? lse : temp_lse_;
      KV_CHECK(is_chain_on_depths_[d]) << "Tree attn not able for MLA for now.";
      Launch(tvmkv_batch_prefill_paged_kv_mla(q, qo_indptr_view_[d].ptr, pages_[local_layer_id],
                                              page_indptr_view_[d].ptr, page_indices_view_[d].ptr,
                                              length_info_view_[d].ptr, attn_output, attn_lse, /*causal=*/0,
                                              sm_scale, qo_indptr_view_[d].size - 1, total_seq_length,
                                              page_indices_view_[d].size, num_total_pages_, num_qo_heads_,
                                              v_head_dim_, qk_head_dim_ - v_head_dim_, page_size_, compute_stream_));
      if (!is_first_kernel) {
        Launch(tvmkv_merge_state_inplace(o, lse, temp_out_, temp_lse_, total_seq_length, num_qo_heads_, v_head_dim_,
                                         compute_stream_));
      } else {
        is_first_kernel = false;
      }
    }
    return !is_first_kernel;
  }

  // :2338-2366
  void ComputeStreamWaitForCopyStream() {
    if (!dirty_aux_data_device_ && !copy_stream_has_work_) return;
    HIP_CHECK(hipSetDevice(device_));
    if (dirty_aux_data_device_) SyncAuxArrayToDevice();
    // Everything on the copy stream (aux upload, fork page copies) happens before the kernels.
    hipEvent_t ev = aux_copied_[aux_slot_];
    HIP_CHECK(hipEventRecord(ev, copy_stream_));
    HIP_CHECK(hipStreamWaitEvent(compute_stream_, ev, 0));
    copy_stream_has_work_ = false;
  }

  // :2373-2525 with the merged-buffer manager of attn_utils.h:812-1062 -- one upload per step.
  void SyncAuxArrayToDevice() {
    KV_CHECK(began_forward_) << "begin_forward has not been called";
    int64_t total_append_length = cur_append_lengths_indptr_.back();
    KV_CHECK(total_append_length == static_cast<int64_t>(append_position_map_.size()))
        << "append position map does not cover the batch";
    aux_slot_ ^= 1;
    // The staging buffer of this slot was last read by the upload two steps ago.
    if (aux_slot_used_[aux_slot_]) HIP_CHECK(hipEventSynchronize(aux_copied_[aux_slot_]));
    int32_t* staging = static_cast<int32_t*>(aux_staging_[aux_slot_]);
    int32_t* device = static_cast<int32_t*>(aux_device_[aux_slot_]);
    int64_t cursor = 0;
    auto put = [&](const int32_t* data, int64_t n) -> AuxView {
      KV_CHECK(cursor + n <= aux_capacity_) << "auxiliary buffer overflow (" << cursor + n << " > " << aux_capacity_
                                            << "): batch or append length beyond the configured limits";
      if (n) std::memcpy(staging + cursor, data, n * sizeof(int32_t));
      AuxView view{device + cursor, n};
      cursor = (cursor + n + 3) / 4 * 4;  // 16-byte aligned starts (attn_utils.h:1048-1052)
      return view;
    };
    auto put_vec = [&](const I32Vec& v) { return put(v.data(), v.size()); };
    auto put_length_info = [&](int d) -> AuxView {
      // (3, n): last_page_len; sliding_window_offset; sink_size (attn_utils.h:483-495)
      int64_t n = last_page_len_[d].size();
      AuxView first = put(last_page_len_[d].data(), n);
      cursor = (first.ptr - device) + n;
      put(sliding_window_offset_[d].data(), n);
      cursor = (first.ptr - device) + 2 * n;
      put(sink_size_[d].data(), n);
      return AuxView{first.ptr, 3 * n};
    };
    q_rope_position_map_view_ = put_vec(q_rope_position_map_);
    for (int d = 0; d < num_depths_; ++d) qo_indptr_view_[d] = put_vec(qo_indptr_[d]);
    for (int d = 0; d < num_depths_; ++d) page_indptr_view_[d] = put_vec(page_indptr_[d]);
    for (int d = 0; d < num_depths_; ++d) page_indices_view_[d] = put_vec(page_indices_[d]);
    if (support_layer_sliding_window_) {
      for (int d = 0; d < num_depths_; ++d) page_indptr_sw_view_[d] = put_vec(page_indptr_sw_[d]);
      for (int d = 0; d < num_depths_; ++d) page_indices_sw_view_[d] = put_vec(page_indices_sw_[d]);
    }
    for (int d = 0; d < num_depths_; ++d) {
      length_info_view_[d] = support_sliding_window_ ? put_length_info(d) : put_vec(last_page_len_[d]);
      if (support_layer_sliding_window_) layer_sw_length_info_view_[d] = put_length_info(d);
    }
    for (int d = 0; d < num_depths_; ++d) {
      k_rope_pos_offset_view_[d] = put_vec(k_rope_pos_offset_[d]);
      if (support_layer_sliding_window_) k_rope_pos_offset_sw_view_[d] = put_vec(k_rope_pos_offset_sw_[d]);
    }
    cur_append_length_indptr_view_ = put_vec(cur_append_lengths_indptr_);
    k_ragged_rope_pos_offset_view_ = put_vec(k_ragged_rope_pos_offset_);
    append_position_map_view_ = put_vec(append_position_map_);
    for (int d = 0; d < num_depths_; ++d) {
      if (!is_chain_on_depths_[d]) {
        tree_attn_mask_view_[d] = put_vec(tree_attn_mask_[d]);
        tree_attn_mn_indptr_view_[d] = put_vec(tree_attn_mn_indptr_[d]);
      }
    }
    if (cursor) {
      // A host that runs ahead of the device must not overwrite arrays that kernels of the step
      // two uploads ago, still queued on the compute stream, have yet to read.
      if (aux_consumed_recorded_[aux_slot_]) HIP_CHECK(hipStreamWaitEvent(copy_stream_, aux_consumed_[aux_slot_], 0));
      HIP_CHECK(hipMemcpyAsync(device, staging, cursor * sizeof(int32_t), hipMemcpyHostToDevice, copy_stream_));
    }
    aux_slot_used_[aux_slot_] = true;
    dirty_aux_data_device_ = false;
  }

  // ---------------------------------------------------------------- configuration
  int64_t page_size_, num_layers_, layer_id_begin_offset_, layer_id_end_offset_;
  int64_t num_qo_heads_, num_kv_heads_, qk_head_dim_, v_head_dim_;
  int64_t num_total_pages_ = 0, prefill_chunk_size_;
  bool support_sliding_window_ = false, support_layer_sliding_window_ = false;
  int64_t layer_sliding_window_size_ = 1024;
  std::vector<int64_t> attn_kinds_;
  int rope_mode_ = TVMKV_ROPE_NORMAL;
  double rotary_scale_, rotary_theta_;
  int64_t reserved_num_seqs_;

  // ---------------------------------------------------------------- pool
  std::vector<int32_t> free_page_ids_;
  std::unordered_map<int64_t, Sequence> seq_map_;
  std::vector<Block> global_block_pool_;
  std::vector<int32_t> free_block_idx_;
  std::vector<int64_t> copy_log_;

  // ---------------------------------------------------------------- current batch
  bool dirty_aux_data_device_ = false;
  bool began_forward_ = false;
  int64_t cur_batch_size_ = 0;
  std::vector<int64_t> cur_seq_ids_, cur_append_lengths_;
  bool is_chain_on_depths_[kMaxBlockDepth];
  int num_depths_ = 0;
  bool append_before_attn_ = false;
  std::vector<bool> use_decode_kernel_;
  bool is_decode_request_ = false;

  I32Vec qo_indptr_[kMaxBlockDepth], page_indptr_[kMaxBlockDepth], page_indices_[kMaxBlockDepth];
  I32Vec page_indptr_sw_[kMaxBlockDepth], page_indices_sw_[kMaxBlockDepth];
  I32Vec last_page_len_[kMaxBlockDepth], sliding_window_offset_[kMaxBlockDepth], sink_size_[kMaxBlockDepth];
  I32Vec k_rope_pos_offset_[kMaxBlockDepth], k_rope_pos_offset_sw_[kMaxBlockDepth];
  I32Vec tree_attn_mask_[kMaxBlockDepth], tree_attn_mn_indptr_[kMaxBlockDepth];
  I32Vec k_ragged_rope_pos_offset_, q_rope_position_map_, append_position_map_, cur_append_lengths_indptr_;
  I32Vec commit_copy_length_indptr_, commit_copy_src_pos_, commit_copy_dst_pos_;

  // ---------------------------------------------------------------- device
  int device_;
  hipStream_t compute_stream_ = nullptr;
  hipStream_t copy_stream_ = nullptr;
  hipEvent_t compute_done_ = nullptr;
  bool compute_event_recorded_ = false;
  bool copy_stream_has_work_ = false;
  std::vector<void*> pages_;
  void *temp_q_ = nullptr, *temp_k_ = nullptr, *temp_v_ = nullptr, *temp_out_ = nullptr;
  float *temp_lse_ = nullptr, *merged_lse_ = nullptr;
  int64_t aux_capacity_ = 0;
  void* aux_device_[2] = {nullptr, nullptr};
  void* aux_staging_[2] = {nullptr, nullptr};
  hipEvent_t aux_copied_[2] = {nullptr, nullptr};
  hipEvent_t aux_consumed_[2] = {nullptr, nullptr};  // recorded on the compute stream behind a slot's last readers
  bool aux_consumed_recorded_[2] = {false, false};
  bool aux_slot_used_[2] = {false, false};
  int aux_slot_ = 0;
  int64_t commit_capacity_ = 0;
  void* commit_device_ = nullptr;
  void* commit_staging_ = nullptr;
  hipEvent_t commit_copied_ = nullptr;
  bool commit_staging_used_ = false;
  AuxView q_rope_position_map_view_, append_position_map_view_, cur_append_length_indptr_view_,
      k_ragged_rope_pos_offset_view_;
  AuxView qo_indptr_view_[kMaxBlockDepth], page_indptr_view_[kMaxBlockDepth], page_indices_view_[kMaxBlockDepth],
      page_indptr_sw_view_[kMaxBlockDepth], page_indices_sw_view_[kMaxBlockDepth],
      length_info_view_[kMaxBlockDepth], layer_sw_length_info_view_[kMaxBlockDepth],
      k_rope_pos_offset_view_[kMaxBlockDepth], k_rope_pos_offset_sw_view_[kMaxBlockDepth],
      tree_attn_mask_view_[kMaxBlockDepth], tree_attn_mn_indptr_view_[kMaxBlockDepth];
};

}  // namespace tvmkv

// =========================================================================== C ABI
struct tvmkv_cache {
  std::unique_ptr<tvmkv::PagedKVCache> impl;
};

extern "C" {

const char* tvmkv_last_error(void) { return tvmkv::g_last_error.c_str(); }
const char* tvmkv_version(void) { return "tvmkv 0.1 (gfx950)"; }

int tvmkv_cache_create(const int64_t* cache_config, int32_t n_config, const int64_t* layer_indptr,
                       int32_t n_layer_indptr, int64_t num_qo_heads, int64_t num_kv_heads, int64_t qk_head_dim,
                       int64_t v_head_dim, const int64_t* attn_kinds, int32_t n_attn_kinds,
                       int32_t enable_kv_transfer, int32_t rope_mode, double rope_scale, double rope_theta,
                       int32_t dtype_bits, int32_t device_id, tvmkv_cache** out) {
  KV_API_BEGIN();
  KV_CHECK(out != nullptr) << "out must not be NULL";
  KV_CHECK(n_config == 5 || n_config == 6)
      << "KV cache config must contain five legacy fields and an optional per-layer sliding window size.";
  // One worker, one group: layer_indptr = [begin, end] (paged_kv_cache.cc:2541-2551).
  KV_CHECK(n_layer_indptr == 2) << "layer_indptr must have num_groups + 1 = 2 entries";
  KV_CHECK(rope_mode >= 0 && rope_mode <= 2) << "invalid rope mode " << rope_mode;
  auto cache = std::make_unique<tvmkv_cache>();
  cache->impl = std::make_unique<tvmkv::PagedKVCache>(
      cache_config, n_config, layer_indptr[0], layer_indptr[1], num_qo_heads, num_kv_heads, qk_head_dim,
      v_head_dim, std::vector<int64_t>(attn_kinds, attn_kinds + n_attn_kinds), enable_kv_transfer != 0, rope_mode,
      rope_scale, rope_theta, dtype_bits, device_id);
  *out = cache.release();
  KV_API_END();
}

void tvmkv_cache_destroy(tvmkv_cache* cache) { delete cache; }

#define KV_CACHE_FN(body) \
  KV_API_BEGIN();         \
  KV_CHECK(cache != nullptr) << "cache is NULL"; \
  body;                   \
  KV_API_END();

int tvmkv_cache_set_stream(tvmkv_cache* cache, void* stream) {
  KV_CACHE_FN(cache->impl->SetStream(static_cast<hipStream_t>(stream)));
}
int tvmkv_kv_state_clear(tvmkv_cache* cache) { KV_CACHE_FN(cache->impl->Clear()); }
int tvmkv_kv_state_add_sequence(tvmkv_cache* cache, int64_t seq_id) {
  KV_CACHE_FN(cache->impl->AddSequence(seq_id));
}
int tvmkv_kv_state_remove_sequence(tvmkv_cache* cache, int64_t seq_id) {
  KV_CACHE_FN(cache->impl->RemoveSequence(seq_id));
}
int tvmkv_kv_state_fork_sequence(tvmkv_cache* cache, int64_t parent_seq_id, int64_t child_seq_id,
                                 int64_t fork_pos) {
  KV_CACHE_FN(cache->impl->ForkSequence(parent_seq_id, child_seq_id, fork_pos));
}
int tvmkv_kv_state_popn(tvmkv_cache* cache, int64_t seq_id, int32_t n) { KV_CACHE_FN(cache->impl->PopN(seq_id, n)); }
int tvmkv_kv_state_begin_forward(tvmkv_cache* cache, const int64_t* seq_ids, const int64_t* append_lengths,
                                 int32_t batch_size, const int64_t* token_tree_parent_ptr, int32_t n_tree) {
  KV_CACHE_FN(cache->impl->BeginForward(seq_ids, append_lengths, batch_size, token_tree_parent_ptr, n_tree));
}
int tvmkv_kv_state_end_forward(tvmkv_cache* cache) { KV_CACHE_FN(cache->impl->EndForward()); }

int tvmkv_attention_kv_cache_enable_sliding_window_for_seq(tvmkv_cache* cache, int64_t seq_id,
                                                           int32_t sliding_window_size, int32_t attn_sink_size) {
  KV_CACHE_FN(cache->impl->EnableSlidingWindowForSeq(seq_id, sliding_window_size, attn_sink_size));
}
int tvmkv_attention_kv_cache_commit_accepted_token_tree_nodes(tvmkv_cache* cache, const int64_t* seq_ids,
                                                              const int64_t* leaf_indices, int32_t n) {
  KV_CACHE_FN(cache->impl->CommitAcceptedTokenTreeNodes(seq_ids, leaf_indices, n));
}
int tvmkv_attention_kv_cache_empty(tvmkv_cache* cache, int32_t* out) { KV_CACHE_FN(*out = cache->impl->Empty()); }
int tvmkv_attention_kv_cache_get_num_available_pages(tvmkv_cache* cache, int32_t* out) {
  KV_CACHE_FN(*out = cache->impl->GetNumAvailablePages());
}
int tvmkv_attention_kv_cache_get_total_sequence_length(tvmkv_cache* cache, int32_t* out) {
  KV_CACHE_FN(*out = cache->impl->GetTotalSequenceLength());
}
int tvmkv_attention_kv_cache_get_query_positions(tvmkv_cache* cache, const int32_t** device_ptr, int64_t* length) {
  KV_CACHE_FN({
    tvmkv::AuxView v = cache->impl->GetQueryPositions();
    *device_ptr = v.ptr;
    *length = v.size;
  });
}
int tvmkv_attention_kv_cache_attention_with_fused_qkv(tvmkv_cache* cache, int64_t layer_id, double sm_scale,
                                                      const void* qkv, int64_t qkv_rows, void* out,
                                                      int64_t out_rows) {
  KV_CACHE_FN(cache->impl->AttentionWithFusedQKV(layer_id, qkv, qkv_rows, out, out_rows, sm_scale));
}
int tvmkv_attention_kv_cache_self_attention(tvmkv_cache* cache, int64_t layer_id, double sm_scale, const void* q,
                                            const void* k, const void* v, void* o, float* lse, int64_t rows,
                                            int32_t k_heads, int32_t qk_dim, int32_t v_dim) {
  KV_CACHE_FN(cache->impl->SelfAttention(layer_id, q, k, v, o, lse, rows, k_heads, qk_dim, v_dim, sm_scale));
}
int tvmkv_attention_kv_cache_cross_attention(tvmkv_cache* cache, int64_t layer_id, double sm_scale, const void* q,
                                             void* o, float* lse, int64_t rows) {
  KV_CACHE_FN(cache->impl->CrossAttention(layer_id, q, o, lse, rows, sm_scale));
}
int tvmkv_attention_kv_cache_attention_with_shared_kv(tvmkv_cache* cache, int64_t source_layer_id, double sm_scale,
                                                      const void* q, const void* current_k, const void* current_v,
                                                      void* o, int64_t rows) {
  KV_CACHE_FN(cache->impl->AttentionWithSharedKV(source_layer_id, q, current_k, current_v, o, rows, sm_scale));
}
int tvmkv_attention_kv_cache_append_mla_kv(tvmkv_cache* cache, int64_t layer_id, const void* kv, int64_t rows) {
  KV_CACHE_FN(cache->impl->AppendMLAKV(layer_id, kv, rows));
}
int tvmkv_attention_kv_cache_merge_attn_output_inplace(tvmkv_cache* cache, void* o_self, float* lse_self,
                                                       const void* o_cross, const float* lse_cross, int64_t rows,
                                                       int32_t heads, int32_t dim) {
  KV_CACHE_FN(cache->impl->MergeAttnOutputInplace(o_self, lse_self, o_cross, lse_cross, rows, heads, dim));
}
int tvmkv_attention_kv_cache_debug_get_kv(tvmkv_cache* cache, int64_t seq_id, int64_t start_pos, int64_t end_pos,
                                          void* k_data, void* v_data) {
  KV_CACHE_FN(cache->impl->DebugGetKV(seq_id, start_pos, end_pos, k_data, v_data, /*mla=*/false));
}
int tvmkv_attention_kv_cache_debug_get_kv_mla(tvmkv_cache* cache, int64_t seq_id, int64_t start_pos,
                                              int64_t end_pos, void* kv_data) {
  KV_CACHE_FN(cache->impl->DebugGetKV(seq_id, start_pos, end_pos, kv_data, nullptr, /*mla=*/true));
}

int tvmkv_cache_get_aux(tvmkv_cache* cache, const char* name, int32_t depth, const int32_t** data, int64_t* size) {
  KV_CACHE_FN({
    const tvmkv::I32Vec* v = cache->impl->GetAux(name, depth);
    *data = v->data();
    *size = v->size();
  });
}
int tvmkv_cache_get_flags(tvmkv_cache* cache, int64_t* flags, int32_t n_flags) {
  KV_CACHE_FN(cache->impl->GetFlags(flags, n_flags));
}
int tvmkv_cache_dump_state(tvmkv_cache* cache, int64_t* buf, int64_t cap, int64_t* needed) {
  KV_CACHE_FN({
    std::vector<int64_t> s = cache->impl->DumpState();
    *needed = s.size();
    KV_CHECK(static_cast<int64_t>(s.size()) <= cap) << "buffer too small: need " << s.size() << " elements";
    std::memcpy(buf, s.data(), s.size() * sizeof(int64_t));
  });
}
int tvmkv_cache_get_copy_log(tvmkv_cache* cache, const int64_t** triples, int64_t* n_triples) {
  KV_CACHE_FN({
    *triples = cache->impl->CopyLog().data();
    *n_triples = cache->impl->CopyLog().size() / 3;
  });
}
int tvmkv_cache_get_pages(tvmkv_cache* cache, int64_t local_layer, void** device_ptr, int64_t* num_bytes) {
  KV_CACHE_FN(*device_ptr = cache->impl->Pages(local_layer, num_bytes));
}

}  // extern "C"
