// The paged KV cache object: device resources and kernel orchestration on top of the host
// bookkeeping of kv_bookkeeping.h.  Verbs, order of checks and error texts follow the reference's
// PagedAttentionKVCacheObj (src/runtime/vm/paged_kv_cache.cc); the device layer is this library's
// own: the step's auxiliary arrays are written by the bookkeeper straight into one of two pinned
// staging buffers and reach the device with a single copy per step on a private copy stream, and
// every kernel is a launcher from include/tvmkv.h.
#include <algorithm>
#include <cstring>
#include <memory>
#include <vector>

#include "common.h"
#include "kv_bookkeeping.h"
#include "runtime_support.h"
#include "typed_kernels.h"

namespace tvmkv {

namespace {
thread_local std::string g_last_error;
}
void SetLastError(const std::string& msg) { g_last_error = msg; }

// One array of the step in device memory.
struct AuxView {
  const int32_t* ptr = nullptr;
  int64_t size = 0;
};

class PagedKVCache {
 public:
  PagedKVCache(const int64_t* cache_config, int n_config, int64_t layer_begin, int64_t layer_end,
               int64_t num_qo_heads, int64_t num_kv_heads, int64_t qk_head_dim, int64_t v_head_dim,
               std::vector<int64_t> attn_kinds, bool enable_kv_transfer, int rope_mode, double rope_scale,
               double rope_theta, int dtype_bits, int device_id)
      : page_size_(cache_config[3]),
        num_layers_(layer_end - layer_begin),
        layer_id_begin_offset_(layer_begin),
        num_qo_heads_(num_qo_heads),
        num_kv_heads_(num_kv_heads),
        qk_head_dim_(qk_head_dim),
        v_head_dim_(v_head_dim),
        prefill_chunk_size_(cache_config[2]),
        attn_kinds_(std::move(attn_kinds)),
        rotary_scale_(rope_scale),
        rotary_theta_(rope_theta),
        device_(device_id) {
    // paged_kv_cache.cc:2606-2619
    const int64_t reserved_num_seqs = cache_config[0];
    const int64_t total_token_capacity = cache_config[1];
    const bool support_sliding_window = cache_config[4] != 0;
    layer_sliding_window_size_ = n_config == 6 ? cache_config[5] : 1024;
    KV_CHECK(page_size_ > 0) << "page_size must be positive";
    num_total_pages_ = (total_token_capacity + page_size_ - 1) / page_size_ + 1;
    if (support_sliding_window) num_total_pages_ += reserved_num_seqs * 2;
    // paged_kv_cache.cc:335-344
    const bool has_layer_sliding =
        std::find(attn_kinds_.begin(), attn_kinds_.end(), TVMKV_ATTN_MHA_SLIDING) != attn_kinds_.end();
    support_sliding_window_ = has_layer_sliding ? false : support_sliding_window;
    rope_mode_ = (support_sliding_window && rope_mode != TVMKV_ROPE_NONE) ? TVMKV_ROPE_INLINE : rope_mode;
    KV_CHECK(layer_sliding_window_size_ > 0) << "Per-layer sliding window size must be positive.";
    const bool has_mla = std::find(attn_kinds_.begin(), attn_kinds_.end(), TVMKV_ATTN_MLA) != attn_kinds_.end();
    if (has_mla) {
      KV_CHECK(!support_sliding_window_) << "Sliding window not supported yet for MLA";
      KV_CHECK(!enable_kv_transfer) << "KV transfer not supported yet for MLA";
    }
    KV_UNSUPPORTED(enable_kv_transfer)
        << "KV transfer (disaggregation) needs a second device and is not built in this library";
    KV_UNSUPPORTED(dtype_bits != 16 && dtype_bits != 32)
        << "KV storage is built for float16 and float32 (got " << dtype_bits << " bits)";
    elem_bits_ = dtype_bits;
    // What the tuned fp16 kernels are not built for runs on the generic ones: float32 storage, pages other than
    // 16 / 32 / 64 / 128 tokens, other head dims -- and head dims 80 / 96 / 112 as soon as the cache has sliding
    // windows or rotates inside the attention kernels (the tuned kernels have those head dims in their plain form).
    bool has_mha_layer = false;
    for (int64_t kind : attn_kinds_) has_mha_layer |= (kind != TVMKV_ATTN_MLA);
    const bool extended = support_sliding_window_ || has_layer_sliding || rope_mode_ == TVMKV_ROPE_INLINE;
    const int head_dim = static_cast<int>(qk_head_dim_);
    const bool tuned_dim = extended ? (head_dim == 64 || head_dim == 128 || head_dim == 256) : tuned_head_dim(head_dim);
    generic_ = has_mha_layer && (elem_bits_ == 32 || !tuned_page_size(static_cast<int>(page_size_)) || (!has_mla && !tuned_dim));
    if (generic_) {
      KV_UNSUPPORTED(has_mla) << "float32 storage, pages other than 16 / 32 / 64 / 128 tokens and other head dims are "
                              << "not built for caches with MLA layers";
      KV_UNSUPPORTED(rope_mode_ == TVMKV_ROPE_INLINE && head_dim % (elem_bits_ == 32 ? 8 : 16) != 0)
          << "RoPE inside the generic attention kernels (a sliding-window cache rotates there) needs a head dim that is a "
          << "multiple of " << (elem_bits_ == 32 ? 8 : 16) << ", got " << head_dim;
      KV_UNSUPPORTED(qk_head_dim_ != v_head_dim_) << "the generic kernels need equal qk and v head dims";
    }
    KV_CHECK(static_cast<int64_t>(attn_kinds_.size()) >= layer_end)
        << "attn_kinds must cover every layer id up to " << layer_end;
    for (int64_t kind : attn_kinds_) {
      KV_UNSUPPORTED(kind != TVMKV_ATTN_MHA && kind != TVMKV_ATTN_MLA && kind != TVMKV_ATTN_MHA_SLIDING)
          << "attention kind " << kind << " is not supported";
    }
    KVConfig config;
    config.page_size = page_size_;
    config.num_total_pages = num_total_pages_;
    config.reserved_num_seqs = reserved_num_seqs;
    config.prefill_chunk_size = prefill_chunk_size_;
    config.layer_sliding_window_size = layer_sliding_window_size_;
    config.support_sliding_window = support_sliding_window_;
    config.support_layer_sliding_window = has_layer_sliding;
    config.rope_inline = rope_mode_ == TVMKV_ROPE_INLINE;
    config.first_layer_is_mla = !attn_kinds_.empty() && attn_kinds_[0] == TVMKV_ATTN_MLA;
    book_ = std::make_unique<KVBookkeeper>(config);
    reserved_num_seqs_ = reserved_num_seqs;
    if (device_ >= 0) InitDevice();
  }

  ~PagedKVCache() { ReleaseDevice(); }

  // ---------------------------------------------------------------- state verbs
  void Clear() {
    book_->Clear();
    page_copies_issued_ = 0;
    aux_needs_upload_ = false;
  }
  void AddSequence(int64_t seq_id) { book_->AddSequence(seq_id); }
  void RemoveSequence(int64_t seq_id) { book_->RemoveSequence(seq_id); }
  void ForkSequence(int64_t parent_seq_id, int64_t child_seq_id, int64_t fork_pos) {
    book_->ForkSequence(parent_seq_id, child_seq_id, fork_pos);
    IssuePageCopies();
  }
  void EnableSlidingWindowForSeq(int64_t seq_id, int32_t sliding_window_size, int32_t attn_sink_size) {
    book_->EnableSlidingWindowForSeq(seq_id, sliding_window_size, attn_sink_size);
  }
  void PopN(int64_t seq_id, int32_t n) {
    book_->PopN(seq_id, n);
    IssuePageCopies();
  }
  bool Empty() const { return book_->Empty(); }
  int32_t GetNumAvailablePages() const { return book_->NumAvailablePages(); }
  int32_t GetTotalSequenceLength() const { return book_->TotalSequenceLength(); }

  // The bookkeeper writes the step's arrays into the staging buffer that is not the one the last
  // upload read; the upload itself waits for the first device call of the step.
  void BeginForward(const int64_t* seq_ids, const int64_t* append_lengths, int64_t batch_size,
                    const int64_t* token_tree_parent_ptr, int64_t n_tree) {
    if (device_ >= 0) {
      // the kernels enqueued since the last step began were the last readers of the buffer in use
      if (aux_read_since_event_[aux_slot_]) {
        HIP_CHECK(hipSetDevice(device_));
        HIP_CHECK(hipEventRecord(aux_consumed_[aux_slot_], compute_stream_));
        aux_consumed_recorded_[aux_slot_] = true;
        aux_read_since_event_[aux_slot_] = false;
      }
      const int next = aux_slot_ ^ 1;
      // this slot's staging memory was last read by the upload two steps ago
      if (aux_slot_used_[next]) HIP_CHECK(hipEventSynchronize(aux_copied_[next]));
      book_->SetStepBuffer(static_cast<int32_t*>(aux_staging_[next]), aux_capacity_);
      aux_needs_upload_ = false;
      book_->BeginForward(seq_ids, append_lengths, batch_size, token_tree_parent_ptr, n_tree);
      aux_slot_ = next;
      aux_needs_upload_ = true;
    } else {
      book_->BeginForward(seq_ids, append_lengths, batch_size, token_tree_parent_ptr, n_tree);
    }
  }

  void EndForward() {}

  // :1566-1659
  void CommitAcceptedTokenTreeNodes(const int64_t* seq_ids, const int64_t* leaf_indices, int num) {
    if (book_->CommitAcceptedTokenTreeNodes(seq_ids, leaf_indices, num)) CompactKVCopy(num);
    IssuePageCopies();  // a pop into a shared block forks
  }

  // ---------------------------------------------------------------- attention (device)
  // :1303-1402
  void AttentionWithFusedQKV(int64_t layer_id, const void* qkv, int64_t qkv_rows, void* out, int64_t out_rows,
                             double sm_scale) {
    RequireDevice();
    const int64_t local_layer_id = CheckLayer(layer_id);
    KV_CHECK(attn_kinds_[layer_id] == TVMKV_ATTN_MHA || attn_kinds_[layer_id] == TVMKV_ATTN_MHA_SLIDING)
        << "attention_with_fused_qkv needs an MHA layer";
    KV_CHECK(out_rows == qkv_rows) << "qkv and output must have the same number of rows";
    const int64_t total_seq_length = TotalAppendLength();
    KV_CHECK(total_seq_length <= qkv_rows)
        << "qkv has " << qkv_rows << " rows, fewer than the batch appends (" << total_seq_length << ")";
    KV_CHECK(total_seq_length <= prefill_chunk_size_)
        << "the batch appends " << total_seq_length << " tokens, more than prefill_chunk_size " << prefill_chunk_size_;
    ComputeStreamWaitForCopyStream();
    const StepLayout& s = book_->step();
    const bool rope_normal = rope_mode_ == TVMKV_ROPE_NORMAL;

    // A chunked-prefill step of a plain cache in two launches: k is rotated and the new k / v rows go
    // into their page slots (part 2 without q, part 3), then one pass over the cached and the new
    // tokens that reads the queries from qkv and rotates them itself (parts 2 and 5).
    if (generic_) {
      // split + RoPE (+ append when the rows may go in before attention), the attention kernels of the step, the
      // append afterwards otherwise: the reference's flow (:1360-1401) on the typed and generic kernels
      const bool early = s.append_before_attn || !support_sliding_window_;
      const bool rotate = rope_normal || rope_ext_factors_ != nullptr;
      Launch(typed_fused_rope(elem_bits_, qkv, Dev(s.q_rope_position_map), temp_q_, temp_k_, temp_v_, rotate, rope_ext_factors_,
                              has_rope_scaling_ ? &rope_scaling_ : nullptr, early ? pages_[local_layer_id] : nullptr,
                              early ? Dev(s.append_position_map) : nullptr, total_seq_length, num_qo_heads_, num_kv_heads_,
                              qk_head_dim_, num_total_pages_, page_size_, rotary_scale_, rotary_theta_, compute_stream_));
      AttentionInternal(layer_id, temp_q_, temp_k_, temp_v_, out, total_seq_length, sm_scale);
      if (!early) {
        Launch(tvmkv_kv_cache_transpose_append(pages_[local_layer_id], temp_k_, temp_v_, Dev(s.append_position_map),
                                               total_seq_length, num_total_pages_, num_kv_heads_, page_size_,
                                               CopyDim(), compute_stream_));
      }
      RecordComputeEvent();
      return;
    }
    if (has_rope_scaling_) {
      // the model's frequency variant lives in the split-rotary kernel only: q, k and v take the round trip
      const bool early = s.append_before_attn || !support_sliding_window_;
      // the reference's kernel for a factor tensor has no apply_rope argument: it always rotates
      const bool rotate = rope_normal || rope_ext_factors_ != nullptr;
      if (early) {
        Launch(tvmkv_fused_rope_append_scaled(qkv, Dev(s.q_rope_position_map), temp_q_, temp_k_, temp_v_, rotate,
                                              rope_ext_factors_, &rope_scaling_, pages_[local_layer_id],
                                              Dev(s.append_position_map), total_seq_length, num_qo_heads_, num_kv_heads_,
                                              qk_head_dim_, num_total_pages_, page_size_, rotary_scale_, rotary_theta_,
                                              compute_stream_));
      } else {
        Launch(tvmkv_fused_rope_scaled(qkv, Dev(s.q_rope_position_map), temp_q_, temp_k_, temp_v_, rotate,
                                       rope_ext_factors_, &rope_scaling_, total_seq_length, num_qo_heads_, num_kv_heads_,
                                       qk_head_dim_, rotary_scale_, rotary_theta_, compute_stream_));
      }
      AttentionInternal(layer_id, temp_q_, temp_k_, temp_v_, out, total_seq_length, sm_scale);
      if (!early) {
        Launch(tvmkv_kv_cache_transpose_append(pages_[local_layer_id], temp_k_, temp_v_, Dev(s.append_position_map),
                                               total_seq_length, num_total_pages_, num_kv_heads_, page_size_,
                                               qk_head_dim_, compute_stream_));
      }
      RecordComputeEvent();
      return;
    }
    // A decode step of a plain cache in one launch: the decode kernel reads q from qkv and rotates it,
    // and the work items of every sequence's last chunk rotate and append the new k / v rows before they
    // attend to them (parts 2, 3 and 5).
    if (FusedDecodeStepApplies(layer_id)) {
      Launch(tvmkv_fused_decode_step(qkv, pages_[local_layer_id], Dev(s.page_indptr[0]), Dev(s.page_indices[0]),
                                     Dev(s.length_info[0]), Dev(s.q_rope_position_map), Dev(s.append_position_map), out,
                                     merged_lse_, rope_normal, rotary_scale_, rotary_theta_, sm_scale,
                                     book_->batch_size(), s.page_indices[0].size, num_total_pages_, num_qo_heads_,
                                     num_kv_heads_, qk_head_dim_, page_size_, compute_stream_));
      RecordComputeEvent();
      return;
    }
    if (OnePassPrefillApplies(layer_id)) {
      Launch(tvmkv_fused_rope_append(qkv, Dev(s.q_rope_position_map), /*q=*/nullptr, temp_k_, temp_v_, rope_normal,
                                     pages_[local_layer_id], Dev(s.append_position_map), total_seq_length,
                                     num_qo_heads_, num_kv_heads_, qk_head_dim_, num_total_pages_, page_size_,
                                     rotary_scale_, rotary_theta_, compute_stream_));
      Launch(tvmkv_batch_prefill_cached_and_new_kv_fused_q(
          qkv, Dev(s.q_rope_position_map), rope_normal, rotary_scale_, rotary_theta_,
          Dev(s.cur_append_lengths_indptr), temp_k_, temp_v_, pages_[local_layer_id], Dev(s.page_indptr[0]),
          Dev(s.page_indices[0]), Dev(s.length_info[0]), out, merged_lse_, sm_scale, book_->batch_size(),
          total_seq_length, s.page_indices[0].size, num_total_pages_, num_qo_heads_, num_kv_heads_, qk_head_dim_,
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
    const bool append_early = s.append_before_attn || !support_sliding_window_;
    if (append_early) {
      Launch(tvmkv_fused_rope_append(qkv, Dev(s.q_rope_position_map), temp_q_, temp_k_, temp_v_, rope_normal,
                                     pages_[local_layer_id], Dev(s.append_position_map), total_seq_length,
                                     num_qo_heads_, num_kv_heads_, qk_head_dim_, num_total_pages_, page_size_,
                                     rotary_scale_, rotary_theta_, compute_stream_));
    } else {
      Launch(tvmkv_fused_rope(qkv, Dev(s.q_rope_position_map), temp_q_, temp_k_, temp_v_, rope_normal,
                              total_seq_length, num_qo_heads_, num_kv_heads_, qk_head_dim_, rotary_scale_,
                              rotary_theta_, compute_stream_));
    }
    // Part 5: attention.
    AttentionInternal(layer_id, temp_q_, temp_k_, temp_v_, out, total_seq_length, sm_scale);
    // Part 6: append after attention (:1396-1401).
    if (!append_early) {
      Launch(tvmkv_kv_cache_transpose_append(pages_[local_layer_id], temp_k_, temp_v_, Dev(s.append_position_map),
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
    const int64_t total_seq_length = TotalAppendLength();
    KV_CHECK(rows == total_seq_length) << "attention_with_shared_kv expects " << total_seq_length << " rows, got " << rows;
    ComputeStreamWaitForCopyStream();
    AttentionInternal(source_layer_id, q, k, v, o, total_seq_length, sm_scale);
    RecordComputeEvent();
  }

  // :1404-1445
  void SelfAttention(int64_t layer_id, const void* q, const void* k, const void* v, void* o, float* lse, int64_t rows,
                     int k_heads, int qk_dim, int v_dim, double sm_scale) {
    RequireDevice();
    CheckLayer(layer_id);
    const int64_t total_seq_length = TotalAppendLength();
    KV_CHECK(rows == total_seq_length) << "self_attention expects " << total_seq_length << " rows, got " << rows;
    ComputeStreamWaitForCopyStream();
    const StepLayout& s = book_->step();
    if (!s.is_chain[0]) {
      KV_CHECK(attn_kinds_[layer_id] == TVMKV_ATTN_MHA) << "Tree attn not able for MLA for now.";
      KV_CHECK(k_heads == num_kv_heads_ && qk_dim == qk_head_dim_ && v_dim == v_head_dim_)
          << "self_attention: k/v shapes do not match the cache";
      MHASelfAttnInternal(q, k, v, o, lse, total_seq_length, sm_scale);
      RecordComputeEvent();
      return;
    }
    const int rotary = attn_kinds_[layer_id] == TVMKV_ATTN_MHA ? (rope_mode_ == TVMKV_ROPE_INLINE) : 0;
    if (generic_ && attn_kinds_[layer_id] == TVMKV_ATTN_MHA) {
      KV_CHECK(k_heads == num_kv_heads_ && qk_dim == qk_head_dim_ && v_dim == v_head_dim_)
          << "self_attention: k/v shapes do not match the cache";
      GenericRagged(q, k, v, o, lse, total_seq_length, sm_scale, /*tree=*/false);
      RecordComputeEvent();
      return;
    }
    Launch(tvmkv_batch_prefill_ragged_kv_scaled(q, Dev(s.cur_append_lengths_indptr), k, v, Dev(s.cur_append_lengths_indptr),
                                                Dev(s.q_rope_position_map), Dev(s.k_ragged_rope_pos_offset), o, lse,
                                                /*causal=*/1, rotary, rotary_scale_, rotary_theta_, sm_scale,
                                                book_->batch_size(), total_seq_length, num_qo_heads_, k_heads, qk_dim, v_dim,
                                                InlineScaling(), compute_stream_));
    RecordComputeEvent();
  }

  // :1447-1485
  void CrossAttention(int64_t layer_id, const void* q, void* o, float* lse, int64_t rows, double sm_scale) {
    RequireDevice();
    const int64_t local_layer_id = CheckLayer(layer_id);
    const int64_t total_seq_length = TotalAppendLength();
    KV_CHECK(rows == total_seq_length) << "cross_attention expects " << total_seq_length << " rows, got " << rows;
    ComputeStreamWaitForCopyStream();
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
    const int64_t local_layer_id = CheckLayer(layer_id);
    KV_CHECK(attn_kinds_[layer_id] == TVMKV_ATTN_MLA) << "append_mla_kv needs an MLA layer";
    const int64_t total_seq_length = TotalAppendLength();
    KV_CHECK(rows <= total_seq_length) << "kv has more rows than the batch appends";
    ComputeStreamWaitForCopyStream();
    Launch(tvmkv_kv_cache_transpose_append_mla(pages_[local_layer_id], kv, Dev(book_->step().append_position_map), rows,
                                               num_total_pages_, page_size_, qk_head_dim_, compute_stream_));
    RecordComputeEvent();
  }

  // :1553-1559
  void MergeAttnOutputInplace(void* o_self, float* lse_self, const void* o_cross, const float* lse_cross, int64_t rows,
                              int heads, int dim) {
    RequireDevice();
    Launch(typed_merge_state_inplace(elem_bits_, o_self, lse_self, o_cross, lse_cross, rows, heads, dim, compute_stream_));
  }

  // :1661-1667
  AuxView GetQueryPositions() {
    RequireDevice();
    KV_CHECK(book_->began_forward()) << "begin_forward has not been called";
    ComputeStreamWaitForCopyStream();
    const AuxSpan& span = book_->step().q_rope_position_map;
    return AuxView{Dev(span), span.size};
  }

  // :1669-1766
  void DebugGetKV(int64_t seq_id, int64_t start_pos, int64_t end_pos, void* k_data, void* v_data, bool mla) {
    RequireDevice();
    const std::vector<int32_t> map = book_->PositionMapOf(seq_id, start_pos, end_pos);
    HIP_CHECK(hipSetDevice(device_));
    int32_t* map_dev = nullptr;
    HIP_CHECK(hipMalloc(&map_dev, map.size() * sizeof(int32_t)));
    try {
      HIP_CHECK(hipMemcpyAsync(map_dev, map.data(), map.size() * sizeof(int32_t), hipMemcpyHostToDevice, compute_stream_));
      for (int64_t layer = 0; layer < num_layers_; ++layer) {
        const int64_t kind = attn_kinds_[layer + layer_id_begin_offset_];
        if (mla) {
          KV_CHECK(kind == TVMKV_ATTN_MLA) << "Only MLA is supported for DebugGetKVMLA";
          Launch(tvmkv_kv_cache_debug_get_kv_mla(pages_[layer], map_dev, k_data, layer, map.size(), num_total_pages_,
                                                 page_size_, qk_head_dim_, compute_stream_));
        } else {
          KV_CHECK(kind == TVMKV_ATTN_MHA) << "Only MHA is supported for DebugGetKV";
          Launch(tvmkv_kv_cache_debug_get_kv(pages_[layer], map_dev, k_data, v_data, layer, map.size(), num_total_pages_,
                                             num_kv_heads_, page_size_, CopyDim(), compute_stream_));
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
  // Host copy of one auxiliary array of the last step (the staging memory the upload reads).
  void GetAux(const std::string& name, int depth, const int32_t** data, int64_t* size) const {
    const std::vector<int32_t>* commit = nullptr;
    if (name == "commit_copy_length_indptr") commit = &book_->commit_copy_length_indptr();
    if (name == "commit_copy_src_pos") commit = &book_->commit_copy_src_pos();
    if (name == "commit_copy_dst_pos") commit = &book_->commit_copy_dst_pos();
    if (commit != nullptr) {
      *data = commit->data();
      *size = static_cast<int64_t>(commit->size());
      return;
    }
    const AuxSpan span = book_->FindAux(name, depth);
    *data = book_->step_buffer() == nullptr ? nullptr : book_->step_buffer() + span.offset;
    *size = span.size;
  }

  void GetFlags(int64_t* flags, int n) const {
    const StepLayout& s = book_->step();
    const int64_t all[9] = {s.num_depths,
                            s.append_before_attn,
                            s.is_decode_request,
                            s.num_depths > 0 ? s.use_decode_kernel[0] : 0,
                            s.num_depths > 1 ? s.use_decode_kernel[1] : 0,
                            s.is_chain[0],
                            s.is_chain[1],
                            num_total_pages_,
                            rope_mode_};
    for (int i = 0; i < n && i < 9; ++i) flags[i] = all[i];
  }

  std::vector<int64_t> DumpState() const { return book_->DumpState(); }
  const std::vector<int64_t>& CopyLog() const { return book_->CopyLog(); }
  void* Pages(int64_t local_layer, int64_t* bytes) {
    RequireDevice();
    KV_CHECK(local_layer >= 0 && local_layer < num_layers_) << "layer " << local_layer << " out of range";
    *bytes = PageBytes(local_layer);
    return pages_[local_layer];
  }
  void SetStream(hipStream_t stream) {
    if (stream == compute_stream_) return;
    if (device_ >= 0 && (compute_work_since_event_ || aux_read_since_event_[aux_slot_])) {
      // the events that later waits rely on belong on the stream the work was enqueued on
      HIP_CHECK(hipSetDevice(device_));
      if (compute_work_since_event_) {
        HIP_CHECK(hipEventRecord(compute_done_, compute_stream_));
        compute_event_recorded_ = true;
        compute_work_since_event_ = false;
      }
      if (aux_read_since_event_[aux_slot_]) {
        HIP_CHECK(hipEventRecord(aux_consumed_[aux_slot_], compute_stream_));
        aux_consumed_recorded_[aux_slot_] = true;
        aux_read_since_event_[aux_slot_] = false;
      }
    }
    compute_stream_ = stream;
  }
  void SetRopeScaling(const tvmkv_rope_scaling* scaling, const float* rope_ext_factors) {
    // a description that differs from the default rotation: another frequency rule, or only part of the head rotated
    has_rope_scaling_ = scaling != nullptr && (scaling->rope_type != TVMKV_ROPE_FREQ_DEFAULT ||
                                               (scaling->rotary_dim > 0 && scaling->rotary_dim != qk_head_dim_));
    // (a cache that rotates inside the attention kernels hands the description to them: they rotate the whole
    // head with the variant's frequencies, python/tvm/relax/frontend/nn/llm/_kernel_common.py:115-127)
    KV_CHECK((scaling != nullptr && scaling->rope_type == TVMKV_ROPE_FREQ_LONGROPE) || rope_ext_factors == nullptr)
        << "rope_ext_factors needs a longrope scaling description";
    if (has_rope_scaling_) rope_scaling_ = *scaling;
    rope_ext_factors_ = rope_ext_factors;
  }

 private:
  // ---------------------------------------------------------------- device layer
  void RequireDevice() const {
    if (device_ < 0) throw Error(TVMKV_ENODEVICE, "this cache was created host-only (device_id = -1)");
  }
  static void Launch(int rc) {
    if (rc != TVMKV_OK) throw Error(rc, tvmkv_last_error());
  }
  int64_t CheckLayer(int64_t layer_id) const {
    const int64_t local_layer_id = layer_id - layer_id_begin_offset_;
    KV_CHECK(local_layer_id >= 0 && local_layer_id < num_layers_) << "layer id " << layer_id << " out of range";
    return local_layer_id;
  }
  int64_t TotalAppendLength() const {
    KV_CHECK(book_->began_forward()) << "begin_forward has not been called";
    return book_->step().total_append_length;
  }
  int64_t PageBytes(int64_t local_layer) const {
    const int64_t kind = attn_kinds_[local_layer + layer_id_begin_offset_];
    // GetKVCacheShape, attn_utils.h:74-87
    if (kind == TVMKV_ATTN_MLA) return num_total_pages_ * page_size_ * qk_head_dim_ * 2;
    return num_total_pages_ * 2 * num_kv_heads_ * page_size_ * qk_head_dim_ * (elem_bits_ / 8);
  }
  // Device address of an array of the current step (nullptr when the step does not have it).
  const int32_t* Dev(const AuxSpan& span) const {
    return span.present() ? static_cast<const int32_t*>(aux_device_[aux_slot_]) + span.offset : nullptr;
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
        HIP_CHECK(hipMalloc(&temp_q_, prefill_chunk_size_ * num_qo_heads_ * qk_head_dim_ * (elem_bits_ / 8)));
        HIP_CHECK(hipMalloc(&temp_k_, prefill_chunk_size_ * num_kv_heads_ * qk_head_dim_ * (elem_bits_ / 8)));
        HIP_CHECK(hipMalloc(&temp_v_, prefill_chunk_size_ * num_kv_heads_ * v_head_dim_ * (elem_bits_ / 8)));
      }
      HIP_CHECK(hipMalloc(&temp_out_, prefill_chunk_size_ * num_qo_heads_ * v_head_dim_ * (elem_bits_ / 8)));
      HIP_CHECK(hipMalloc(&temp_lse_, prefill_chunk_size_ * num_qo_heads_ * sizeof(float)));
      HIP_CHECK(hipMalloc(&merged_lse_, prefill_chunk_size_ * num_qo_heads_ * sizeof(float)));
      aux_capacity_ = book_->RequiredCapacity();
      for (int i = 0; i < 2; ++i) {
        HIP_CHECK(hipMalloc(&aux_device_[i], aux_capacity_ * sizeof(int32_t)));
        HIP_CHECK(hipHostMalloc(&aux_staging_[i], aux_capacity_ * sizeof(int32_t), hipHostMallocDefault));
        HIP_CHECK(hipEventCreateWithFlags(&aux_copied_[i], hipEventDisableTiming));
        HIP_CHECK(hipEventCreateWithFlags(&aux_consumed_[i], hipEventDisableTiming));
      }
      // token-tree commit: copy_length_indptr + (2, copies) positions (attn_utils.h:1010-1021)
      const int64_t r = reserved_num_seqs_, c = prefill_chunk_size_;
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
      aux_consumed_recorded_[i] = aux_slot_used_[i] = aux_read_since_event_[i] = false;
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

  // Kernels of the step were enqueued on the compute stream.  Nothing is recorded here: an event
  // record between the launches of two layers costs the device ~5 us of idle time each, so the
  // events are recorded where somebody is about to wait for them (CopyStreamWaitsForCompute,
  // BeginForward).
  void RecordComputeEvent() {
    compute_work_since_event_ = true;
    aux_read_since_event_[aux_slot_] = true;  // by kernels that read the auxiliary buffer in use
  }

  // Orders what is enqueued on the copy stream next after everything enqueued on the compute stream so far.
  void CopyStreamWaitsForCompute() {
    if (compute_work_since_event_) {
      HIP_CHECK(hipEventRecord(compute_done_, compute_stream_));
      compute_event_recorded_ = true;
      compute_work_since_event_ = false;
    }
    if (compute_event_recorded_) HIP_CHECK(hipStreamWaitEvent(copy_stream_, compute_done_, 0));
  }

  // The partial-page copies that forks have asked for since the last call (:721-734).  They run on the
  // copy stream, after everything enqueued on the compute stream so far (the source page may have
  // been written by the previous step's append).
  void IssuePageCopies() {
    const std::vector<int64_t>& log = book_->CopyLog();
    if (page_copies_issued_ == log.size()) return;
    // everything up to here is (about to be) issued: a long log drops its oldest entries on the way out
    struct Trim {
      KVBookkeeper* book;
      size_t* issued;
      ~Trim() { *issued -= book->TrimCopyLog(*issued); }
    } trim{book_.get(), &page_copies_issued_};
    if (device_ < 0) {
      page_copies_issued_ = log.size();
      return;
    }
    HIP_CHECK(hipSetDevice(device_));
    CopyStreamWaitsForCompute();
    for (; page_copies_issued_ < log.size(); page_copies_issued_ += 3) {
      const int32_t src = static_cast<int32_t>(log[page_copies_issued_]);
      const int32_t tgt = static_cast<int32_t>(log[page_copies_issued_ + 1]);
      const int64_t copy_length = log[page_copies_issued_ + 2];
      for (int64_t layer = 0; layer < num_layers_; ++layer) {
        if (attn_kinds_[layer + layer_id_begin_offset_] == TVMKV_ATTN_MLA) {
          Launch(tvmkv_copy_single_page_mla(pages_[layer], src, tgt, copy_length, num_total_pages_, page_size_,
                                            qk_head_dim_, copy_stream_));
        } else {
          Launch(tvmkv_copy_single_page(pages_[layer], src, tgt, copy_length, num_total_pages_, num_kv_heads_,
                                        page_size_, CopyDim(), copy_stream_));
        }
      }
    }
    copy_stream_has_work_ = true;
  }

  // :736-770
  void CompactKVCopy(int64_t batch_size) {
    const std::vector<int32_t>& indptr = book_->commit_copy_length_indptr();
    const int total_copy_length = indptr.back();
    KV_CHECK(total_copy_length >= 0) << "negative copy length";
    if (total_copy_length == 0 || device_ < 0) return;
    HIP_CHECK(hipSetDevice(device_));
    // one upload: [copy_length_indptr (batch + 1), padded to 16 bytes | src positions | dst positions]
    const int64_t n_indptr = static_cast<int64_t>(indptr.size());
    const int64_t pos_begin = (n_indptr + 3) / 4 * 4;
    KV_CHECK(pos_begin + 2 * static_cast<int64_t>(total_copy_length) <= commit_capacity_)
        << "token-tree commit copies " << total_copy_length << " slots, more than the cache was sized for";
    // the staging buffer is reused: wait until the previous commit's upload has read it
    if (commit_staging_used_) HIP_CHECK(hipEventSynchronize(commit_copied_));
    int32_t* staging = static_cast<int32_t*>(commit_staging_);
    std::memcpy(staging, indptr.data(), n_indptr * sizeof(int32_t));
    std::memcpy(staging + pos_begin, book_->commit_copy_src_pos().data(), total_copy_length * sizeof(int32_t));
    std::memcpy(staging + pos_begin + total_copy_length, book_->commit_copy_dst_pos().data(),
                total_copy_length * sizeof(int32_t));
    int32_t* device = static_cast<int32_t*>(commit_device_);
    // after the attention kernels of the step that computed on these slots
    CopyStreamWaitsForCompute();
    HIP_CHECK(hipMemcpyAsync(device, staging, (pos_begin + 2 * total_copy_length) * sizeof(int32_t),
                             hipMemcpyHostToDevice, copy_stream_));
    HIP_CHECK(hipEventRecord(commit_copied_, copy_stream_));
    commit_staging_used_ = true;
    for (int64_t layer = 0; layer < num_layers_; ++layer) {
      Launch(tvmkv_compact_kv_copy(pages_[layer], device, device + pos_begin, batch_size, total_copy_length,
                                   num_total_pages_, num_kv_heads_, page_size_, CopyDim(), copy_stream_));
    }
    // The next step's first kernel waits for the copy stream (paged_kv_cache.cc:767-769).
    copy_stream_has_work_ = true;
  }

  // A chunked-prefill step of a plain cache (one depth, no sliding window, no inline RoPE, no token
  // tree) can run as one pass over the cached and the new tokens.
  // One sequence per entry, one token each, appended before attention, one level of blocks, a plain cache
  // whose keys are stored rotated (or not rotated at all) with the default frequencies.
  bool FusedDecodeStepApplies(int64_t layer_id) const {
    const StepLayout& s = book_->step();
    return !generic_ && s.append_before_attn && s.is_decode_request && s.num_depths == 1 && s.is_chain[0] &&
           s.use_decode_kernel[0] && !support_sliding_window_ && attn_kinds_[layer_id] == TVMKV_ATTN_MHA && rope_mode_ != TVMKV_ROPE_INLINE &&
           !has_rope_scaling_ && qk_head_dim_ == v_head_dim_ &&
           (qk_head_dim_ == 64 || qk_head_dim_ == 128 || qk_head_dim_ == 256) && option(kOptNoFusedDecodeStep) == 0;
  }

  bool OnePassPrefillApplies(int64_t layer_id) const {
    const StepLayout& s = book_->step();
    return !generic_ && !s.append_before_attn && s.num_depths == 1 && s.is_chain[0] && !s.use_decode_kernel[0] &&
           s.page_indices[0].size > 0 && !support_sliding_window_ && attn_kinds_[layer_id] == TVMKV_ATTN_MHA &&
           rope_mode_ != TVMKV_ROPE_INLINE && qk_head_dim_ == v_head_dim_ && (qk_head_dim_ == 64 || qk_head_dim_ == 128);
  }

  // :2161-2180
  void AttentionInternal(int64_t layer_id, const void* q, const void* k, const void* v, void* output,
                         int64_t total_seq_length, double sm_scale) {
    const int64_t local_layer_id = layer_id - layer_id_begin_offset_;
    const StepLayout& s = book_->step();
    // A chunked-prefill step of a plain cache: self-attention over the new tokens, attention over the
    // cached ones and their merge (:2169-2177, :2285-2292) in one pass over both key sets.
    if (OnePassPrefillApplies(layer_id)) {
      Launch(tvmkv_batch_prefill_cached_and_new_kv(
          q, Dev(s.cur_append_lengths_indptr), k, v, pages_[local_layer_id], Dev(s.page_indptr[0]), Dev(s.page_indices[0]),
          Dev(s.length_info[0]), output, merged_lse_, sm_scale, book_->batch_size(), total_seq_length,
          s.page_indices[0].size, num_total_pages_, num_qo_heads_, num_kv_heads_, qk_head_dim_, page_size_,
          compute_stream_));
      return;
    }
    bool is_first_kernel = true;
    if (!s.append_before_attn) {
      is_first_kernel = false;
      MHASelfAttnInternal(q, k, v, output, merged_lse_, total_seq_length, sm_scale);
    }
    const bool self_attn_computed = !is_first_kernel;
    const bool cross_attn_computed = MHACrossAttnInternal(
        local_layer_id, q, output, merged_lse_, total_seq_length, sm_scale, is_first_kernel,
        /*causal=*/!s.append_before_attn && attn_kinds_[layer_id] == TVMKV_ATTN_MHA_SLIDING);
    KV_CHECK(self_attn_computed || cross_attn_computed) << "Both self-attention and cross-attention are not computed.";
  }

  // :2182-2203
  void MHASelfAttnInternal(const void* q, const void* k, const void* v, void* o, float* lse, int64_t total_seq_length,
                           double sm_scale) {
    const StepLayout& s = book_->step();
    const int rope_inline = rope_mode_ == TVMKV_ROPE_INLINE;
    if (generic_) {
      if (!s.is_chain[0]) {
        KV_CHECK(s.tree_attn_mask[0].present() && s.tree_attn_mn_indptr[0].present()) << "token-tree mask is not on the device";
      }
      GenericRagged(q, k, v, o, lse, total_seq_length, sm_scale, /*tree=*/!s.is_chain[0]);
      return;
    }
    if (s.is_chain[0]) {
      Launch(tvmkv_batch_prefill_ragged_kv_scaled(q, Dev(s.cur_append_lengths_indptr), k, v, Dev(s.cur_append_lengths_indptr),
                                                  Dev(s.q_rope_position_map), Dev(s.k_ragged_rope_pos_offset), o, lse,
                                                  /*causal=*/1, rope_inline, rotary_scale_, rotary_theta_, sm_scale,
                                                  book_->batch_size(), total_seq_length, num_qo_heads_, num_kv_heads_,
                                                  qk_head_dim_, v_head_dim_, InlineScaling(), compute_stream_));
    } else {
      // the batch forms token trees
      KV_CHECK(s.tree_attn_mask[0].present() && s.tree_attn_mn_indptr[0].present()) << "token-tree mask is not on the device";
      KV_CHECK(qk_head_dim_ == v_head_dim_) << "tree attention needs equal qk and v head dims";
      Launch(tvmkv_batch_tree_attn_scaled(q, Dev(s.cur_append_lengths_indptr), k, v, Dev(s.cur_append_lengths_indptr),
                                          Dev(s.q_rope_position_map), Dev(s.tree_attn_mn_indptr[0]), Dev(s.tree_attn_mask[0]), o,
                                          lse, rope_inline, rotary_scale_, rotary_theta_, sm_scale, book_->batch_size(),
                                          total_seq_length, num_qo_heads_, num_kv_heads_, qk_head_dim_, InlineScaling(),
                                          compute_stream_));
    }
  }

  // feature extent of a K/V row for the copy kernels, which move rows as fp16 elements whatever they hold
  int32_t CopyDim() const { return copy_dim(elem_bits_, static_cast<int32_t>(qk_head_dim_)); }

  // causal self-attention over the step's new tokens (or the token-tree mask) on the generic kernel
  void GenericRagged(const void* q, const void* k, const void* v, void* o, float* lse, int64_t total_seq_length,
                     double sm_scale, bool tree) {
    const StepLayout& s = book_->step();
    GenericAttention a;
    a.what = "self attention";
    a.elem_bits = elem_bits_;
    a.q = q;
    a.q_indptr = Dev(s.cur_append_lengths_indptr);
    a.k = k;
    a.v = v;
    a.kv_indptr = Dev(s.cur_append_lengths_indptr);
    if (tree) {
      a.tree_indptr = Dev(s.tree_attn_mn_indptr[0]);
      a.tree_labels = Dev(s.tree_attn_mask[0]);
    }
    // RoPE inside the kernel: a chain's key t sits at k_ragged_rope_pos_offset[b] + t, a tree's keys at the
    // positions of its query tokens (their depths), as in the tuned calls
    a.rotary_mode = rope_mode_ == TVMKV_ROPE_INLINE;
    a.q_rope_position = Dev(s.q_rope_position_map);
    a.k_rope_pos_offset = tree ? nullptr : Dev(s.k_ragged_rope_pos_offset);
    a.rope_scale = rotary_scale_;
    a.rope_theta = rotary_theta_;
    a.rope_scaling = InlineScaling();
    a.out = o;
    a.lse = lse;
    a.total_q = total_seq_length;
    a.batch = book_->batch_size();
    a.h_q = static_cast<int32_t>(num_qo_heads_);
    a.h_kv = static_cast<int32_t>(num_kv_heads_);
    a.d = static_cast<int32_t>(qk_head_dim_);
    a.causal = 1;
    a.sm_scale = sm_scale;
    Launch(generic_attention(a, compute_stream_));
  }

  // :2216-2299
  bool MHACrossAttnInternal(int64_t local_layer_id, const void* q, void* o, float* lse, int64_t total_seq_length,
                            double sm_scale, bool is_first_kernel, bool causal) {
    const StepLayout& s = book_->step();
    KV_CHECK(s.num_depths >= 1) << "The number of effective depths must be greater or equal to 1.";
    const bool sliding_layer = attn_kinds_[local_layer_id + layer_id_begin_offset_] == TVMKV_ATTN_MHA_SLIDING;
    const int sliding_window = (support_sliding_window_ || sliding_layer) ? 1 : 0;
    const double rotary_theta = sliding_layer ? 10000 : rotary_theta_;
    const double rotary_scale = sliding_layer ? 1 : rotary_scale_;
    const int rotary_mode = rope_mode_ == TVMKV_ROPE_INLINE;
    bool cross_attn_computed = false;
    // The reference walks the depths in order and merges each state into the first (:2216-2299).  The merge
    // is symmetric, and the paged-prefill kernel can merge into an existing state in its own epilogue while the
    // decode and tree kernels need a temporary output and a merge launch: the depths that run those go first,
    // so that one of them writes (o, lse) directly and the prefill depths need no launch of their own to merge
    // (a decode step over a shared prompt: four launches per layer instead of five).
    int order[kMaxBlockDepth];
    int n_order = 0;
    for (int pass = 0; pass < 2; ++pass) {
      for (int d = 0; d < s.num_depths; ++d) {
        const bool merges_itself = !generic_ && !(s.append_before_attn && !s.is_chain[d]) && !s.use_decode_kernel[d];
        if (merges_itself == (pass == 1)) order[n_order++] = d;
      }
    }
    for (int at = 0; at < n_order; ++at) {
      const int d = order[at];
      if (s.page_indices[d].size == 0) continue;
      void* attn_output = is_first_kernel ? o : temp_out_;
      float* attn_lse = is_first_kernel ? lse : temp_lse_;
      const AuxSpan& page_indices_span = sliding_layer ? s.page_indices_sw[d] : s.page_indices[d];
      const int32_t* page_indptr = Dev(sliding_layer ? s.page_indptr_sw[d] : s.page_indptr[d]);
      const int32_t* page_indices = Dev(page_indices_span);
      const int32_t* length_info = Dev(sliding_layer ? s.layer_sw_length_info[d] : s.length_info[d]);
      const int32_t* k_rope_pos = Dev(sliding_layer ? s.k_rope_pos_offset_sw[d] : s.k_rope_pos_offset[d]);
      const int32_t* qo_indptr = Dev(s.qo_indptr[d]);
      const int32_t* q_pos = Dev(s.q_rope_position_map);
      const int64_t entries = s.qo_indptr[d].size - 1;
      const int64_t nnz_pages = page_indices_span.size;
      if (generic_) {
        GenericAttention a;
        a.what = "cross attention";
        a.elem_bits = elem_bits_;
        a.q = q;
        a.q_indptr = qo_indptr;
        a.pages = pages_[local_layer_id];
        a.page_indptr = page_indptr;
        a.page_values = page_indices;
        a.last_page_len = length_info;
        if (s.append_before_attn && !s.is_chain[d]) {
          KV_CHECK(s.tree_attn_mask[d].present() && s.tree_attn_mn_indptr[d].present())
              << "token-tree mask is not on the device";
          a.tree_indptr = Dev(s.tree_attn_mn_indptr[d]);
          a.tree_labels = Dev(s.tree_attn_mask[d]);
        }
        a.out = attn_output;
        a.lse = attn_lse;
        a.total_q = total_seq_length;
        a.nnz_pages = nnz_pages;
        a.num_pages = num_total_pages_;
        a.batch = static_cast<int32_t>(entries);
        a.h_q = static_cast<int32_t>(num_qo_heads_);
        a.h_kv = static_cast<int32_t>(num_kv_heads_);
        a.d = static_cast<int32_t>(qk_head_dim_);
        a.page_size = static_cast<int32_t>(page_size_);
        a.causal = causal;
        a.sm_scale = sm_scale;
        a.sliding_window = sliding_window;
        a.layer_window = static_cast<int32_t>(layer_sliding_window_size_);
        a.rotary_mode = rotary_mode;
        a.q_rope_position = q_pos;
        a.k_rope_pos_offset = k_rope_pos;
        a.rope_scale = rotary_scale;
        a.rope_theta = rotary_theta;
        a.rope_scaling = InlineScaling();
        Launch(generic_attention(a, compute_stream_));
      } else if (s.append_before_attn && !s.is_chain[d]) {
        KV_CHECK(s.tree_attn_mask[d].present() && s.tree_attn_mn_indptr[d].present())
            << "token-tree mask is not on the device";
        Launch(tvmkv_tree_attn_paged_kv(q, qo_indptr, pages_[local_layer_id], page_indptr, page_indices, length_info,
                                        k_rope_pos, q_pos, attn_output, attn_lse, rotary_mode, rotary_scale, rotary_theta,
                                        sm_scale, Dev(s.tree_attn_mn_indptr[d]), Dev(s.tree_attn_mask[d]), entries,
                                        total_seq_length, nnz_pages, num_total_pages_, num_qo_heads_, num_kv_heads_,
                                        qk_head_dim_, page_size_, sliding_window, compute_stream_));
      } else if (s.use_decode_kernel[d]) {
        Launch(tvmkv_batch_decode_paged_kv_scaled(q, pages_[local_layer_id], page_indptr, page_indices, length_info,
                                                  k_rope_pos, q_pos, attn_output, attn_lse, rotary_mode, rotary_scale,
                                                  rotary_theta, sm_scale, entries, nnz_pages, num_total_pages_,
                                                  num_qo_heads_, num_kv_heads_, qk_head_dim_, page_size_, sliding_window,
                                                  InlineScaling(), compute_stream_));
      } else if (!is_first_kernel) {
        // The prefill kernel merges its state into (o, lse) in its epilogue: one launch for the
        // kernel and the merge of :2285-2292, and no temporary output.
        Launch(tvmkv_batch_prefill_paged_kv_scaled(q, qo_indptr, pages_[local_layer_id], page_indptr, page_indices,
                                                   length_info, k_rope_pos, q_pos, o, lse, causal, rotary_mode, rotary_scale,
                                                   rotary_theta, sm_scale, entries, total_seq_length, nnz_pages,
                                                   num_total_pages_, num_qo_heads_, num_kv_heads_, qk_head_dim_, page_size_,
                                                   sliding_window, layer_sliding_window_size_, /*merge_into=*/1,
                                                   InlineScaling(), compute_stream_));
        cross_attn_computed = true;
        continue;
      } else {
        Launch(tvmkv_batch_prefill_paged_kv_scaled(q, qo_indptr, pages_[local_layer_id], page_indptr, page_indices,
                                                   length_info, k_rope_pos, q_pos, attn_output, attn_lse, causal, rotary_mode,
                                                   rotary_scale, rotary_theta, sm_scale, entries, total_seq_length, nnz_pages,
                                                   num_total_pages_, num_qo_heads_, num_kv_heads_, qk_head_dim_, page_size_,
                                                   sliding_window, layer_sliding_window_size_, /*merge_into=*/0,
                                                   InlineScaling(), compute_stream_));
      }
      if (!is_first_kernel) {
        Launch(typed_merge_state_inplace(elem_bits_, o, lse, temp_out_, temp_lse_, total_seq_length, num_qo_heads_,
                                         v_head_dim_, compute_stream_));
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
    const StepLayout& s = book_->step();
    KV_CHECK(s.num_depths >= 1) << "The number of effective depths must be greater or equal to 1.";
    bool is_first_kernel = true;
    for (int d = 0; d < s.num_depths; ++d) {
      if (s.page_indices[d].size == 0) continue;
      void* attn_output = is_first_kernel ? o : temp_out_;
      float* attn_lse = is_first_kernel ? lse : temp_lse_;
      KV_CHECK(s.is_chain[d]) << "Tree attn not able for MLA for now.";
      Launch(tvmkv_batch_prefill_paged_kv_mla(q, Dev(s.qo_indptr[d]), pages_[local_layer_id], Dev(s.page_indptr[d]),
                                              Dev(s.page_indices[d]), Dev(s.length_info[d]), attn_output, attn_lse,
                                              /*causal=*/0, sm_scale, s.qo_indptr[d].size - 1, total_seq_length,
                                              s.page_indices[d].size, num_total_pages_, num_qo_heads_, v_head_dim_,
                                              qk_head_dim_ - v_head_dim_, page_size_, compute_stream_));
      if (!is_first_kernel) {
        Launch(tvmkv_merge_state_inplace(o, lse, temp_out_, temp_lse_, total_seq_length, num_qo_heads_, v_head_dim_,
                                         compute_stream_));
      } else {
        is_first_kernel = false;
      }
    }
    return !is_first_kernel;
  }

  // :2338-2366: the step's arrays go up once, at the first device call of the step (one copy of the
  // part of the staging buffer in use), and the compute stream waits for everything on the copy
  // stream (that upload, fork page copies, commit compaction).
  void ComputeStreamWaitForCopyStream() {
    if (!aux_needs_upload_ && !copy_stream_has_work_) return;
    HIP_CHECK(hipSetDevice(device_));
    if (aux_needs_upload_) {
      const int64_t used = book_->step().used;
      if (used > 0) {
        // A host that runs ahead of the device must not overwrite arrays that kernels of the step
        // two uploads ago, still queued on the compute stream, have yet to read.
        if (aux_consumed_recorded_[aux_slot_]) HIP_CHECK(hipStreamWaitEvent(copy_stream_, aux_consumed_[aux_slot_], 0));
        HIP_CHECK(hipMemcpyAsync(aux_device_[aux_slot_], aux_staging_[aux_slot_], used * sizeof(int32_t),
                                 hipMemcpyHostToDevice, copy_stream_));
      }
      aux_slot_used_[aux_slot_] = true;
      aux_needs_upload_ = false;
    }
    hipEvent_t ev = aux_copied_[aux_slot_];
    HIP_CHECK(hipEventRecord(ev, copy_stream_));
    HIP_CHECK(hipStreamWaitEvent(compute_stream_, ev, 0));
    copy_stream_has_work_ = false;
  }

  // ---------------------------------------------------------------- configuration
  int64_t page_size_, num_layers_, layer_id_begin_offset_;
  int64_t num_qo_heads_, num_kv_heads_, qk_head_dim_, v_head_dim_;
  int64_t num_total_pages_ = 0, prefill_chunk_size_, reserved_num_seqs_ = 0;
  bool support_sliding_window_ = false;
  int elem_bits_ = 16;    // storage type of the MHA layers: 16 (fp16) or 32 (float32)
  bool generic_ = false;  // the MHA layers run on the typed / generic kernels (typed_kernels.h)
  int64_t layer_sliding_window_size_ = 1024;
  std::vector<int64_t> attn_kinds_;
  int rope_mode_ = TVMKV_ROPE_NORMAL;
  double rotary_scale_, rotary_theta_;

  // the frequency variant of the in-kernel RoPE: the attention kernels of a cache in inline-RoPE mode
  const tvmkv_rope_scaling* InlineScaling() const {
    return (has_rope_scaling_ && rope_mode_ == TVMKV_ROPE_INLINE) ? &rope_scaling_ : nullptr;
  }
  bool has_rope_scaling_ = false;
  tvmkv_rope_scaling rope_scaling_{};
  const float* rope_ext_factors_ = nullptr;

  std::unique_ptr<KVBookkeeper> book_;
  size_t page_copies_issued_ = 0;  // elements of the bookkeeper's copy log already on the copy stream

  // ---------------------------------------------------------------- device
  int device_;
  hipStream_t compute_stream_ = nullptr;
  hipStream_t copy_stream_ = nullptr;
  hipEvent_t compute_done_ = nullptr;
  bool compute_event_recorded_ = false;
  bool compute_work_since_event_ = false;
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
  bool aux_read_since_event_[2] = {false, false};
  bool aux_slot_used_[2] = {false, false};
  bool aux_needs_upload_ = false;
  int aux_slot_ = 0;
  int64_t commit_capacity_ = 0;
  void* commit_device_ = nullptr;
  void* commit_staging_ = nullptr;
  hipEvent_t commit_copied_ = nullptr;
  bool commit_staging_used_ = false;
};

}  // namespace tvmkv

// =========================================================================== C ABI
struct tvmkv_cache {
  std::unique_ptr<tvmkv::PagedKVCache> impl;
};

extern "C" {

const char* tvmkv_last_error(void) { return tvmkv::g_last_error.c_str(); }
const char* tvmkv_version(void) { return "tvmkv 0.2 (gfx950)"; }

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
      cache_config, n_config, layer_indptr[0], layer_indptr[1], num_qo_heads, num_kv_heads, qk_head_dim, v_head_dim,
      std::vector<int64_t>(attn_kinds, attn_kinds + n_attn_kinds), enable_kv_transfer != 0, rope_mode, rope_scale,
      rope_theta, dtype_bits, device_id);
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
int tvmkv_cache_set_rope_scaling(tvmkv_cache* cache, const tvmkv_rope_scaling* scaling, const float* rope_ext_factors) {
  KV_CACHE_FN(cache->impl->SetRopeScaling(scaling, rope_ext_factors));
}
int tvmkv_kv_state_clear(tvmkv_cache* cache) { KV_CACHE_FN(cache->impl->Clear()); }
int tvmkv_kv_state_add_sequence(tvmkv_cache* cache, int64_t seq_id) { KV_CACHE_FN(cache->impl->AddSequence(seq_id)); }
int tvmkv_kv_state_remove_sequence(tvmkv_cache* cache, int64_t seq_id) {
  KV_CACHE_FN(cache->impl->RemoveSequence(seq_id));
}
int tvmkv_kv_state_fork_sequence(tvmkv_cache* cache, int64_t parent_seq_id, int64_t child_seq_id, int64_t fork_pos) {
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
                                                      const void* qkv, int64_t qkv_rows, void* out, int64_t out_rows) {
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
int tvmkv_attention_kv_cache_debug_get_kv_mla(tvmkv_cache* cache, int64_t seq_id, int64_t start_pos, int64_t end_pos,
                                              void* kv_data) {
  KV_CACHE_FN(cache->impl->DebugGetKV(seq_id, start_pos, end_pos, kv_data, nullptr, /*mla=*/true));
}

int tvmkv_cache_get_aux(tvmkv_cache* cache, const char* name, int32_t depth, const int32_t** data, int64_t* size) {
  KV_CACHE_FN(cache->impl->GetAux(name, depth, data, size));
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
