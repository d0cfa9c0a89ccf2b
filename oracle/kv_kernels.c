/*
 * TEST INFRASTRUCTURE ONLY -- CPU restatement of the reference's llvm-target
 * KV-cache kernels.  Nothing in the shipped package may link or call this
 * file; it is the checker for the HIP kernels and the CPU baseline of the
 * benchmark.
 *
 * Every function follows one TVMScript kernel of the reference, statement by
 * statement (serial loops, fp16 storage, fp32 arithmetic, base-2 softmax,
 * online-softmax state initialised to m = -5e4, d = 1).  Citations are
 * file:line into the reference tree:
 *
 *   orc_fused_rope              python/tvm/relax/frontend/nn/llm/position_embedding.py:525-565
 *                               (frequency: :32-67, rotate-half term: :493-523)
 *   orc_transpose_append        python/tvm/relax/frontend/nn/llm/_page_kernels.py:40-74
 *   orc_transpose_append_mla    _page_kernels.py:77-103
 *   orc_debug_get_kv(_mla)      _page_kernels.py:106-166
 *   orc_copy_single_page(_mla)  _page_kernels.py:169-232
 *   orc_compact_kv_copy         _page_kernels.py:266-293
 *   orc_decode                  python/tvm/relax/frontend/nn/llm/_decode_kernels.py:49-178
 *   orc_merge_state_inplace     _decode_kernels.py:414-452
 *   orc_prefill_paged           python/tvm/relax/frontend/nn/llm/_prefill_kernels.py:54-214
 *   orc_prefill_ragged          _prefill_kernels.py:677-791
 *   orc_tree_attn_ragged        python/tvm/relax/frontend/nn/llm/tree_attn.py:93-259
 *   orc_tree_attn_paged         tree_attn.py:634-797 (mask: tree_attn.py:48-65)
 *   orc_prefill_paged_mla       _prefill_kernels.py:927-1071 (GPU-only kernel in the
 *                               reference; restated here row by row, see below)
 *   helpers                     python/tvm/relax/frontend/nn/llm/_kernel_common.py:115-170
 *
 * Parity pins (tests/test_oracle_*.py): RoPE against the numpy closed form of
 * the reference's own test (tests/python/relax/
 * test_runtime_builtin_paged_attention_kv_cache_cpu.py:305-324), attention
 * against softmax(QK^T*scale + causal mask)V with GQA head repeat (:499-535),
 * merge against the two-way log-sum-exp identity, append/gather by round trip.
 *
 * PARITY UNPINNED relative to "the reference's llvm kernels":
 *   orc_prefill_paged_mla -- the reference has no llvm MLA kernel
 *   (python/tvm/relax/frontend/nn/llm/kv_cache.py:676-677); this function is
 *   pinned to the mathematical definition (torch closed form of
 *   tests/python/relax/test_runtime_builtin_paged_attention_kv_cache_mla_tir.py:351-398)
 *   only.
 *
 * Deliberate deviations from the reference text, none of which changes a
 * result for valid inputs:
 *   - _prefill_kernels.py:162 loops row_idx over max_num_pages*page_size and
 *     guards with row_idx < kv_len; here the loop bound is kv_len.
 *   - _prefill_kernels.py:204 reads scale_O[d_idx] from a 1-element buffer;
 *     restated as scale_O[0].
 *   - new_m (:132) is an uninitialised allocation in the reference; it starts
 *     at m_val here (it only matters when the very first column of a row is
 *     masked out).
 */
#include <immintrin.h>
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* The reference builds every kernel for a storage dtype (its tests run "float16" and "float32",
 * tests/python/relax/test_runtime_builtin_paged_attention_kv_cache_cpu.py:269-276); arithmetic is float32
 * either way and results are cast to the storage type where the TIR kernels cast.  This file is compiled
 * twice: as it is for fp16 storage (liborc_kernels.so), and with -DORC_F32 for float32 storage
 * (liborc_kernels_f32.so), where `f16` names a float and the conversions are the identity. */
#ifdef ORC_F32
typedef float f16;
static inline float h2f(f16 h) { return h; }
static inline f16 f2h(float f) { return f; }
static inline f16 negated(f16 x) { return -x; }
#else
typedef uint16_t f16;

static inline float h2f(f16 h) { return _cvtsh_ss(h); }
static inline f16 f2h(float f) { return _cvtss_sh(f, _MM_FROUND_TO_NEAREST_INT | _MM_FROUND_NO_EXC); }
static inline f16 negated(f16 x) { return (f16)(x ^ 0x8000u); }
#endif

#define LOG2E_F ((float)1.4426950408889634) /* math.log2(math.exp(1)) */

/* ---- _kernel_common.py:155-170 ------------------------------------------------ */
static inline int kv_chunk_len(int num_pages, int page_size, int seq_id, const int32_t* length_info,
                               int B, int sliding_window) {
  if (num_pages == 0) return 0;
  if (!sliding_window) return (num_pages - 1) * page_size + length_info[seq_id];
  return (num_pages - 1) * page_size + length_info[seq_id] - length_info[B + seq_id] +
         length_info[2 * B + seq_id];
}

static inline int seq_offset(int pos, int seq_id, const int32_t* length_info, int B,
                             int sliding_window) {
  if (!sliding_window) return pos;
  int sink = length_info[2 * B + seq_id];
  return pos < sink ? pos : pos - sink + length_info[B + seq_id];
}

/* _kernel_common.py:130-144 */
static inline int causal_mask(int causal, int row, int col, int kv_len, int qo_len) {
  return causal > 0 ? (col < kv_len - qo_len + row + 1) : (col < kv_len);
}

static inline int causal_or_sliding_cross_mask(int causal, int row, int col, int kv_len, int qo_len,
                                               int sliding_window_size) {
  int visible_past = sliding_window_size - row - 1;
  if (visible_past < 0) visible_past = 0;
  if (causal > 0 && sliding_window_size > 0) {
    int lo = kv_len - visible_past;
    if (lo < 0) lo = 0;
    return col < kv_len && col >= lo;
  }
  return causal_mask(causal, row, col, kv_len, qo_len);
}

/* tree_attn.py:48-65: the last tree_order_len keys of the sequence are the nodes of its token tree;
 * tree_order holds (first, second) per node = its DFS order and the end of its subtree's range.
 * A query node sees every key before the tree and the tree nodes that are its ancestors or itself. */
static inline int check_tree_order(const int32_t* tree_order_indptr, const int32_t* tree_order,
                                   int batch, int row, int col, int kv_len, int qo_len) {
  int tree_order_len = tree_order_indptr[batch + 1] - tree_order_indptr[batch];
  int tree_start = kv_len - tree_order_len;
  int child_idx_in_tree = row + tree_order_len - qo_len;
  int parent_idx_in_tree = col - tree_start;
  if (!(col < kv_len)) return 0;
  if (col < tree_start) return 1;
  const int32_t* child = tree_order + 2 * (int64_t)(tree_order_indptr[batch] + child_idx_in_tree);
  const int32_t* parent = tree_order + 2 * (int64_t)(tree_order_indptr[batch] + parent_idx_in_tree);
  return child[0] >= parent[0] && child[0] < parent[1];
}

/* ---- RoPE (position_embedding.py:32-67 + _kernel_common.py:115-127) ----------- */
/* x points at element 0 of the head vector; returns the rotated element d,
 * rounded to fp16 exactly where the reference casts. */
static inline f16 rope_elem(const f16* x, int d, int rotary_dim, float pos_times_scale, float theta) {
  float freq = pos_times_scale / powf(theta, (float)((d * 2) % rotary_dim) / (float)rotary_dim);
  float c = cosf(freq) * h2f(x[d]);
  f16 other = d < rotary_dim / 2 ? negated(x[d + rotary_dim / 2]) : x[d - rotary_dim / 2];
  float s = sinf(freq) * h2f(other);
  return f2h(c + s);
}

void orc_fused_rope(const f16* qkv, const int32_t* position_map, f16* q, f16* k, f16* v,
                    int64_t seq_len, int num_q_heads, int num_kv_heads, int head_dim,
                    int rotary_dim, int64_t apply_rope, float theta, float scale) {
  int fused_heads = num_q_heads + 2 * num_kv_heads;
  for (int64_t s = 0; s < seq_len; ++s) {
    for (int h = 0; h < fused_heads; ++h) {
      const f16* x = qkv + (s * fused_heads + h) * head_dim;
      for (int d = 0; d < head_dim; ++d) {
        if (h < num_q_heads) {
          q[(s * num_q_heads + h) * head_dim + d] =
              (apply_rope > 0 && d < rotary_dim)
                  ? rope_elem(x, d, rotary_dim, (float)position_map[s] * scale, theta)
                  : x[d];
        } else if (h < num_q_heads + num_kv_heads) {
          k[(s * num_kv_heads + (h - num_q_heads)) * head_dim + d] =
              (apply_rope > 0 && d < rotary_dim)
                  ? rope_elem(x, d, rotary_dim, (float)position_map[s] * scale, theta)
                  : x[d];
        } else {
          v[(s * num_kv_heads + (h - num_q_heads - num_kv_heads)) * head_dim + d] = x[d];
        }
      }
    }
  }
}

/* ---- RoPE frequency variants (position_embedding.py:130-299) ------------------------
 * The reference compiles one of these into the kernel of a model.  Everything is float32 as in the
 * TIR expression (python constants become float32 immediates); the angle of element d at scaled
 * position s:
 *   default   s / theta^((2d mod R)/R)                                                      (:32-67)
 *   llama3    s * ((1-smooth)*f/factor + smooth*f), f = 1/theta^(..),
 *             smooth = clip(alpha*f - beta, 0, 1)                                           (:130-161)
 *   longrope  s / (ext[d mod R/2] * theta^(..)); cos and sin times
 *             sqrt(1 + ln(max/orig)/ln(orig)) when max > orig                               (:164-188)
 *   yarn      s * (inter*(1-mask) + extra*mask), extra = 1/theta^(..), inter = extra/factor,
 *             mask = 1 - clip((d - low)/(high - low), 0, 1) with d the ELEMENT index and the
 *             correction dims low/high not rounded (:191-255; the published YaRN code floors and
 *             ceils them and ramps over R/2 frequencies, the reference does neither)
 * Pins (tests/test_oracle_kernels.py): llama3 against the piecewise form of the Llama-3.1 release
 * (unchanged above the high-frequency wavelength, divided by `factor` below the low one, linear in
 * between); yarn against the published formula with its rounding removed and, for factor = 1,
 * against default; longrope with unit factors and max = orig against default, bit for bit. */
typedef struct {
  int32_t rope_type; /* 0 default, 1 llama3, 2 longrope, 3 yarn, 4 gptj, 5 llama4 */
  int32_t rotary_dim; /* 0 = head_dim */
  double factor, low_freq_factor, high_freq_factor, beta_fast, beta_slow;
  int64_t max_position_embeddings, original_max_position_embeddings;
} orc_rope_scaling;

/* angle and magnitude of element d; ext = the factor half to use or NULL */
float orc_rope_angle(const orc_rope_scaling* sc, float s, int d, int R, float theta, const float* ext,
                     float* magnitude) {
  float power = powf(theta, (float)((d * 2) % R) / (float)R);
  *magnitude = 1.0f;
  if (sc == NULL || sc->rope_type == 0) return s / power;
  if (sc->rope_type == 4) return s / powf(theta, (float)((2 * (d / 2)) % R) / (float)R); /* rope_freq_gptj, :70-76 */
  if (sc->rope_type == 5) { /* rope_freq_llama4, :79-127 */
    float orig = 1.0f / powf(theta, (float)(2 * (d / 2)) / (float)R);
    if (sc->high_freq_factor == sc->low_freq_factor) {
      float wavelength = (float)(2 * M_PI) / orig;
      float threshold = (float)((double)sc->original_max_position_embeddings / sc->low_freq_factor);
      return s * (wavelength > threshold ? orig / (float)sc->factor : orig);
    }
    double inv_diff = 1.0 / (sc->high_freq_factor - sc->low_freq_factor);
    float inv_factor = (float)(1.0 / sc->factor);
    float alpha = (float)((double)sc->original_max_position_embeddings / (2 * M_PI) * inv_diff);
    float beta = (float)(sc->low_freq_factor * inv_diff);
    float smooth = fmaxf(0.0f, fminf(1.0f, alpha * orig - beta));
    return s * ((1.0f - smooth) * orig * inv_factor + smooth * orig);
  }
  if (sc->rope_type == 1) {
    float orig = 1.0f / power;
    double inv_diff = 1.0 / (sc->high_freq_factor - sc->low_freq_factor);
    float inv_factor = (float)(1.0 / sc->factor);
    float alpha = (float)((double)sc->original_max_position_embeddings / (2 * M_PI) * inv_diff);
    float beta = (float)(sc->low_freq_factor * inv_diff);
    float smooth = fmaxf(0.0f, fminf(1.0f, alpha * orig - beta));
    return s * ((1.0f - smooth) * orig * inv_factor + smooth * orig);
  }
  if (sc->rope_type == 2) {
    double scale = (double)sc->max_position_embeddings / (double)sc->original_max_position_embeddings;
    if (scale > 1.0)
      *magnitude = (float)sqrt(1.0 + log(scale) / log((double)sc->original_max_position_embeddings));
    float divisor = power;
    if (ext != NULL) divisor = ext[d % (R / 2)] * divisor;
    return s / divisor;
  }
  double inv_theta_log_scale = 1.0 / (2.0 * log((double)theta)); /* kv_cache.py:363-365 */
  double lo = R * log((double)sc->original_max_position_embeddings / (sc->beta_fast * 2 * M_PI)) * inv_theta_log_scale;
  double hi = R * log((double)sc->original_max_position_embeddings / (sc->beta_slow * 2 * M_PI)) * inv_theta_log_scale;
  float low = (float)(lo > 0 ? lo : 0), high = (float)(hi < R - 1 ? hi : R - 1);
  if (low == high) high += 0.001f;
  float extra = 1.0f / power;
  float inter = 1.0f / ((float)sc->factor * power);
  float mask = 1.0f - fmaxf(fminf(((float)d - low) / (high - low), 1.0f), 0.0f);
  return s * (inter * (1.0f - mask) + extra * mask);
}

/* The RoPE of the attention kernels (_kernel_common.py:115-127): the whole head, rotate-half pairing,
 * the model's frequency variant baked in when the reference builds the kernel (rope_scaling argument of
 * the kernel factories, _decode_kernels.py:49,181; _prefill_kernels.py:54-60,217-223,677,795).  Here the
 * variant is a setting of the oracle library: NULL = default frequencies.  The attention kernels pass no
 * factor tensor, so longrope is the default frequencies times its magnitude (position_embedding.py:164-188). */
static const orc_rope_scaling* g_inline_scaling = NULL;
static orc_rope_scaling g_inline_scaling_copy;
void orc_set_inline_rope_scaling(const orc_rope_scaling* sc) {
  if (sc == NULL) {
    g_inline_scaling = NULL;
  } else {
    g_inline_scaling_copy = *sc;
    g_inline_scaling = &g_inline_scaling_copy;
  }
}
static inline f16 rope_elem_inline(const f16* x, int d, int D, float pos_times_scale, float theta) {
  if (g_inline_scaling == NULL) return rope_elem(x, d, D, pos_times_scale, theta);
  float magnitude;
  float freq = orc_rope_angle(g_inline_scaling, pos_times_scale, d, D, theta, NULL, &magnitude);
  float c = cosf(freq) * magnitude * h2f(x[d]);
  f16 other = d < D / 2 ? negated(x[d + D / 2]) : x[d - D / 2];
  float sn = sinf(freq) * magnitude * h2f(other);
  return f2h(c + sn);
}

/* fused_rope / fused_rope_longrope_scaling (position_embedding.py:525-667) with a frequency variant.
 * ext_factors: NULL or R floats, long factors then short ones; the long ones apply when
 * seq_len > original_max_position_embeddings (:601). */
void orc_fused_rope_scaled(const f16* qkv, const int32_t* position_map, f16* q, f16* k, f16* v,
                           int64_t seq_len, int num_q_heads, int num_kv_heads, int head_dim,
                           int64_t apply_rope, float theta, float scale, const orc_rope_scaling* sc,
                           const float* ext_factors) {
  int fused_heads = num_q_heads + 2 * num_kv_heads;
  int R = (sc != NULL && sc->rotary_dim > 0) ? sc->rotary_dim : head_dim; /* position_embedding.py:507-520 */
  const float* ext = ext_factors;
  if (ext != NULL && sc != NULL && !(seq_len > sc->original_max_position_embeddings)) ext += R / 2;
  for (int64_t s = 0; s < seq_len; ++s) {
    for (int h = 0; h < fused_heads; ++h) {
      const f16* x = qkv + (s * fused_heads + h) * head_dim;
      f16* dst = h < num_q_heads ? q + (s * num_q_heads + h) * head_dim
                 : h < num_q_heads + num_kv_heads
                     ? k + (s * num_kv_heads + (h - num_q_heads)) * head_dim
                     : v + (s * num_kv_heads + (h - num_q_heads - num_kv_heads)) * head_dim;
      for (int d = 0; d < head_dim; ++d) {
        if (h >= num_q_heads + num_kv_heads || !(apply_rope > 0) || d >= R) {
          dst[d] = x[d];
          continue;
        }
        float magnitude;
        float freq = orc_rope_angle(sc, (float)position_map[s] * scale, d, R, theta, ext, &magnitude);
        float c = (cosf(freq) * magnitude) * h2f(x[d]);
        f16 other = d < R / 2 ? negated(x[d + R / 2]) : x[d - R / 2];
        if (sc != NULL && sc->rope_type == 4) other = d % 2 == 0 ? negated(x[d + 1]) : x[d - 1]; /* :509-514 */
        float sn = (sinf(freq) * magnitude) * h2f(other);
        dst[d] = f2h(c + sn);
      }
    }
  }
}

/* ---- page kernels ------------------------------------------------------------ */
#define PAGE_AT(pages, Hkv, ps, D, page, kv, h, slot) \
  ((pages) + ((((int64_t)(page) * 2 + (kv)) * (Hkv) + (h)) * (ps) + (slot)) * (int64_t)(D))

void orc_transpose_append(f16* pages, const f16* k_data, const f16* v_data,
                          const int32_t* position_map, int64_t ntoken, int Hkv, int page_size,
                          int D) {
  for (int64_t g = 0; g < ntoken; ++g) {
    int32_t position = position_map[g];
    if (position == -1) continue;
    for (int h = 0; h < Hkv; ++h) {
      f16* kd = PAGE_AT(pages, Hkv, page_size, D, position / page_size, 0, h, position % page_size);
      f16* vd = PAGE_AT(pages, Hkv, page_size, D, position / page_size, 1, h, position % page_size);
      for (int f = 0; f < D; ++f) {
        kd[f] = k_data[(g * Hkv + h) * D + f];
        vd[f] = v_data[(g * Hkv + h) * D + f];
      }
    }
  }
}

void orc_transpose_append_mla(f16* pages, const f16* kv_data, const int32_t* position_map,
                              int64_t ntoken, int page_size, int d_qk) {
  for (int64_t g = 0; g < ntoken; ++g) {
    int32_t position = position_map[g];
    if (position == -1) continue;
    f16* dst = pages + ((int64_t)(position / page_size) * page_size + position % page_size) * d_qk;
    for (int f = 0; f < d_qk; ++f) dst[f] = kv_data[g * d_qk + f];
  }
}

void orc_debug_get_kv(const f16* pages, const int32_t* position_map, f16* k_data, f16* v_data,
                      int64_t layer_id, int64_t seqlen, int Hkv, int page_size, int D) {
  for (int64_t p = 0; p < seqlen; ++p) {
    int32_t position = position_map[p];
    for (int h = 0; h < Hkv; ++h) {
      const f16* ks = PAGE_AT(pages, Hkv, page_size, D, position / page_size, 0, h, position % page_size);
      const f16* vs = PAGE_AT(pages, Hkv, page_size, D, position / page_size, 1, h, position % page_size);
      int64_t o = ((layer_id * seqlen + p) * Hkv + h) * D;
      for (int d = 0; d < D; ++d) {
        k_data[o + d] = ks[d];
        v_data[o + d] = vs[d];
      }
    }
  }
}

void orc_debug_get_kv_mla(const f16* pages, const int32_t* position_map, f16* kv_data,
                          int64_t layer_id, int64_t seqlen, int page_size, int d_qk) {
  for (int64_t p = 0; p < seqlen; ++p) {
    int32_t position = position_map[p];
    const f16* src = pages + ((int64_t)(position / page_size) * page_size + position % page_size) * d_qk;
    for (int d = 0; d < d_qk; ++d) kv_data[(layer_id * seqlen + p) * d_qk + d] = src[d];
  }
}

void orc_copy_single_page(f16* pages, int64_t src_page_id, int64_t tgt_page_id, int64_t copy_length,
                          int Hkv, int page_size, int D) {
  int64_t total = copy_length * Hkv * D;
  for (int64_t i = 0; i < total; ++i) {
    int vh = (int)(i / (copy_length * D));
    int vp = (int)(i % (copy_length * D) / D);
    int vd = (int)(i % D);
    PAGE_AT(pages, Hkv, page_size, D, tgt_page_id, 0, vh, vp)[vd] =
        PAGE_AT(pages, Hkv, page_size, D, src_page_id, 0, vh, vp)[vd];
    PAGE_AT(pages, Hkv, page_size, D, tgt_page_id, 1, vh, vp)[vd] =
        PAGE_AT(pages, Hkv, page_size, D, src_page_id, 1, vh, vp)[vd];
  }
}

void orc_copy_single_page_mla(f16* pages, int64_t src_page_id, int64_t tgt_page_id,
                              int64_t copy_length, int page_size, int d_qk) {
  for (int64_t i = 0; i < copy_length * d_qk; ++i) {
    int64_t vp = i / d_qk, vd = i % d_qk;
    pages[(tgt_page_id * page_size + vp) * d_qk + vd] = pages[(src_page_id * page_size + vp) * d_qk + vd];
  }
}

void orc_compact_kv_copy(f16* pages, const int32_t* copy_length_indptr, const int32_t* copy_src_dst_pos,
                         int32_t batch_size, int32_t total_copy_length, int Hkv, int page_size, int D) {
  for (int b = 0; b < batch_size; ++b)
    for (int h = 0; h < Hkv; ++h)
      for (int d = 0; d < D; ++d)
        for (int i = 0; i < copy_length_indptr[b + 1] - copy_length_indptr[b]; ++i) {
          int32_t src_pos = copy_src_dst_pos[copy_length_indptr[b] + i];
          int32_t dst_pos = copy_src_dst_pos[total_copy_length + copy_length_indptr[b] + i];
          PAGE_AT(pages, Hkv, page_size, D, dst_pos / page_size, 0, h, dst_pos % page_size)[d] =
              PAGE_AT(pages, Hkv, page_size, D, src_pos / page_size, 0, h, src_pos % page_size)[d];
          PAGE_AT(pages, Hkv, page_size, D, dst_pos / page_size, 1, h, dst_pos % page_size)[d] =
              PAGE_AT(pages, Hkv, page_size, D, src_pos / page_size, 1, h, src_pos % page_size)[d];
        }
}

/* ---- batch_decode_paged_kv_cpu (_decode_kernels.py:103-176) -------------------- */
void orc_decode(const f16* Q, const f16* pages, const int32_t* page_table_indptr,
                const int32_t* page_table_values, const int32_t* length_info,
                const int32_t* k_rope_pos_offset, const int32_t* q_rope_position, f16* output,
                float* lse, int B, int H_qo, int H_kv, int D, int page_size, int sliding_window,
                int rotary_mode, float rope_scale, float rope_theta, float sm_scale) {
  int group_size = H_qo / H_kv;
  float* O_local = (float*)malloc(sizeof(float) * D * 4);
  float *Q_local = O_local + D, *K_local = Q_local + D, *V_local = K_local + D;
  for (int b = 0; b < B; ++b) {
    int begin = page_table_indptr[b], end = page_table_indptr[b + 1];
    int kv_len = kv_chunk_len(end - begin, page_size, b, length_info, B, sliding_window);
    for (int h_qo = 0; h_qo < H_qo; ++h_qo) {
      float m_val = -5e4f, d_val = 1.0f;
      const f16* qrow = Q + ((int64_t)b * H_qo + h_qo) * D;
      for (int d = 0; d < D; ++d) O_local[d] = 0.0f;
      for (int d = 0; d < D; ++d)
        Q_local[d] = rotary_mode == 1
                         ? h2f(rope_elem_inline(qrow, d, D, (float)q_rope_position[b] * rope_scale, rope_theta))
                         : h2f(qrow[d]);
      for (int row_idx = 0; row_idx < kv_len; ++row_idx) {
        int so = seq_offset(row_idx, b, length_info, B, sliding_window);
        int page_no = page_table_values[begin + so / page_size];
        int page_offset = so % page_size;
        const f16* krow = PAGE_AT(pages, H_kv, page_size, D, page_no, 0, h_qo / group_size, page_offset);
        const f16* vrow = PAGE_AT(pages, H_kv, page_size, D, page_no, 1, h_qo / group_size, page_offset);
        for (int d = 0; d < D; ++d)
          K_local[d] = rotary_mode == 1
                           ? h2f(rope_elem_inline(krow, d, D, (float)(k_rope_pos_offset[b] + row_idx) * rope_scale, rope_theta))
                           : h2f(krow[d]);
        float S_val = 0.0f;
        for (int d = 0; d < D; ++d) S_val += Q_local[d] * K_local[d];
        S_val *= sm_scale * LOG2E_F;
        float new_m = fmaxf(m_val, S_val);
        d_val = d_val * exp2f(m_val - new_m) + exp2f(S_val - new_m);
        float scale_O = exp2f(m_val - new_m);
        for (int d = 0; d < D; ++d) O_local[d] = O_local[d] * scale_O;
        m_val = new_m;
        for (int d = 0; d < D; ++d) V_local[d] = h2f(vrow[d]);
        float factor = exp2f(S_val - m_val);
        for (int d = 0; d < D; ++d) O_local[d] = O_local[d] + V_local[d] * factor;
      }
      for (int d = 0; d < D; ++d) {
        O_local[d] = O_local[d] / d_val;
        output[((int64_t)b * H_qo + h_qo) * D + d] = f2h(O_local[d]);
      }
      lse[(int64_t)b * H_qo + h_qo] = m_val + log2f(d_val);
    }
  }
  free(O_local);
}

/* ---- merge_state_inplace_cpu (_decode_kernels.py:432-450) ---------------------- */
void orc_merge_state_inplace(f16* V, float* S, const f16* V_other, const float* S_other, int64_t N,
                             int H, int D) {
  for (int64_t n = 0; n < N; ++n)
    for (int h = 0; h < H; ++h) {
      float s_val = S[n * H + h], s_other_val = S_other[n * H + h];
      float s_max = fmaxf(s_val, s_other_val);
      s_val = exp2f(s_val - s_max);
      s_other_val = exp2f(s_other_val - s_max);
      float scale = s_val / (s_val + s_other_val);
      float other_scale = s_other_val / (s_val + s_other_val);
      for (int d = 0; d < D; ++d) {
        int64_t i = (n * H + h) * D + d;
        V[i] = f2h(h2f(V[i]) * scale + h2f(V_other[i]) * other_scale);
      }
      S[n * H + h] = log2f(s_val + s_other_val) + s_max;
    }
}

/* ---- batch_prefill_paged_kv_cpu (_prefill_kernels.py:121-213) ------------------ */
/* tree_order_indptr == NULL: batch_prefill_paged_kv_cpu.  Otherwise tree_attn_paged_kv_cpu
 * (tree_attn.py:634-797), which is the same loop nest with _check_tree_order as its mask. */
static void prefill_paged_impl(const f16* q, const int32_t* q_indptr, const f16* pages,
                               const int32_t* page_indptr, const int32_t* page_values,
                               const int32_t* length_info, const int32_t* k_rope_pos_offset,
                               const int32_t* q_rope_position, f16* output, float* lse, int batch_size,
                               int h_q, int h_kv, int d, int page_size, int sliding_window,
                               int sliding_window_size, int causal, int rotary_mode, float rope_scale,
                               float rope_theta, float sm_scale, const int32_t* tree_order_indptr,
                               const int32_t* tree_order) {
  int group_size = h_q / h_kv;
  float* O_local = (float*)malloc(sizeof(float) * d * 4);
  float *Q_local = O_local + d, *K_local = Q_local + d, *V_local = K_local + d;
  for (int h_qo = 0; h_qo < h_q; ++h_qo) {
    for (int b_idx = 0; b_idx < batch_size; ++b_idx) {
      int begin = page_indptr[b_idx], end = page_indptr[b_idx + 1];
      int kv_len = kv_chunk_len(end - begin, page_size, b_idx, length_info, batch_size, sliding_window);
      int qo_len = q_indptr[b_idx + 1] - q_indptr[b_idx];
      /* new_m lives across the query rows of a sequence as in the reference (_prefill_kernels.py:192-201
       * never resets it): a row that sees no key at all -- rows from sliding_window_size - 1 on under the
       * per-layer window mask -- is scaled by the previous row's maximum and ends as 0 / 0.  The tests
       * leave such rows out of the comparison and pin the library's answer for them (out 0, lse -5e4). */
      float new_m = -5e4f;
      for (int q_idx = 0; q_idx < qo_len; ++q_idx) {
        float m_val = -5e4f, d_val = 1.0f;
        if (q_idx == 0) new_m = m_val;
        for (int i = 0; i < d; ++i) O_local[i] = 0.0f;
        int curl_q = q_indptr[b_idx] + q_idx;
        const f16* qrow = q + ((int64_t)curl_q * h_q + h_qo) * d;
        for (int i = 0; i < d; ++i)
          Q_local[i] = rotary_mode == 1
                           ? h2f(rope_elem_inline(qrow, i, d, (float)q_rope_position[curl_q] * rope_scale, rope_theta))
                           : h2f(qrow[i]);
        for (int row_idx = 0; row_idx < kv_len; ++row_idx) {
          int so = seq_offset(row_idx, b_idx, length_info, batch_size, sliding_window);
          int page_no = page_values[begin + so / page_size];
          int page_offset = so % page_size;
          const f16* krow = PAGE_AT(pages, h_kv, page_size, d, page_no, 0, h_qo / group_size, page_offset);
          const f16* vrow = PAGE_AT(pages, h_kv, page_size, d, page_no, 1, h_qo / group_size, page_offset);
          for (int i = 0; i < d; ++i) {
            K_local[i] = rotary_mode == 1
                             ? h2f(rope_elem_inline(krow, i, d, (float)(k_rope_pos_offset[b_idx] + row_idx) * rope_scale, rope_theta))
                             : h2f(krow[i]);
            V_local[i] = h2f(vrow[i]);
          }
          float S_val = 0.0f;
          for (int i = 0; i < d; ++i) S_val += Q_local[i] * K_local[i];
          S_val *= sm_scale * LOG2E_F;
          int visible = tree_order_indptr
                            ? check_tree_order(tree_order_indptr, tree_order, b_idx, q_idx, row_idx, kv_len, qo_len)
                            : causal_or_sliding_cross_mask(causal, q_idx, row_idx, kv_len, qo_len,
                                                           sliding_window ? sliding_window_size : 0);
          if (visible) {
            new_m = fmaxf(m_val, S_val);
          } else {
            S_val = -5e4f;
          }
          d_val *= exp2f(m_val - new_m);
          d_val += exp2f(S_val - new_m);
          float scale_O = exp2f(m_val - new_m);
          m_val = new_m;
          float factor = exp2f(S_val - m_val);
          for (int i = 0; i < d; ++i) O_local[i] = O_local[i] * scale_O;
          for (int i = 0; i < d; ++i) O_local[i] += V_local[i] * factor;
        }
        for (int i = 0; i < d; ++i) {
          O_local[i] = O_local[i] / d_val;
          output[((int64_t)curl_q * h_q + h_qo) * d + i] = f2h(O_local[i]);
        }
        lse[(int64_t)curl_q * h_q + h_qo] = m_val + log2f(d_val);
      }
    }
  }
  free(O_local);
}

void orc_prefill_paged(const f16* q, const int32_t* q_indptr, const f16* pages,
                       const int32_t* page_indptr, const int32_t* page_values,
                       const int32_t* length_info, const int32_t* k_rope_pos_offset,
                       const int32_t* q_rope_position, f16* output, float* lse, int batch_size,
                       int h_q, int h_kv, int d, int page_size, int sliding_window,
                       int sliding_window_size, int causal, int rotary_mode, float rope_scale,
                       float rope_theta, float sm_scale) {
  prefill_paged_impl(q, q_indptr, pages, page_indptr, page_values, length_info, k_rope_pos_offset,
                     q_rope_position, output, lse, batch_size, h_q, h_kv, d, page_size, sliding_window,
                     sliding_window_size, causal, rotary_mode, rope_scale, rope_theta, sm_scale, NULL, NULL);
}

/* tree_attn_paged_kv_cpu (tree_attn.py:634-797); the reference asserts rotary_mode == 0 (:700-702) */
void orc_tree_attn_paged(const f16* q, const int32_t* q_indptr, const f16* pages,
                         const int32_t* page_indptr, const int32_t* page_values,
                         const int32_t* length_info, const int32_t* k_rope_pos_offset,
                         const int32_t* q_rope_position, f16* output, float* lse, int batch_size,
                         int h_q, int h_kv, int d, int page_size, int sliding_window, int rotary_mode,
                         float rope_scale, float rope_theta, float sm_scale,
                         const int32_t* tree_order_indptr, const int32_t* tree_order) {
  prefill_paged_impl(q, q_indptr, pages, page_indptr, page_values, length_info, k_rope_pos_offset,
                     q_rope_position, output, lse, batch_size, h_q, h_kv, d, page_size, sliding_window, 0, 0,
                     rotary_mode, rope_scale, rope_theta, sm_scale, tree_order_indptr, tree_order);
}

/* ---- batch_prefill_ragged_kv (cpu) (_prefill_kernels.py:715-790) ----------------
 * mn_indptr == NULL: the causal kernel.  Otherwise tree_attn_cpu (tree_attn.py:93-259): the same
 * two-pass loop nest with _check_tree_order as its mask; under inline RoPE its keys are rotated to
 * q_rope_position[kv_indptr[b] + k_idx] (:207-219) instead of k_rope_pos_offset[b] + k_idx. */
static void prefill_ragged_impl(const f16* q, const int32_t* q_indptr, const f16* k, const f16* v,
                                const int32_t* kv_indptr, const int32_t* q_rope_position,
                                const int32_t* k_rope_pos_offset, f16* output, float* lse, int batch_size,
                                int h_q, int h_kv, int d_qk, int d_v, int causal, int rotary_mode,
                                float rope_scale, float rope_theta, float sm_scale,
                                const int32_t* mn_indptr, const int32_t* mask) {
  int group_size = h_q / h_kv;
  int max_kv = 1;
  for (int b = 0; b < batch_size; ++b)
    if (kv_indptr[b + 1] - kv_indptr[b] > max_kv) max_kv = kv_indptr[b + 1] - kv_indptr[b];
  float* attention_scores = (float*)malloc(sizeof(float) * (size_t)max_kv * h_q * 2);
  float* exp_scores = attention_scores + (size_t)max_kv * h_q;
  float* hbuf = (float*)malloc(sizeof(float) * (h_q * 6 + d_v + d_qk));
  float *softmax_sum = hbuf, *m_prev = hbuf + h_q, *m_new = hbuf + 2 * h_q, *d_prev = hbuf + 3 * h_q,
        *d_new = hbuf + 4 * h_q, *max_score = hbuf + 5 * h_q, *p_sum = hbuf + 6 * h_q,
        *qbuf = hbuf + 6 * h_q + d_v;
  for (int b = 0; b < batch_size; ++b) {
    int qo_len = q_indptr[b + 1] - q_indptr[b];
    int kv_len = kv_indptr[b + 1] - kv_indptr[b];
    for (int q_idx = 0; q_idx < qo_len; ++q_idx) {
      for (int i = 0; i < h_q; ++i) {
        max_score[i] = -5e4f;
        m_prev[i] = -5e4f;
        d_prev[i] = 1.0f;
        m_new[i] = -5e4f; /* never read before the k loop assigns it when kv_len > 0 */
      }
      for (int h = 0; h < h_q; ++h) {
        int h_kv_idx = h / group_size;
        const f16* qrow = q + ((int64_t)(q_indptr[b] + q_idx) * h_q + h) * d_qk;
        for (int i = 0; i < d_qk; ++i)
          qbuf[i] = rotary_mode == 1
                        ? h2f(rope_elem_inline(qrow, i, d_qk, (float)q_rope_position[q_indptr[b] + q_idx] * rope_scale, rope_theta))
                        : h2f(qrow[i]);
        for (int k_idx = 0; k_idx < kv_len; ++k_idx) {
          float attention_score;
          int visible = mn_indptr ? check_tree_order(mn_indptr, mask, b, q_idx, k_idx, kv_len, qo_len)
                                  : causal_mask(causal, q_idx, k_idx, kv_len, qo_len);
          if (visible) {
            const f16* krow = k + ((int64_t)(kv_indptr[b] + k_idx) * h_kv + h_kv_idx) * d_qk;
            float result = 0.0f;
            int k_pos = rotary_mode != 1 ? 0
                        : (mn_indptr ? q_rope_position[kv_indptr[b] + k_idx] : k_rope_pos_offset[b] + k_idx);
            for (int i = 0; i < d_qk; ++i) {
              float key_val = rotary_mode == 1
                                  ? h2f(rope_elem_inline(krow, i, d_qk, (float)k_pos * rope_scale, rope_theta))
                                  : h2f(krow[i]);
              result += qbuf[i] * key_val;
            }
            attention_score = result * LOG2E_F * sm_scale;
          } else {
            attention_score = -5e4f * LOG2E_F * sm_scale;
          }
          attention_scores[(size_t)k_idx * h_q + h] = attention_score;
          max_score[h] = fmaxf(max_score[h], attention_score);
          m_new[h] = fmaxf(m_prev[h], max_score[h]);
        }
      }
      for (int h = 0; h < h_q; ++h) d_new[h] = d_prev[h] * exp2f(m_prev[h] - m_new[h]);
      for (int h = 0; h < h_q; ++h) {
        softmax_sum[h] = 0.0f;
        for (int k_idx = 0; k_idx < kv_len; ++k_idx) {
          exp_scores[(size_t)k_idx * h_q + h] = exp2f(attention_scores[(size_t)k_idx * h_q + h] - m_new[h]);
          softmax_sum[h] += exp_scores[(size_t)k_idx * h_q + h];
        }
        d_new[h] += softmax_sum[h];
      }
      for (int h = 0; h < h_q; ++h) {
        int h_kv_idx = h / group_size;
        for (int i = 0; i < d_v; ++i) p_sum[i] = 0.0f;
        for (int v_idx = 0; v_idx < kv_len; ++v_idx) {
          float weight = exp_scores[(size_t)v_idx * h_q + h] / d_new[h];
          const f16* vrow = v + ((int64_t)(kv_indptr[b] + v_idx) * h_kv + h_kv_idx) * d_v;
          for (int i = 0; i < d_v; ++i) p_sum[i] += h2f(vrow[i]) * weight;
        }
        for (int i = 0; i < d_v; ++i)
          output[((int64_t)(q_indptr[b] + q_idx) * h_q + h) * d_v + i] = f2h(p_sum[i]);
        lse[(int64_t)(q_indptr[b] + q_idx) * h_q + h] = m_new[h] + log2f(d_new[h]);
      }
    }
  }
  free(attention_scores);
  free(hbuf);
}

void orc_prefill_ragged(const f16* q, const int32_t* q_indptr, const f16* k, const f16* v,
                        const int32_t* kv_indptr, const int32_t* q_rope_position,
                        const int32_t* k_rope_pos_offset, f16* output, float* lse, int batch_size,
                        int h_q, int h_kv, int d_qk, int d_v, int causal, int rotary_mode,
                        float rope_scale, float rope_theta, float sm_scale) {
  prefill_ragged_impl(q, q_indptr, k, v, kv_indptr, q_rope_position, k_rope_pos_offset, output, lse, batch_size,
                      h_q, h_kv, d_qk, d_v, causal, rotary_mode, rope_scale, rope_theta, sm_scale, NULL, NULL);
}

/* tree_attn_cpu (tree_attn.py:93-259) */
void orc_tree_attn_ragged(const f16* q, const int32_t* q_indptr, const f16* k, const f16* v,
                          const int32_t* kv_indptr, const int32_t* q_rope_position,
                          const int32_t* mn_indptr, const int32_t* mask, f16* output, float* lse,
                          int batch_size, int h_q, int h_kv, int d, int rotary_mode, float rope_scale,
                          float rope_theta, float sm_scale) {
  prefill_ragged_impl(q, q_indptr, k, v, kv_indptr, q_rope_position, NULL, output, lse, batch_size, h_q, h_kv, d,
                      d, 0, rotary_mode, rope_scale, rope_theta, sm_scale, mn_indptr, mask);
}

/* ---- batch_prefill_paged_kv_mla (_prefill_kernels.py:979-1064) ------------------
 * The reference only has the tiled GPU form.  Per output row its arithmetic is:
 * S = sum_j q[j]*kv[j] over all d_qk features, scaled by sm_scale*log2(e); online
 * softmax per tile with masked entries contributing exp2(-5e4 - m); O accumulates
 * p * kv[:d_latent]; out = O/d, lse = m + log2 d.  Restated here one key row at a
 * time (tile size 1), which is the same recurrence the llvm decode kernel uses. */
void orc_prefill_paged_mla(const f16* q, const int32_t* q_indptr, const f16* pages,
                           const int32_t* page_indptr, const int32_t* page_values,
                           const int32_t* length_info, f16* output, float* lse, int batch_size,
                           int h_q, int d_latent, int d_rope, int page_size, int sliding_window,
                           int causal, float sm_scale) {
  int d_qk = d_latent + d_rope;
  float* O_local = (float*)malloc(sizeof(float) * (d_latent + d_qk));
  float* Q_local = O_local + d_latent;
  for (int b_idx = 0; b_idx < batch_size; ++b_idx) {
    int begin = page_indptr[b_idx], end = page_indptr[b_idx + 1];
    int kv_len = kv_chunk_len(end - begin, page_size, b_idx, length_info, batch_size, sliding_window);
    int qo_len = q_indptr[b_idx + 1] - q_indptr[b_idx];
    for (int q_idx = 0; q_idx < qo_len; ++q_idx) {
      int cur_L = q_indptr[b_idx] + q_idx;
      for (int h = 0; h < h_q; ++h) {
        float m_val = -5e4f, d_val = 1.0f;
        for (int i = 0; i < d_latent; ++i) O_local[i] = 0.0f;
        for (int i = 0; i < d_qk; ++i) Q_local[i] = h2f(q[((int64_t)cur_L * h_q + h) * d_qk + i]);
        for (int row_idx = 0; row_idx < kv_len; ++row_idx) {
          int so = seq_offset(row_idx, b_idx, length_info, batch_size, sliding_window);
          int page_no = page_values[begin + so / page_size];
          const f16* kvrow = pages + ((int64_t)page_no * page_size + so % page_size) * d_qk;
          float S_val = 0.0f;
          for (int i = 0; i < d_qk; ++i) S_val += Q_local[i] * h2f(kvrow[i]);
          S_val *= sm_scale * LOG2E_F;
          float m_prev = m_val;
          if (causal_mask(causal, q_idx, row_idx, kv_len, qo_len)) {
            m_val = fmaxf(m_val, S_val);
          } else {
            S_val = -5e4f;
          }
          float p = exp2f(S_val - m_val);
          float o_scale = exp2f(m_prev - m_val);
          d_val = d_val * o_scale + p;
          for (int i = 0; i < d_latent; ++i) O_local[i] = O_local[i] * o_scale + p * h2f(kvrow[i]);
        }
        for (int i = 0; i < d_latent; ++i)
          output[((int64_t)cur_L * h_q + h) * d_latent + i] = f2h(O_local[i] / d_val);
        lse[(int64_t)cur_L * h_q + h] = m_val + log2f(d_val);
      }
    }
  }
  free(O_local);
}

/* ---- OpenMP-free helper for the benchmark: run orc_decode on a sub-range of the
 * batch so that several host threads can be timed side by side. ------------------ */
void orc_decode_range(const f16* Q, const f16* pages, const int32_t* page_table_indptr,
                      const int32_t* page_table_values, const int32_t* length_info,
                      const int32_t* k_rope_pos_offset, const int32_t* q_rope_position, f16* output,
                      float* lse, int b_begin, int b_end, int B, int H_qo, int H_kv, int D,
                      int page_size, float sm_scale) {
  /* Non-sliding, rotary_mode 0 only: each batch row is independent, so calling the
   * literal kernel on a one-row view gives the same numbers as the full call. */
  for (int b = b_begin; b < b_end; ++b) {
    int32_t indptr[2] = {page_table_indptr[b], page_table_indptr[b + 1]};
    orc_decode(Q + (int64_t)b * H_qo * D, pages, indptr, page_table_values, length_info + b,
               k_rope_pos_offset + b, q_rope_position + b, output + (int64_t)b * H_qo * D,
               lse + (int64_t)b * H_qo, 1, H_qo, H_kv, D, page_size, 0, 0, 1.0f, 1e4f, sm_scale);
  }
}
