// DLPack-level entry points (include/tvmkv_dlpack.h): one per kernel slot of the reference's cache,
// in the slot's own argument order.  Each validates its tensors, resolves `data + byte_offset`, reads
// the shapes out of the tensors and calls the pointer-level launcher of include/tvmkv.h.
#include <hip/hip_runtime_api.h>

#include <initializer_list>

#include "../../include/tvmkv_dlpack.h"
#include "common.h"
#include "typed_kernels.h"

namespace tvmkv {
namespace {

// kStorage: the storage type of an MHA cache, float16 or float32 (the reference builds its kernels for either)
enum Kind { kF16, kF32, kI32, kStorage };

const char* KindName(Kind kind) {
  return kind == kF16 ? "float16" : kind == kF32 ? "float32" : kind == kI32 ? "int32" : "float16 or float32";
}

// One validated tensor argument.
struct Arg {
  const DLTensor* t;
  const char* name;
  int64_t dim(int i) const { return t->shape[i]; }
  int ndim() const { return t->ndim; }
  void* ptr() const { return static_cast<char*>(t->data) + t->byte_offset; }
  const int32_t* i32() const { return static_cast<const int32_t*>(ptr()); }
  float* f32() const { return static_cast<float*>(ptr()); }
};

// Checks shared by every tensor: present, on a ROCm device, dtype, compact layout, alignment.
Arg Take(const DLTensor* t, const char* name, Kind kind, std::initializer_list<int> ndims) {
  KV_CHECK(t != nullptr) << name << " is NULL";
  KV_CHECK(t->device.device_type == kDLROCM)
      << name << " must be a ROCm device tensor (device_type " << static_cast<int>(kDLROCM) << "), got device_type "
      << t->device.device_type;
  const uint8_t code = kind == kI32 ? kDLInt : kDLFloat;
  const uint8_t bits = kind == kF16 ? 16 : kind == kStorage ? t->dtype.bits : 32;
  KV_CHECK(t->dtype.code == code && t->dtype.bits == bits && (bits == 16 || bits == 32) && t->dtype.lanes == 1)
      << name << " must be " << KindName(kind) << ", got dtype (code " << static_cast<int>(t->dtype.code) << ", bits "
      << static_cast<int>(t->dtype.bits) << ", lanes " << t->dtype.lanes << ")";
  bool ndim_ok = false;
  for (int n : ndims) ndim_ok |= (t->ndim == n);
  KV_CHECK(ndim_ok) << name << " has " << t->ndim << " dimensions, expected " << *ndims.begin()
                    << (ndims.size() > 1 ? " (or another listed form)" : "");
  KV_CHECK(t->ndim == 0 || t->shape != nullptr) << name << " has no shape";
  int64_t elements = 1;
  for (int i = 0; i < t->ndim; ++i) {
    KV_CHECK(t->shape[i] >= 0) << name << " has a negative extent";
    elements *= t->shape[i];
  }
  if (t->strides != nullptr) {
    int64_t expect = 1;
    for (int i = t->ndim - 1; i >= 0; --i) {
      KV_CHECK(t->shape[i] == 1 || t->strides[i] == expect)
          << name << " must be compact row-major (stride " << t->strides[i] << " at dimension " << i << ", expected "
          << expect << ")";
      expect *= t->shape[i];
    }
  }
  KV_CHECK(elements == 0 || t->data != nullptr) << name << " has no data";
  const uintptr_t address = reinterpret_cast<uintptr_t>(t->data) + t->byte_offset;
  const uintptr_t alignment = (kind == kF16 || kind == kStorage) ? 16 : 4;  // K/V/q rows are read 16 bytes at a time
  KV_CHECK(address % alignment == 0) << name << " (data + byte_offset) must be aligned to " << alignment << " bytes";
  return Arg{t, name};
}

// The storage type of a call: every kStorage tensor has the same one; returns its width in bits.
int StorageBits(std::initializer_list<Arg> args) {
  const Arg& first = *args.begin();
  for (const Arg& a : args) {
    KV_CHECK(a.t->dtype.bits == first.t->dtype.bits)
        << a.name << " is float" << static_cast<int>(a.t->dtype.bits) << " but " << first.name << " is float"
        << static_cast<int>(first.t->dtype.bits);
  }
  return first.t->dtype.bits;
}
// float32 storage runs on the generic kernels, which have no in-kernel RoPE over a token tree in the page pool
// (the reference's kernel asserts the same, tree_attn.py:700-702)
void NoRotaryTreeOverPages(int bits, int64_t rotary_mode, const char* what) {
  if (bits == 32 && rotary_mode != 0) {
    Thrower t(TVMKV_EUNSUPPORTED, "");
    t << what << ": RoPE inside the kernel is not built for token trees over the page pool";
    t.Throw();
  }
}

// All tensors of a call live on one device; returns its id.
int SameDevice(std::initializer_list<Arg> args) {
  const Arg& first = *args.begin();
  for (const Arg& a : args) {
    KV_CHECK(a.t->device.device_id == first.t->device.device_id)
        << a.name << " is on device " << a.t->device.device_id << " but " << first.name << " is on device "
        << first.t->device.device_id;
  }
  return first.t->device.device_id;
}

void Expect(bool ok, const Arg& a, const char* what) {
  if (ok) return;
  Thrower t(TVMKV_EINVAL, "");
  t << a.name << " has shape (";
  for (int i = 0; i < a.ndim(); ++i) t << (i ? ", " : "") << a.dim(i);
  t << "), expected " << what;
  t.Throw();
}

// Every check has passed: the tensors' device becomes current and the launcher runs.
template <typename F>
void Launch(int device, F&& launcher) {
  HIP_CHECK(hipSetDevice(device));
  const int rc = launcher();
  if (rc != TVMKV_OK) throw Error(rc, tvmkv_last_error());
}

// length_info: (batch,) selects the plain kernels, (3, batch) the sliding-window ones.
int SlidingForm(const Arg& length_info, int64_t batch) {
  if (length_info.ndim() == 1) {
    Expect(length_info.dim(0) == batch, length_info, "(batch,)");
    return 0;
  }
  Expect(length_info.dim(0) == 3 && length_info.dim(1) == batch, length_info, "(3, batch)");
  return 1;
}

// What the paged MHA kernels share: q (rows, h_q, d), pages (num_pages, 2, h_kv, page_size, d), the
// page table of `batch` entries, out and lse of the query rows.
struct PagedShapes {
  int64_t rows, batch, nnz_pages, num_pages;
  int32_t h_q, h_kv, d, page_size;
  int sliding;
};
PagedShapes CheckPaged(const Arg& q, const Arg& pages, const Arg& page_indptr, const Arg& page_indices,
                       const Arg& length_info, const Arg& k_rope_pos_offset, const Arg& q_rope_position,
                       const Arg& out, const Arg& lse) {
  PagedShapes s;
  s.rows = q.dim(0);
  s.h_q = static_cast<int32_t>(q.dim(1));
  s.d = static_cast<int32_t>(q.dim(2));
  Expect(pages.dim(1) == 2 && pages.dim(4) == s.d, pages, "(num_pages, 2, h_kv, page_size, head_dim of q)");
  s.num_pages = pages.dim(0);
  s.h_kv = static_cast<int32_t>(pages.dim(2));
  s.page_size = static_cast<int32_t>(pages.dim(3));
  Expect(page_indptr.dim(0) >= 1, page_indptr, "(batch + 1,)");
  s.batch = page_indptr.dim(0) - 1;
  s.nnz_pages = page_indices.dim(0);
  s.sliding = SlidingForm(length_info, s.batch);
  Expect(k_rope_pos_offset.dim(0) == s.batch, k_rope_pos_offset, "(batch,)");
  Expect(q_rope_position.dim(0) >= s.rows, q_rope_position, "(at least the rows of q,)");
  Expect(out.dim(0) == s.rows && out.dim(1) == s.h_q && out.dim(2) == s.d, out, "the shape of q");
  Expect(lse.dim(0) == s.rows && lse.dim(1) == s.h_q, lse, "(rows of q, h_q)");
  return s;
}

// The paged MHA slots on float32 storage: the generic kernel.
GenericAttention PagedGeneric(const char* what, const PagedShapes& s, const Arg& q, const Arg* qo_indptr, const Arg& pages,
                              const Arg& page_indptr, const Arg& page_indices, const Arg& length_info, const Arg& k_off,
                              const Arg& q_pos, const Arg& out, const Arg& lse, int64_t causal, int64_t rotary_mode,
                              double rope_scale, double rope_theta, const tvmkv_rope_scaling* rope_scaling,
                              int64_t layer_window, double sm_scale) {
  GenericAttention a;
  a.what = what;
  a.sliding_window = s.sliding;
  a.layer_window = static_cast<int32_t>(layer_window);
  a.rotary_mode = rotary_mode;
  a.q_rope_position = q_pos.i32();
  a.k_rope_pos_offset = k_off.i32();
  a.rope_scale = rope_scale;
  a.rope_theta = rope_theta;
  a.rope_scaling = rope_scaling;
  a.elem_bits = 32;
  a.q = q.ptr();
  a.q_indptr = qo_indptr != nullptr ? qo_indptr->i32() : nullptr;
  a.pages = pages.ptr();
  a.page_indptr = page_indptr.i32();
  a.page_values = page_indices.i32();
  a.last_page_len = length_info.i32();
  a.out = out.ptr();
  a.lse = lse.f32();
  a.total_q = s.rows;
  a.nnz_pages = s.nnz_pages;
  a.num_pages = s.num_pages;
  a.batch = static_cast<int32_t>(s.batch);
  a.h_q = s.h_q;
  a.h_kv = s.h_kv;
  a.d = s.d;
  a.page_size = s.page_size;
  a.causal = causal > 0;
  a.sm_scale = sm_scale;
  return a;
}

}  // namespace
}  // namespace tvmkv

using namespace tvmkv;

extern "C" {

int tvmkv_dl_fused_rope(const DLTensor* qkv_, const DLTensor* position_map_, const DLTensor* q_, const DLTensor* k_,
                        const DLTensor* v_, int64_t apply_rope, const DLTensor* rope_ext_factors,
                        const tvmkv_rope_scaling* scaling, double rope_scale, double rope_theta, void* stream) {
  KV_API_BEGIN();
  Arg qkv = Take(qkv_, "qkv", kStorage, {3}), pos = Take(position_map_, "q_rope_position_map", kI32, {1});
  Arg q = Take(q_, "q", kStorage, {3}), k = Take(k_, "k", kStorage, {3}), v = Take(v_, "v", kStorage, {3});
  const int device = SameDevice({qkv, pos, q, k, v});
  const int bits = StorageBits({qkv, q, k, v});
  const int64_t rows = qkv.dim(0);
  const int64_t d = qkv.dim(2);
  Expect(q.dim(0) == rows && q.dim(2) == d, q, "(rows of qkv, h_q, head_dim of qkv)");
  Expect(k.dim(0) == rows && k.dim(2) == d, k, "(rows of qkv, h_kv, head_dim of qkv)");
  Expect(v.dim(0) == rows && v.dim(1) == k.dim(1) && v.dim(2) == d, v, "the shape of k");
  Expect(qkv.dim(1) == q.dim(1) + 2 * k.dim(1), qkv, "(rows, h_q + 2 * h_kv, head_dim)");
  Expect(pos.dim(0) >= rows, pos, "(at least the rows of qkv,)");
  const float* factors = nullptr;
  if (rope_ext_factors != nullptr) {
    Arg f = Take(rope_ext_factors, "rope_ext_factors", kF32, {1});
    SameDevice({qkv, f});
    Expect(f.dim(0) == d, f, "(head_dim,): long factors, then short factors");
    factors = f.f32();
    apply_rope = 1;
  }
  Launch(device, [&] { return typed_fused_rope(bits, qkv.ptr(), pos.i32(), q.ptr(), k.ptr(), v.ptr(), apply_rope, factors, scaling,
                                               /*pages=*/nullptr, /*append_position_map=*/nullptr, rows,
                                               static_cast<int32_t>(q.dim(1)), static_cast<int32_t>(k.dim(1)),
                                               static_cast<int32_t>(d), 0, 0, rope_scale, rope_theta, stream); });
  KV_API_END();
}

int tvmkv_dl_transpose_append(const DLTensor* pages_, const DLTensor* k_, const DLTensor* v_, const DLTensor* pos_,
                              void* stream) {
  KV_API_BEGIN();
  Arg pages = Take(pages_, "pages", kStorage, {5}), k = Take(k_, "k_data", kStorage, {3}), v = Take(v_, "v_data", kStorage, {3});
  Arg pos = Take(pos_, "append_position_map", kI32, {1});
  const int device = SameDevice({pages, k, v, pos});
  const int bits = StorageBits({pages, k, v});
  Expect(pages.dim(1) == 2, pages, "(num_pages, 2, h_kv, page_size, head_dim)");
  const int64_t rows = pos.dim(0);
  Expect(k.dim(0) >= rows && k.dim(1) == pages.dim(2) && k.dim(2) == pages.dim(4), k,
         "(at least the length of append_position_map, h_kv of pages, head_dim of pages)");
  Expect(v.dim(0) >= rows && v.dim(1) == pages.dim(2) && v.dim(2) == pages.dim(4), v, "the shape of k_data");
  Launch(device, [&] { return tvmkv_kv_cache_transpose_append(pages.ptr(), k.ptr(), v.ptr(), pos.i32(), rows, pages.dim(0),
                                         static_cast<int32_t>(pages.dim(2)), static_cast<int32_t>(pages.dim(3)),
                                         copy_dim(bits, static_cast<int32_t>(pages.dim(4))), stream); });
  KV_API_END();
}

int tvmkv_dl_transpose_append_mla(const DLTensor* pages_, const DLTensor* kv_, const DLTensor* pos_, void* stream) {
  KV_API_BEGIN();
  Arg pages = Take(pages_, "pages", kF16, {3}), kv = Take(kv_, "kv_data", kF16, {2, 3});
  Arg pos = Take(pos_, "append_position_map", kI32, {1});
  const int device = SameDevice({pages, kv, pos});
  const int64_t rows = pos.dim(0);
  // kv_data is (rows, d_qk), or (rows, 1, d_qk) as some front ends keep the head axis
  const int64_t d_qk = kv.dim(kv.ndim() - 1);
  Expect(kv.dim(0) >= rows && d_qk == pages.dim(2) && (kv.ndim() == 2 || kv.dim(1) == 1), kv,
         "(at least the length of append_position_map, [1,] last extent of pages)");
  Launch(device, [&] { return tvmkv_kv_cache_transpose_append_mla(pages.ptr(), kv.ptr(), pos.i32(), rows, pages.dim(0),
                                             static_cast<int32_t>(pages.dim(1)), static_cast<int32_t>(d_qk), stream); });
  KV_API_END();
}

int tvmkv_dl_batch_prefill_ragged_kv_scaled(const DLTensor* q_, const DLTensor* qo_indptr_, const DLTensor* k_,
                                     const DLTensor* v_, const DLTensor* kv_indptr_, const DLTensor* q_rope_position_,
                                     const DLTensor* k_rope_pos_offset_, const DLTensor* out_, const DLTensor* lse_,
                                     int64_t causal, int64_t rotary_mode, double rope_scale, double rope_theta,
                                     double sm_scale, const tvmkv_rope_scaling* rope_scaling, void* stream) {
  KV_API_BEGIN();
  Arg q = Take(q_, "q", kStorage, {3}), qo_indptr = Take(qo_indptr_, "qo_indptr", kI32, {1});
  Arg k = Take(k_, "k", kStorage, {3}), v = Take(v_, "v", kStorage, {3}), kv_indptr = Take(kv_indptr_, "kv_indptr", kI32, {1});
  Arg q_pos = Take(q_rope_position_, "q_rope_position", kI32, {1});
  Arg k_off = Take(k_rope_pos_offset_, "k_rope_pos_offset", kI32, {1});
  Arg out = Take(out_, "out", kStorage, {3}), lse = Take(lse_, "lse", kF32, {2});
  const int device = SameDevice({q, qo_indptr, k, v, kv_indptr, q_pos, k_off, out, lse});
  const int bits = StorageBits({q, k, v, out});
  const int64_t rows = q.dim(0);
  Expect(qo_indptr.dim(0) >= 1, qo_indptr, "(batch + 1,)");
  const int64_t batch = qo_indptr.dim(0) - 1;
  Expect(kv_indptr.dim(0) == batch + 1, kv_indptr, "(batch + 1,)");
  Expect(k.dim(2) == q.dim(2), k, "(total_kv, h_kv, head_dim of q)");
  Expect(v.dim(0) == k.dim(0) && v.dim(1) == k.dim(1), v, "(total_kv, h_kv, d_v)");
  Expect(k_off.dim(0) == batch, k_off, "(batch,)");
  Expect(q_pos.dim(0) >= rows, q_pos, "(at least the rows of q,)");
  Expect(out.dim(0) == rows && out.dim(1) == q.dim(1) && out.dim(2) == v.dim(2), out, "(rows of q, h_q, d_v)");
  Expect(lse.dim(0) == rows && lse.dim(1) == q.dim(1), lse, "(rows of q, h_q)");
  if (bits == 32) {
    Expect(v.dim(2) == q.dim(2), v, "(total_kv, h_kv, head_dim of q) for float32 storage");
    GenericAttention a;
    a.what = "batch_prefill_ragged_kv";
    a.elem_bits = 32;
    a.q = q.ptr();
    a.q_indptr = qo_indptr.i32();
    a.k = k.ptr();
    a.v = v.ptr();
    a.kv_indptr = kv_indptr.i32();
    a.out = out.ptr();
    a.lse = lse.f32();
    a.total_q = rows;
    a.batch = static_cast<int32_t>(batch);
    a.h_q = static_cast<int32_t>(q.dim(1));
    a.h_kv = static_cast<int32_t>(k.dim(1));
    a.d = static_cast<int32_t>(q.dim(2));
    a.causal = causal > 0;
    a.sm_scale = sm_scale;
    a.rotary_mode = rotary_mode;
    a.q_rope_position = q_pos.i32();
    a.k_rope_pos_offset = k_off.i32();
    a.rope_scale = rope_scale;
    a.rope_theta = rope_theta;
    a.rope_scaling = rope_scaling;
    Launch(device, [&] { return generic_attention(a, stream); });
    return TVMKV_OK;
  }
  Launch(device, [&] { return tvmkv_batch_prefill_ragged_kv_scaled(q.ptr(), qo_indptr.i32(), k.ptr(), v.ptr(), kv_indptr.i32(), q_pos.i32(),
                                       k_off.i32(), out.ptr(), lse.f32(), causal, rotary_mode, rope_scale, rope_theta,
                                       sm_scale, static_cast<int32_t>(batch), rows, static_cast<int32_t>(q.dim(1)),
                                       static_cast<int32_t>(k.dim(1)), static_cast<int32_t>(q.dim(2)),
                                       static_cast<int32_t>(v.dim(2)), rope_scaling, stream); });
  KV_API_END();
}

int tvmkv_dl_batch_prefill_paged_kv_scaled(const DLTensor* q_, const DLTensor* qo_indptr_, const DLTensor* pages_,
                                    const DLTensor* page_indptr_, const DLTensor* page_indices_,
                                    const DLTensor* length_info_, const DLTensor* k_rope_pos_offset_,
                                    const DLTensor* q_rope_position_, const DLTensor* out_, const DLTensor* lse_,
                                    int64_t causal, int64_t rotary_mode, double rope_scale, double rope_theta,
                                    double sm_scale, int64_t layer_sliding_window_size, const tvmkv_rope_scaling* rope_scaling, void* stream) {
  KV_API_BEGIN();
  Arg q = Take(q_, "q", kStorage, {3}), qo_indptr = Take(qo_indptr_, "qo_indptr", kI32, {1});
  Arg pages = Take(pages_, "pages", kStorage, {5}), page_indptr = Take(page_indptr_, "page_indptr", kI32, {1});
  Arg page_indices = Take(page_indices_, "page_indices", kI32, {1});
  Arg length_info = Take(length_info_, "length_info", kI32, {1, 2});
  Arg k_off = Take(k_rope_pos_offset_, "k_rope_pos_offset", kI32, {1});
  Arg q_pos = Take(q_rope_position_, "q_rope_position", kI32, {1});
  Arg out = Take(out_, "out", kStorage, {3}), lse = Take(lse_, "lse", kF32, {2});
  const int device = SameDevice({q, qo_indptr, pages, page_indptr, page_indices, length_info, k_off, q_pos, out, lse});
  const int bits = StorageBits({q, pages, out});
  const PagedShapes s = CheckPaged(q, pages, page_indptr, page_indices, length_info, k_off, q_pos, out, lse);
  Expect(qo_indptr.dim(0) == s.batch + 1, qo_indptr, "(batch + 1,)");
  if (bits == 32) {
    const GenericAttention a = PagedGeneric("batch_prefill_paged_kv", s, q, &qo_indptr, pages, page_indptr, page_indices,
                                            length_info, k_off, q_pos, out, lse, causal, rotary_mode, rope_scale, rope_theta,
                                            rope_scaling, layer_sliding_window_size, sm_scale);
    Launch(device, [&] { return generic_attention(a, stream); });
    return TVMKV_OK;
  }
  Launch(device, [&] { return tvmkv_batch_prefill_paged_kv_scaled(q.ptr(), qo_indptr.i32(), pages.ptr(), page_indptr.i32(), page_indices.i32(),
                                      length_info.i32(), k_off.i32(), q_pos.i32(), out.ptr(), lse.f32(), causal,
                                      rotary_mode, rope_scale, rope_theta, sm_scale, static_cast<int32_t>(s.batch), s.rows,
                                      s.nnz_pages, s.num_pages, s.h_q, s.h_kv, s.d, s.page_size, s.sliding,
                                      static_cast<int32_t>(layer_sliding_window_size), /*merge_into=*/0, rope_scaling, stream); });
  KV_API_END();
}

int tvmkv_dl_batch_decode_paged_kv_scaled(const DLTensor* q_, const DLTensor* pages_, const DLTensor* page_indptr_,
                                   const DLTensor* page_indices_, const DLTensor* length_info_,
                                   const DLTensor* k_rope_pos_offset_, const DLTensor* q_rope_position_,
                                   const DLTensor* out_, const DLTensor* lse_, int64_t rotary_mode, double rope_scale,
                                   double rope_theta, double sm_scale, const tvmkv_rope_scaling* rope_scaling, void* stream) {
  KV_API_BEGIN();
  Arg q = Take(q_, "q", kStorage, {3}), pages = Take(pages_, "pages", kStorage, {5});
  Arg page_indptr = Take(page_indptr_, "page_indptr", kI32, {1});
  Arg page_indices = Take(page_indices_, "page_indices", kI32, {1});
  Arg length_info = Take(length_info_, "length_info", kI32, {1, 2});
  Arg k_off = Take(k_rope_pos_offset_, "k_rope_pos_offset", kI32, {1});
  Arg q_pos = Take(q_rope_position_, "q_rope_position", kI32, {1});
  Arg out = Take(out_, "out", kStorage, {3}), lse = Take(lse_, "lse", kF32, {2});
  const int device = SameDevice({q, pages, page_indptr, page_indices, length_info, k_off, q_pos, out, lse});
  const int bits = StorageBits({q, pages, out});
  const PagedShapes s = CheckPaged(q, pages, page_indptr, page_indices, length_info, k_off, q_pos, out, lse);
  Expect(s.rows == s.batch, q, "(batch, h_q, head_dim): one query per page-table entry");
  if (bits == 32) {
    const GenericAttention a = PagedGeneric("batch_decode_paged_kv", s, q, nullptr, pages, page_indptr, page_indices, length_info,
                                            k_off, q_pos, out, lse, 0, rotary_mode, rope_scale, rope_theta, rope_scaling, 0,
                                            sm_scale);
    Launch(device, [&] { return generic_attention(a, stream); });
    return TVMKV_OK;
  }
  Launch(device, [&] { return tvmkv_batch_decode_paged_kv_scaled(q.ptr(), pages.ptr(), page_indptr.i32(), page_indices.i32(), length_info.i32(),
                                     k_off.i32(), q_pos.i32(), out.ptr(), lse.f32(), rotary_mode, rope_scale, rope_theta,
                                     sm_scale, static_cast<int32_t>(s.batch), s.nnz_pages, s.num_pages, s.h_q, s.h_kv, s.d,
                                     s.page_size, s.sliding, rope_scaling, stream); });
  KV_API_END();
}

int tvmkv_dl_tree_attn_paged_kv(const DLTensor* q_, const DLTensor* qo_indptr_, const DLTensor* pages_,
                                const DLTensor* page_indptr_, const DLTensor* page_indices_,
                                const DLTensor* length_info_, const DLTensor* k_rope_pos_offset_,
                                const DLTensor* q_rope_position_, const DLTensor* out_, const DLTensor* lse_,
                                int64_t rotary_mode, double rope_scale, double rope_theta, double sm_scale,
                                const DLTensor* tree_attn_mn_indptr_, const DLTensor* tree_attn_mask_, void* stream) {
  KV_API_BEGIN();
  Arg q = Take(q_, "q", kStorage, {3}), qo_indptr = Take(qo_indptr_, "qo_indptr", kI32, {1});
  Arg pages = Take(pages_, "pages", kStorage, {5}), page_indptr = Take(page_indptr_, "page_indptr", kI32, {1});
  Arg page_indices = Take(page_indices_, "page_indices", kI32, {1});
  Arg length_info = Take(length_info_, "length_info", kI32, {1, 2});
  Arg k_off = Take(k_rope_pos_offset_, "k_rope_pos_offset", kI32, {1});
  Arg q_pos = Take(q_rope_position_, "q_rope_position", kI32, {1});
  Arg out = Take(out_, "out", kStorage, {3}), lse = Take(lse_, "lse", kF32, {2});
  const int bits = StorageBits({q, pages, out});
  Arg mn_indptr = Take(tree_attn_mn_indptr_, "tree_attn_mn_indptr", kI32, {1});
  Arg mask = Take(tree_attn_mask_, "tree_attn_mask", kI32, {1, 2});
  const int device = SameDevice({q, qo_indptr, pages, page_indptr, page_indices, length_info, k_off, q_pos, out, lse, mn_indptr, mask});
  const PagedShapes s = CheckPaged(q, pages, page_indptr, page_indices, length_info, k_off, q_pos, out, lse);
  Expect(qo_indptr.dim(0) == s.batch + 1, qo_indptr, "(batch + 1,)");
  Expect(mn_indptr.dim(0) == s.batch + 1, mn_indptr, "(batch + 1,)");
  // two labels per tree node, flat (the reference uploads it so) or as (nodes, 2)
  Expect(mask.ndim() == 2 ? mask.dim(1) == 2 : mask.dim(0) % 2 == 0, mask, "(2 * nodes,) or (nodes, 2)");
  NoRotaryTreeOverPages(bits, rotary_mode, "tree_attn_paged_kv");
  if (bits == 32) {
    GenericAttention a = PagedGeneric("tree_attn_paged_kv", s, q, &qo_indptr, pages, page_indptr, page_indices, length_info,
                                      k_off, q_pos, out, lse, 0, 0, 1.0, 1e4, nullptr, 0, sm_scale);
    a.tree_indptr = mn_indptr.i32();
    a.tree_labels = mask.i32();
    Launch(device, [&] { return generic_attention(a, stream); });
    return TVMKV_OK;
  }
  Launch(device, [&] { return tvmkv_tree_attn_paged_kv(q.ptr(), qo_indptr.i32(), pages.ptr(), page_indptr.i32(), page_indices.i32(),
                                  length_info.i32(), k_off.i32(), q_pos.i32(), out.ptr(), lse.f32(), rotary_mode, rope_scale,
                                  rope_theta, sm_scale, mn_indptr.i32(), mask.i32(), static_cast<int32_t>(s.batch), s.rows,
                                  s.nnz_pages, s.num_pages, s.h_q, s.h_kv, s.d, s.page_size, s.sliding, stream); });
  KV_API_END();
}

int tvmkv_dl_batch_tree_attn_scaled(const DLTensor* q_, const DLTensor* qo_indptr_, const DLTensor* k_, const DLTensor* v_,
                             const DLTensor* kv_indptr_, const DLTensor* q_rope_position_,
                             const DLTensor* tree_attn_mn_indptr_, const DLTensor* tree_attn_mask_, const DLTensor* out_,
                             const DLTensor* lse_, int64_t rotary_mode, double rope_scale, double rope_theta,
                             double sm_scale, const tvmkv_rope_scaling* rope_scaling, void* stream) {
  KV_API_BEGIN();
  Arg q = Take(q_, "q", kStorage, {3}), qo_indptr = Take(qo_indptr_, "qo_indptr", kI32, {1});
  Arg k = Take(k_, "k", kStorage, {3}), v = Take(v_, "v", kStorage, {3}), kv_indptr = Take(kv_indptr_, "kv_indptr", kI32, {1});
  Arg q_pos = Take(q_rope_position_, "q_rope_position", kI32, {1});
  Arg mn_indptr = Take(tree_attn_mn_indptr_, "tree_attn_mn_indptr", kI32, {1});
  Arg mask = Take(tree_attn_mask_, "tree_attn_mask", kI32, {1, 2});
  Arg out = Take(out_, "out", kStorage, {3}), lse = Take(lse_, "lse", kF32, {2});
  const int device = SameDevice({q, qo_indptr, k, v, kv_indptr, q_pos, mn_indptr, mask, out, lse});
  const int bits = StorageBits({q, k, v, out});
  const int64_t rows = q.dim(0);
  Expect(qo_indptr.dim(0) >= 1, qo_indptr, "(batch + 1,)");
  const int64_t batch = qo_indptr.dim(0) - 1;
  Expect(kv_indptr.dim(0) == batch + 1, kv_indptr, "(batch + 1,)");
  Expect(mn_indptr.dim(0) == batch + 1, mn_indptr, "(batch + 1,)");
  Expect(mask.ndim() == 2 ? mask.dim(1) == 2 : mask.dim(0) % 2 == 0, mask, "(2 * nodes,) or (nodes, 2)");
  Expect(k.dim(2) == q.dim(2), k, "(total_kv, h_kv, head_dim of q)");
  Expect(v.dim(0) == k.dim(0) && v.dim(1) == k.dim(1) && v.dim(2) == k.dim(2), v, "the shape of k");
  Expect(q_pos.dim(0) >= rows, q_pos, "(at least the rows of q,)");
  Expect(out.dim(0) == rows && out.dim(1) == q.dim(1) && out.dim(2) == q.dim(2), out, "the shape of q");
  Expect(lse.dim(0) == rows && lse.dim(1) == q.dim(1), lse, "(rows of q, h_q)");
  if (bits == 32) {
    GenericAttention a;
    a.what = "batch_tree_attn";
    a.elem_bits = 32;
    a.q = q.ptr();
    a.q_indptr = qo_indptr.i32();
    a.k = k.ptr();
    a.v = v.ptr();
    a.kv_indptr = kv_indptr.i32();
    a.tree_indptr = mn_indptr.i32();
    a.tree_labels = mask.i32();
    a.out = out.ptr();
    a.lse = lse.f32();
    a.total_q = rows;
    a.batch = static_cast<int32_t>(batch);
    a.h_q = static_cast<int32_t>(q.dim(1));
    a.h_kv = static_cast<int32_t>(k.dim(1));
    a.d = static_cast<int32_t>(q.dim(2));
    a.sm_scale = sm_scale;
    a.rotary_mode = rotary_mode;  // key t of sequence b sits at q_rope_position[kv_indptr[b] + t]
    a.q_rope_position = q_pos.i32();
    a.rope_scale = rope_scale;
    a.rope_theta = rope_theta;
    a.rope_scaling = rope_scaling;
    Launch(device, [&] { return generic_attention(a, stream); });
    return TVMKV_OK;
  }
  Launch(device, [&] { return tvmkv_batch_tree_attn_scaled(q.ptr(), qo_indptr.i32(), k.ptr(), v.ptr(), kv_indptr.i32(), q_pos.i32(), mn_indptr.i32(),
                               mask.i32(), out.ptr(), lse.f32(), rotary_mode, rope_scale, rope_theta, sm_scale,
                               static_cast<int32_t>(batch), rows, static_cast<int32_t>(q.dim(1)),
                               static_cast<int32_t>(k.dim(1)), static_cast<int32_t>(q.dim(2)), rope_scaling, stream); });
  KV_API_END();
}

int tvmkv_dl_batch_prefill_paged_kv_mla(const DLTensor* q_, const DLTensor* qo_indptr_, const DLTensor* pages_,
                                        const DLTensor* page_indptr_, const DLTensor* page_indices_,
                                        const DLTensor* length_info_, const DLTensor* out_, const DLTensor* lse_,
                                        int64_t causal, double sm_scale, void* stream) {
  KV_API_BEGIN();
  Arg q = Take(q_, "q", kF16, {3}), qo_indptr = Take(qo_indptr_, "qo_indptr", kI32, {1});
  Arg pages = Take(pages_, "pages", kF16, {3}), page_indptr = Take(page_indptr_, "page_indptr", kI32, {1});
  Arg page_indices = Take(page_indices_, "page_indices", kI32, {1});
  Arg length_info = Take(length_info_, "length_info", kI32, {1});
  Arg out = Take(out_, "out", kF16, {3}), lse = Take(lse_, "lse", kF32, {2});
  const int device = SameDevice({q, qo_indptr, pages, page_indptr, page_indices, length_info, out, lse});
  const int64_t rows = q.dim(0);
  Expect(page_indptr.dim(0) >= 1, page_indptr, "(batch + 1,)");
  const int64_t batch = page_indptr.dim(0) - 1;
  Expect(qo_indptr.dim(0) == batch + 1, qo_indptr, "(batch + 1,)");
  Expect(length_info.dim(0) == batch, length_info, "(batch,)");
  Expect(pages.dim(2) == q.dim(2), pages, "(num_pages, page_size, last extent of q)");
  const int64_t d_latent = out.dim(2);
  Expect(out.dim(0) == rows && out.dim(1) == q.dim(1) && d_latent < q.dim(2), out, "(rows of q, h_q, d_latent)");
  Expect(lse.dim(0) == rows && lse.dim(1) == q.dim(1), lse, "(rows of q, h_q)");
  Launch(device, [&] { return tvmkv_batch_prefill_paged_kv_mla(q.ptr(), qo_indptr.i32(), pages.ptr(), page_indptr.i32(), page_indices.i32(),
                                          length_info.i32(), out.ptr(), lse.f32(), causal, sm_scale,
                                          static_cast<int32_t>(batch), rows, page_indices.dim(0), pages.dim(0),
                                          static_cast<int32_t>(q.dim(1)), static_cast<int32_t>(d_latent),
                                          static_cast<int32_t>(q.dim(2) - d_latent), static_cast<int32_t>(pages.dim(1)),
                                          stream); });
  KV_API_END();
}

int tvmkv_dl_merge_state_inplace(const DLTensor* v_, const DLTensor* s_, const DLTensor* v_other_,
                                 const DLTensor* s_other_, void* stream) {
  KV_API_BEGIN();
  Arg v = Take(v_, "v", kStorage, {3}), s = Take(s_, "s", kF32, {2});
  Arg v_other = Take(v_other_, "v_other", kStorage, {3}), s_other = Take(s_other_, "s_other", kF32, {2});
  const int device = SameDevice({v, s, v_other, s_other});
  const int bits = StorageBits({v, v_other});
  Expect(s.dim(0) == v.dim(0) && s.dim(1) == v.dim(1), s, "(rows of v, heads of v)");
  Expect(v_other.dim(0) >= v.dim(0) && v_other.dim(1) == v.dim(1) && v_other.dim(2) == v.dim(2), v_other, "the shape of v");
  Expect(s_other.dim(0) >= v.dim(0) && s_other.dim(1) == v.dim(1), s_other, "the shape of s");
  Launch(device, [&] { return typed_merge_state_inplace(bits, v.ptr(), s.f32(), v_other.ptr(), s_other.f32(), v.dim(0),
                                                        static_cast<int32_t>(v.dim(1)), static_cast<int32_t>(v.dim(2)), stream); });
  KV_API_END();
}

int tvmkv_dl_copy_single_page(const DLTensor* pages_, int64_t src_page_id, int64_t tgt_page_id, int64_t copy_length,
                              void* stream) {
  KV_API_BEGIN();
  Arg pages = Take(pages_, "pages", kStorage, {5, 3});
  const int device = SameDevice({pages});
  const int bits = StorageBits({pages});
  if (pages.ndim() == 5) {
    Expect(pages.dim(1) == 2, pages, "(num_pages, 2, h_kv, page_size, head_dim)");
    Launch(device, [&] { return tvmkv_copy_single_page(pages.ptr(), src_page_id, tgt_page_id, copy_length, pages.dim(0),
                                  static_cast<int32_t>(pages.dim(2)), static_cast<int32_t>(pages.dim(3)),
                                  copy_dim(bits, static_cast<int32_t>(pages.dim(4))), stream); });
  } else {
    KV_UNSUPPORTED(bits != 16) << "copy_single_page: the MLA cache is built for float16 storage only";
    Launch(device, [&] { return tvmkv_copy_single_page_mla(pages.ptr(), src_page_id, tgt_page_id, copy_length, pages.dim(0),
                                      static_cast<int32_t>(pages.dim(1)), static_cast<int32_t>(pages.dim(2)), stream); });
  }
  KV_API_END();
}

int tvmkv_dl_debug_get_kv(const DLTensor* pages_, const DLTensor* position_map_, const DLTensor* k_data_,
                          const DLTensor* v_data_, int64_t layer_id, void* stream) {
  KV_API_BEGIN();
  Arg pages = Take(pages_, "pages", kStorage, {5}), pos = Take(position_map_, "position_map", kI32, {1});
  Arg k = Take(k_data_, "k_data", kStorage, {4}), v = Take(v_data_, "v_data", kStorage, {4});
  const int device = SameDevice({pages, pos, k, v});
  const int bits = StorageBits({pages, k, v});
  Expect(pages.dim(1) == 2, pages, "(num_pages, 2, h_kv, page_size, head_dim)");
  Expect(k.dim(1) == pos.dim(0) && k.dim(2) == pages.dim(2) && k.dim(3) == pages.dim(4), k,
         "(num_layers, length of position_map, h_kv, head_dim)");
  Expect(v.dim(0) == k.dim(0) && v.dim(1) == k.dim(1) && v.dim(2) == k.dim(2) && v.dim(3) == k.dim(3), v,
         "the shape of k_data");
  KV_CHECK(layer_id >= 0 && layer_id < k.dim(0)) << "layer_id " << layer_id << " is outside k_data's " << k.dim(0) << " layers";
  Launch(device, [&] { return tvmkv_kv_cache_debug_get_kv(pages.ptr(), pos.i32(), k.ptr(), v.ptr(), layer_id, pos.dim(0), pages.dim(0),
                                     static_cast<int32_t>(pages.dim(2)), static_cast<int32_t>(pages.dim(3)),
                                     copy_dim(bits, static_cast<int32_t>(pages.dim(4))), stream); });
  KV_API_END();
}

int tvmkv_dl_debug_get_kv_mla(const DLTensor* pages_, const DLTensor* position_map_, const DLTensor* kv_data_,
                              int64_t layer_id, void* stream) {
  KV_API_BEGIN();
  Arg pages = Take(pages_, "pages", kF16, {3}), pos = Take(position_map_, "position_map", kI32, {1});
  Arg kv = Take(kv_data_, "kv_data", kF16, {3});
  const int device = SameDevice({pages, pos, kv});
  Expect(kv.dim(1) == pos.dim(0) && kv.dim(2) == pages.dim(2), kv, "(num_layers, length of position_map, last extent of pages)");
  KV_CHECK(layer_id >= 0 && layer_id < kv.dim(0)) << "layer_id " << layer_id << " is outside kv_data's " << kv.dim(0) << " layers";
  Launch(device, [&] { return tvmkv_kv_cache_debug_get_kv_mla(pages.ptr(), pos.i32(), kv.ptr(), layer_id, pos.dim(0), pages.dim(0),
                                         static_cast<int32_t>(pages.dim(1)), static_cast<int32_t>(pages.dim(2)), stream); });
  KV_API_END();
}

int tvmkv_dl_compact_kv_copy(const DLTensor* pages_, const DLTensor* copy_length_indptr_,
                             const DLTensor* copy_src_dst_pos_, int64_t batch_size, void* stream) {
  KV_API_BEGIN();
  Arg pages = Take(pages_, "pages", kStorage, {5}), indptr = Take(copy_length_indptr_, "copy_length_indptr", kI32, {1});
  Arg pos = Take(copy_src_dst_pos_, "copy_src_dst_pos", kI32, {2});
  const int device = SameDevice({pages, indptr, pos});
  Expect(pages.dim(1) == 2, pages, "(num_pages, 2, h_kv, page_size, head_dim)");
  KV_CHECK(batch_size >= 0 && indptr.dim(0) >= batch_size + 1)
      << "copy_length_indptr has " << indptr.dim(0) << " entries, fewer than batch_size + 1 = " << batch_size + 1;
  Expect(pos.dim(0) == 2, pos, "(2, total_copy_length)");
  Launch(device, [&] { return tvmkv_compact_kv_copy(pages.ptr(), indptr.i32(), pos.i32(), static_cast<int32_t>(batch_size),
                               static_cast<int32_t>(pos.dim(1)), pages.dim(0), static_cast<int32_t>(pages.dim(2)),
                               static_cast<int32_t>(pages.dim(3)),
                               copy_dim(pages.t->dtype.bits, static_cast<int32_t>(pages.dim(4))), stream); });
  KV_API_END();
}

// The entry points without a frequency variant: the default frequencies theta^(-2i/d).
int tvmkv_dl_batch_prefill_ragged_kv(const DLTensor* q, const DLTensor* qo_indptr, const DLTensor* k, const DLTensor* v,
                                     const DLTensor* kv_indptr, const DLTensor* q_rope_position,
                                     const DLTensor* k_rope_pos_offset, const DLTensor* out, const DLTensor* lse,
                                     int64_t causal, int64_t rotary_mode, double rope_scale, double rope_theta,
                                     double sm_scale, void* stream) {
  return tvmkv_dl_batch_prefill_ragged_kv_scaled(q, qo_indptr, k, v, kv_indptr, q_rope_position, k_rope_pos_offset, out, lse,
                                                 causal, rotary_mode, rope_scale, rope_theta, sm_scale, nullptr, stream);
}

int tvmkv_dl_batch_prefill_paged_kv(const DLTensor* q, const DLTensor* qo_indptr, const DLTensor* pages,
                                    const DLTensor* page_indptr, const DLTensor* page_indices, const DLTensor* length_info,
                                    const DLTensor* k_rope_pos_offset, const DLTensor* q_rope_position, const DLTensor* out,
                                    const DLTensor* lse, int64_t causal, int64_t rotary_mode, double rope_scale,
                                    double rope_theta, double sm_scale, int64_t layer_sliding_window_size, void* stream) {
  return tvmkv_dl_batch_prefill_paged_kv_scaled(q, qo_indptr, pages, page_indptr, page_indices, length_info, k_rope_pos_offset,
                                                q_rope_position, out, lse, causal, rotary_mode, rope_scale, rope_theta,
                                                sm_scale, layer_sliding_window_size, nullptr, stream);
}

int tvmkv_dl_batch_decode_paged_kv(const DLTensor* q, const DLTensor* pages, const DLTensor* page_indptr,
                                   const DLTensor* page_indices, const DLTensor* length_info,
                                   const DLTensor* k_rope_pos_offset, const DLTensor* q_rope_position, const DLTensor* out,
                                   const DLTensor* lse, int64_t rotary_mode, double rope_scale, double rope_theta,
                                   double sm_scale, void* stream) {
  return tvmkv_dl_batch_decode_paged_kv_scaled(q, pages, page_indptr, page_indices, length_info, k_rope_pos_offset,
                                               q_rope_position, out, lse, rotary_mode, rope_scale, rope_theta, sm_scale,
                                               nullptr, stream);
}

int tvmkv_dl_batch_tree_attn(const DLTensor* q, const DLTensor* qo_indptr, const DLTensor* k, const DLTensor* v,
                             const DLTensor* kv_indptr, const DLTensor* q_rope_position,
                             const DLTensor* tree_attn_mn_indptr, const DLTensor* tree_attn_mask, const DLTensor* out,
                             const DLTensor* lse, int64_t rotary_mode, double rope_scale, double rope_theta,
                             double sm_scale, void* stream) {
  return tvmkv_dl_batch_tree_attn_scaled(q, qo_indptr, k, v, kv_indptr, q_rope_position, tree_attn_mn_indptr, tree_attn_mask,
                                         out, lse, rotary_mode, rope_scale, rope_theta, sm_scale, nullptr, stream);
}

}  // extern "C"
