// MLA (multi-head latent attention) paged kernel -- placeholder translation unit until the
// MFMA kernel lands; the launcher reports TVMKV_EUNSUPPORTED.
#include "kernels_common.cuh"

extern "C" int tvmkv_batch_prefill_paged_kv_mla(const void* q, const int32_t* q_indptr, const void* pages,
                                                const int32_t* page_indptr, const int32_t* page_values,
                                                const int32_t* length_info, void* output, float* lse,
                                                int64_t causal, double sm_scale, int32_t batch_size,
                                                int64_t total_q, int64_t nnz_pages, int64_t num_pages, int32_t h_q,
                                                int32_t d_latent, int32_t d_rope, int32_t page_size, void* stream) {
  KV_API_BEGIN();
  KV_UNSUPPORTED(true) << "batch_prefill_paged_kv_mla: not built yet";
  KV_API_END();
}
