// Host-only part of the C ABI: argument validation, error strings and the
// varlen chunk bookkeeping.  No device code and nothing here touches a GPU.
#include "pal_common.h"
#include "pal_host.h"

extern "C" {

int pal_abi_version(void) { return PAL_ABI_VERSION; }

const char* pal_strerror(int code) {
  switch (code) {
    case PAL_OK: return "ok";
    case PAL_E_NULL: return "a required pointer is NULL";
    case PAL_E_DIM: return "a dimension is non-positive or out of range";
    case PAL_E_HEADDIM:
      return "dk and dv must be multiples of 16 in [16, 256] (dk one of 16,32,48,64,96,128,192,256 for the recurrent "
             "Palimpsa path; the chunked Palimpsa backward also keeps a dk x dv carry tile in LDS: "
             "4 dk (dv + 8) + 256 (max(dk, dv) + 4) + 32 dv + 288 <= 163840 bytes, e.g. up to 128x192, 192x128, 256x64; "
             "fp32 rows without PAL_FLAG_FP32_FAST: 8 dk (dv + 8) in that sum and head dims up to 128, "
             "e.g. 96x96, 64x128, 128x64)";
    case PAL_E_DTYPE: return "unsupported element type";
    case PAL_E_VARLEN_BATCH: return "cu_seqlens needs batch size 1";
    case PAL_E_CU_SEQLENS: return "cu_seqlens must start at 0, be non-decreasing and end at the token count";
    case PAL_E_WORKSPACE: return "workspace missing or too small";
    case PAL_E_CHUNK: return "total_chunks does not match the sequence lengths";
    case PAL_E_STATE: return "state flags and state pointers disagree";
    case PAL_E_CAPACITY: return "output table too small";
    case PAL_E_ALIGN: return "pointer not aligned (row tensors and states: 16 bytes; gate tensor: 4 bytes)";
    case PAL_E_SCRATCH:
      return "the call needs more tile-start states than the library's static scratch holds "
             "(total_chunks * n_heads * dv * dk * 8 bytes > PAL_STATIC_SCRATCH_BYTES); split the sequence";
    default: break;
  }
  if (code > 0) return hipGetErrorString((hipError_t)code);
  return "unknown palimpsa_hip error";
}

int pal_validate_dims(const PalDims* d) {
  if (!d) return PAL_E_NULL;
  if (d->batch <= 0 || d->seq_len <= 0 || d->n_seqs <= 0 || d->n_heads <= 0) return PAL_E_DIM;
  if (d->n_heads > 65535) return PAL_E_DIM;
  if ((int64_t)d->batch * d->seq_len > (int64_t)1 << 30) return PAL_E_DIM;
  if (d->dk < 16 || d->dk > 256 || (d->dk & 15) || d->dv < 16 || d->dv > 256 || (d->dv & 15))
    return PAL_E_HEADDIM;
  if (d->dtype != PAL_DTYPE_F32 && d->dtype != PAL_DTYPE_BF16) return PAL_E_DTYPE;
  if (d->gate_dtype != PAL_DTYPE_F32 && d->gate_dtype != PAL_DTYPE_BF16) return PAL_E_DTYPE;
  if (d->var_dtype != PAL_DTYPE_F32 && d->var_dtype != PAL_DTYPE_BF16) return PAL_E_DTYPE;
  if (d->flags & PAL_FLAG_VARLEN) {
    if (d->batch != 1) return PAL_E_VARLEN_BATCH;
    if (d->n_seqs > d->seq_len) return PAL_E_CU_SEQLENS;
  } else {
    if (d->n_seqs != d->batch) return PAL_E_DIM;
  }
  if (!(d->scale == d->scale)) return PAL_E_DIM;  // NaN
  if (d->n_qk_heads < 0 || (d->n_qk_heads > 0 && d->n_heads % d->n_qk_heads != 0)) return PAL_E_DIM;
  return PAL_OK;
}

int pal_build_chunk_table(const int64_t* cu, int32_t n_seqs, int32_t* table_out, int32_t capacity,
                          int32_t* offsets_out) {
  if (!cu) return PAL_E_NULL;
  if (n_seqs <= 0) return PAL_E_DIM;
  if (cu[0] != 0) return PAL_E_CU_SEQLENS;
  int64_t total = 0;
  if (offsets_out) offsets_out[0] = 0;
  for (int32_t n = 0; n < n_seqs; ++n) {
    int64_t s = cu[n], e = cu[n + 1];
    if (e < s || e > ((int64_t)1 << 30)) return PAL_E_CU_SEQLENS;
    int32_t idx = 0;
    for (int64_t c0 = s; c0 < e; c0 += PAL_CHUNK, ++idx) {
      if (table_out) {
        if (total >= capacity) return PAL_E_CAPACITY;
        int64_t len = e - c0 < PAL_CHUNK ? e - c0 : PAL_CHUNK;
        table_out[4 * total + 0] = n;
        table_out[4 * total + 1] = (int32_t)c0;
        table_out[4 * total + 2] = (int32_t)len;
        table_out[4 * total + 3] = idx;
      }
      ++total;
    }
    if (total > 0x7fffffff) return PAL_E_DIM;
    if (offsets_out) offsets_out[n + 1] = (int32_t)total;
  }
  return (int)total;
}

}  // extern "C"

namespace pal {

int check_fwd_common(const PalDims* d, const PalFwdTensors* t) {
  int rc = pal_validate_dims(d);
  if (rc) return rc;
  if (d->flags & PAL_FLAG_STATE_MU_BF16) return PAL_E_STATE;   // pal_recurrent_fwd clears it before it comes here
  if (!t) return PAL_E_NULL;
  if (!t->q || !t->k || !t->v || !t->b || !t->gt || !t->g || !t->Ip || !t->o) return PAL_E_NULL;
  const bool has_init = d->flags & PAL_FLAG_HAS_INIT;
  if (has_init != (t->init_mu != nullptr) || has_init != (t->init_I != nullptr)) return PAL_E_STATE;
  const bool store = d->flags & PAL_FLAG_STORE_FINAL;
  if (store != (t->final_mu != nullptr) || store != (t->final_I != nullptr)) return PAL_E_STATE;
  const bool var = d->flags & PAL_FLAG_HAS_VAR;
  if (var && !t->o_var) return PAL_E_NULL;
  const bool varlen = d->flags & PAL_FLAG_VARLEN;
  if (varlen != (t->cu_seqlens != nullptr)) return PAL_E_CU_SEQLENS;
  const void* ptrs[] = {t->q, t->k, t->v, t->b, t->o, t->o_var, t->init_mu, t->init_I,
                        t->final_mu, t->final_I, t->chunk_mu, t->chunk_I};
  for (const void* p : ptrs)
    if (p && !is_aligned16(p)) return PAL_E_ALIGN;
  if (!is_aligned4(t->gt)) return PAL_E_ALIGN;   // gates are fetched as the aligned 32-bit word that holds them
  return PAL_OK;
}

int check_chunk_common(const PalDims* d, const PalFwdTensors* t) {
  int rc = check_fwd_common(d, t);
  if (rc) return rc;
  if (!t->chunk_mu || !t->chunk_I) return PAL_E_NULL;
  if (d->total_chunks <= 0) return PAL_E_CHUNK;
  if (d->flags & PAL_FLAG_VARLEN) {
    if (!t->chunk_table || !t->chunk_offsets) return PAL_E_NULL;
    // every document has at least one token per chunk and at most PAL_CHUNK
    int64_t lo = ((int64_t)d->seq_len + PAL_CHUNK - 1) / PAL_CHUNK;
    int64_t hi = (int64_t)d->seq_len / PAL_CHUNK + d->n_seqs;
    if (d->total_chunks < lo || d->total_chunks > hi) return PAL_E_CHUNK;
  } else {
    int64_t per = ((int64_t)d->seq_len + PAL_CHUNK - 1) / PAL_CHUNK;
    if ((int64_t)d->total_chunks != per * d->batch) return PAL_E_CHUNK;
  }
  return PAL_OK;
}

int check_bwd_common(const PalDims* d, const PalBwdTensors* gr) {
  if (!gr) return PAL_E_NULL;
  if (!gr->d_o || !gr->dq || !gr->dk || !gr->dv || !gr->db || !gr->dgt || !gr->dg || !gr->dIp)
    return PAL_E_NULL;
  if ((d->flags & PAL_FLAG_HAS_VAR) && !gr->d_o_var) return PAL_E_NULL;
  if ((gr->d_init_mu != nullptr) != (gr->d_init_I != nullptr)) return PAL_E_STATE;
  if (gr->d_init_mu && !(d->flags & PAL_FLAG_HAS_INIT)) return PAL_E_STATE;
  const void* ptrs[] = {gr->d_o, gr->d_o_var, gr->dq, gr->dk, gr->dv, gr->db, gr->d_init_mu, gr->d_init_I};
  for (const void* p : ptrs)
    if (p && !is_aligned16(p)) return PAL_E_ALIGN;
  return PAL_OK;
}

}  // namespace pal
