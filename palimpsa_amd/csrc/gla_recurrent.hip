// Token-serial forward of scalar-gated linear attention (any T >= 1; T == 1 is single-step decode):
//     S_t = f_t S_{t-1} + k_t v_t^T ,   o_t = scale * S_t^T q_t ,   f_t = exp(-gt_t * g) ,
// the Palimpsa recurrence without its precision state, with the state kept as S [N, H, dk, dv] — the
// layout the layer's cache holds on this path (fla's simple_gla, called at
// palimpsa/layers/palimpsa.py:293-300), so that a decode step reads and writes the state exactly once
// and nothing has to be transposed.
//
// Mapping: one workgroup of 4 waves per (sequence, head, block of 64 value columns).  Lane = value
// column, so every state access of a wave is 256 contiguous bytes; wave w keeps the key rows
// [w dk/4, (w+1) dk/4) of its columns in registers for the whole sequence.  k_t and q_t are uniform
// over a wave; the four partial outputs of a token meet in LDS (double buffered: one barrier per token).
// Bound: HBM (4 dk dv bytes in and out per sequence, head and step).
#include "pal_common.h"
#include "pal_host.h"
#include "pal_profile.h"

namespace pal {

struct GlaRecArgs {
  const void *q, *k, *v, *gt;
  const float* g;
  void* o;
  const float* init;
  float* final_;
  const int32_t* cu_seqlens;
  int32_t T, H, dk, dv, n_seqs, gate_bf16;
  int32_t Hq;   // heads of q and k (H, or a divisor of it: a group of H / Hq value heads shares one)
  float scale;
};

template <typename TIn, int NQ>   // NQ = dk / 4 key rows per wave
__global__ __launch_bounds__(256) void gla_recurrent_fwd_kernel(GlaRecArgs a) {
  __shared__ float sO[2][4][64];
  const int tid = threadIdx.x, lane = tid & 63;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int dk = a.dk, dv = a.dv, H = a.H;
  const int n_dblk = (dv + 63) >> 6;
  const int dblk = blockIdx.x % n_dblk;
  const int nh = blockIdx.x / n_dblk;
  const int h = nh % H, n = nh / H;
  const int d = dblk * 64 + lane;
  const bool on = d < dv;
  int64_t bos;
  int T;
  if (a.cu_seqlens) {
    int b0;
    packed_seq_bounds(a.cu_seqlens, n, a.T, b0, T);
    bos = b0;
  } else {
    bos = (int64_t)n * a.T;
    T = a.T;
  }
  const float gh = a.g[h] * kLog2e;
  const float scale = a.scale;
  const int n0 = w * NQ;
  const int64_t sbase = ((int64_t)nh * dk + n0) * dv + d;

  float S[NQ];
#pragma unroll
  for (int e = 0; e < NQ; ++e) S[e] = 0.f;
  if (a.init && on) {
#pragma unroll
    for (int e = 0; e < NQ; ++e) S[e] = __builtin_nontemporal_load(a.init + sbase + (int64_t)e * dv);
  }
  const int Hq = a.Hq, hq = h / (H / Hq);
  const TIn* qp = (const TIn*)a.q + (bos * Hq + hq) * dk + n0;
  const TIn* kp = (const TIn*)a.k + (bos * Hq + hq) * dk + n0;
  const TIn* vp = (const TIn*)a.v + (bos * H + h) * dv + d;
  TIn* op = (TIn*)a.o + (bos * H + h) * dv + d;
  for (int t = 0; t < T; ++t) {
    const int64_t off_k = (int64_t)t * Hq * dk, off_v = (int64_t)t * H * dv;
    const float f = fast_exp2(-load_gate(a.gt, (bos + t) * H + h, a.gate_bf16) * gh);
    const float v = on ? to_f32(vp[off_v]) : 0.f;
    float acc = 0.f;
#pragma unroll
    for (int e = 0; e < NQ; ++e) {
      const float kk = to_f32(kp[off_k + e]), qq = to_f32(qp[off_k + e]);
      S[e] = fmaf(f, S[e], kk * v);
      acc = fmaf(S[e], qq, acc);
    }
    sO[t & 1][w][lane] = acc;
    __syncthreads();
    if (w == 0 && on) {
      const float tot = (sO[t & 1][0][lane] + sO[t & 1][1][lane]) + (sO[t & 1][2][lane] + sO[t & 1][3][lane]);
      op[off_v] = from_f32<TIn>(tot * scale);
    }
  }
  if (a.final_ && on) {
#pragma unroll
    for (int e = 0; e < NQ; ++e) __builtin_nontemporal_store(S[e], a.final_ + sbase + (int64_t)e * dv);
  }
}

template <typename TIn, int NQ>
static int launch_gla_rec_nq(const GlaRecArgs& a, hipStream_t s) {
  const int64_t blocks = (int64_t)a.n_seqs * a.H * ((a.dv + 63) / 64);
  if (blocks > 0x7fffffff) return PAL_E_DIM;
  PAL_TIMED_LAUNCH(kKernGlaRecurrentFwd, s, (gla_recurrent_fwd_kernel<TIn, NQ>), dim3((unsigned)blocks), dim3(256), 0, s, a);
  PAL_HIP_LAUNCH_CHECK();
  return PAL_OK;
}

template <typename TIn>
static int launch_gla_rec(const GlaRecArgs& a, hipStream_t s) {
  switch (a.dk / 16) {
    case 1: return launch_gla_rec_nq<TIn, 4>(a, s);
    case 2: return launch_gla_rec_nq<TIn, 8>(a, s);
    case 3: return launch_gla_rec_nq<TIn, 12>(a, s);
    case 4: return launch_gla_rec_nq<TIn, 16>(a, s);
    case 5: return launch_gla_rec_nq<TIn, 20>(a, s);
    case 6: return launch_gla_rec_nq<TIn, 24>(a, s);
    case 7: return launch_gla_rec_nq<TIn, 28>(a, s);
    case 8: return launch_gla_rec_nq<TIn, 32>(a, s);
    case 9: return launch_gla_rec_nq<TIn, 36>(a, s);
    case 10: return launch_gla_rec_nq<TIn, 40>(a, s);
    case 11: return launch_gla_rec_nq<TIn, 44>(a, s);
    case 12: return launch_gla_rec_nq<TIn, 48>(a, s);
    case 13: return launch_gla_rec_nq<TIn, 52>(a, s);
    case 14: return launch_gla_rec_nq<TIn, 56>(a, s);
    case 15: return launch_gla_rec_nq<TIn, 60>(a, s);
    case 16: return launch_gla_rec_nq<TIn, 64>(a, s);
    default: return PAL_E_HEADDIM;
  }
}

}  // namespace pal

extern "C" int pal_gla_recurrent_fwd(const PalDims* d, const PalFwdTensors* t, void* stream) {
  using namespace pal;
  if (int rc = pal_validate_dims(d)) return rc;
  if (!t) return PAL_E_NULL;
  if (!t->q || !t->k || !t->v || !t->gt || !t->g || !t->o) return PAL_E_NULL;
  if (d->flags & PAL_FLAG_HAS_VAR) return PAL_E_STATE;
  if (d->flags & PAL_FLAG_STATE_MU_BF16) return PAL_E_STATE;
  if (((d->flags & PAL_FLAG_HAS_INIT) != 0) != (t->init_mu != nullptr)) return PAL_E_STATE;
  if (((d->flags & PAL_FLAG_STORE_FINAL) != 0) != (t->final_mu != nullptr)) return PAL_E_STATE;
  const bool varlen = d->flags & PAL_FLAG_VARLEN;
  if (varlen != (t->cu_seqlens != nullptr)) return PAL_E_CU_SEQLENS;
  const void* ptrs[] = {t->q, t->k, t->v, t->o, t->init_mu, t->final_mu};
  for (const void* p : ptrs)
    if (p && !is_aligned16(p)) return PAL_E_ALIGN;
  if (!is_aligned4(t->gt)) return PAL_E_ALIGN;   // one alignment rule for the gate tensor at every entry point
  GlaRecArgs a;
  a.q = t->q; a.k = t->k; a.v = t->v; a.gt = t->gt; a.g = t->g; a.o = t->o;
  a.init = t->init_mu; a.final_ = t->final_mu; a.cu_seqlens = t->cu_seqlens;
  a.T = d->seq_len; a.H = d->n_heads; a.dk = d->dk; a.dv = d->dv; a.n_seqs = d->n_seqs;
  a.Hq = d->n_qk_heads > 0 ? d->n_qk_heads : d->n_heads;
  a.gate_bf16 = d->gate_dtype == PAL_DTYPE_BF16;
  a.scale = d->scale;
  hipStream_t s = (hipStream_t)stream;
  if (d->dtype == PAL_DTYPE_BF16) return launch_gla_rec<bf16_t>(a, s);
  return launch_gla_rec<float>(a, s);
}
