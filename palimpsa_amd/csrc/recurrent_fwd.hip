// Token-serial Palimpsa forward (any T >= 1; T == 1 is single-step decode).
//
// Replaces fused_palimpsa_recurrent_fwd_kernel of the reference
// (palimpsa/ops/palimpsa/fused_recurrent_palimpsa.py:24-154).  Same arithmetic:
//   f = exp(-gt*g); M = f*M + v k^T; Jbar = f*Jbar + b (k*k)^T; I = Jbar + Ip;
//   o = scale * (M/I) q ; o_var = scale * (1/I) (q*q)
// with the (mu, I) external state form of :88-96 and :145-154.
//
// Mapping (wave64): one wave per (sequence, head, tile of 4*RD value rows).
// A row of the dv x dk state is spread over the 16 lanes of a DPP row, NPL =
// dk/16 entries per lane, so a wave covers 4 value rows at a time; each lane
// keeps RD*NPL entries of M and of Jbar in registers for the whole sequence.
// The sum over dk is a 4-step DPP rotation inside the row.  Memory access is
// the only cost that matters at T == 1: every lane issues all its state loads
// up front as 16-byte vectors that are contiguous across the row.
#include "pal_common.h"
#include "pal_host.h"
#include "pal_profile.h"

namespace pal {

struct RecArgs {
  const void *q, *k, *v, *b, *gt;
  const float *g, *Ip;
  void *o, *o_var;
  const float *init_mu, *init_I;
  float *final_mu, *final_I;
  const int32_t* cu_seqlens;
  int32_t T, H, dk, dv, n_seqs;
  int32_t Hq;   // heads of q and k (H, or a divisor of it: a group of H / Hq value heads shares one)
  int32_t gate_bf16, var_bf16;
  uint32_t flags;
  float scale;
};

// n index of element e of lane j (j = lane % 16); VW-wide vectors interleaved across the row.
// WIDE (the bf16 cache format of mu): 8-wide vectors where a lane has 8 entries, so that the bf16 state moves in
// 16-byte pieces like the fp32 one (with 8-byte pieces the kernel ran at 0.69 of the HBM rate instead of 0.79).
template <int NPL, bool WIDE = false>
struct NMap {
  static constexpr int VW = (WIDE && NPL % 8 == 0) ? 8 : (NPL % 4 == 0) ? 4 : ((NPL % 2 == 0) ? 2 : 1);
  static constexpr int NV = NPL / VW;
  __device__ static __forceinline__ int vec_start(int j, int iv) { return 16 * VW * iv + VW * j; }
};

// VW elements (1, 2, 4 or 8) as fp32; the 8-wide forms are one 16-byte access for bf16 and two for fp32
template <int VW, typename T>
__device__ __forceinline__ void load_n(const T* p, float* out) {
  if constexpr (VW == 8) {
    if constexpr (std::is_same_v<T, bf16_t>) {
      const bf16x8 x = *(const bf16x8*)p;
#pragma unroll
      for (int e = 0; e < 8; ++e) out[e] = (float)x[e];
    } else {
      load_vec<4>(p, out);
      load_vec<4>(p + 4, out + 4);
    }
  } else {
    load_vec<VW>(p, out);
  }
}
template <int VW, typename T>
__device__ __forceinline__ void load_n_stream(const T* p, float* out) {
  if constexpr (VW == 8) {
    if constexpr (std::is_same_v<T, bf16_t>) {
      const bf16x8 x = __builtin_bit_cast(bf16x8, __builtin_nontemporal_load((const f32x4*)p));
#pragma unroll
      for (int e = 0; e < 8; ++e) out[e] = (float)x[e];
    } else {
      load_vec_stream<4>(p, out);
      load_vec_stream<4>(p + 4, out + 4);
    }
  } else {
    load_vec_stream<VW>(p, out);
  }
}
template <int VW, typename T>
__device__ __forceinline__ void store_n_stream(T* p, const float* in) {
  if constexpr (VW == 8) {
    if constexpr (std::is_same_v<T, bf16_t>) {
      bf16x8 x;
#pragma unroll
      for (int e = 0; e < 8; ++e) x[e] = (bf16_t)in[e];
      __builtin_nontemporal_store(__builtin_bit_cast(f32x4, x), (f32x4*)p);
    } else {
      store_vec_stream<4>(p, in);
      store_vec_stream<4>(p + 4, in + 4);
    }
  } else {
    store_vec_stream<VW>(p, in);
  }
}

// PF = tokens whose rows are in flight.  PF = 1 (decode): the next token's rows are requested while the current one
// is processed.  A long token-serial run is bound by the latency of those requests (0.3-0.6 us per token against
// 0.1-0.2 us of arithmetic), so it keeps PF tokens in registers: a token is processed from its set and the set is
// reloaded at once with the token PF ahead (always issued, clamped to the last token, so that the number of
// requests in flight is the same in every iteration and the compiler can wait for exactly the oldest set).
template <typename TIn, int NPL, int RD, bool MU16, int PF, bool HAS_VAR>
__global__ __launch_bounds__(64) void recurrent_fwd_kernel(RecArgs a) {
  using Map = NMap<NPL, MU16>;
  constexpr int VW = Map::VW;
  constexpr int NV = Map::NV;
  const int lane = threadIdx.x;
  const int j = lane & 15;
  const int grp = lane >> 4;
  const int n_dtiles = a.dv / (4 * RD);
  const int tile = blockIdx.x % n_dtiles;
  const int nh = blockIdx.x / n_dtiles;
  const int h = nh % a.H;
  const int n = nh / a.H;
  const int dk = a.dk, dv = a.dv, H = a.H;

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
  const float Ip = a.Ip[h];
  const float scale = a.scale;
  constexpr bool mu16 = MU16;   // mu kept in bf16 between calls (a cache format of decode)

  int drow[RD];
#pragma unroll
  for (int rr = 0; rr < RD; ++rr) drow[rr] = tile * (4 * RD) + rr * 4 + grp;

  float M[RD][NPL], J[RD][NPL];
  if (a.init_mu) {
#pragma unroll
    for (int rr = 0; rr < RD; ++rr) {
      const int64_t base = ((int64_t)nh * dv + drow[rr]) * dk;
#pragma unroll
      for (int iv = 0; iv < NV; ++iv) {
        float mu[VW], I[VW];
        if constexpr (mu16) load_n_stream<VW>((const bf16_t*)a.init_mu + base + Map::vec_start(j, iv), mu);
        else load_n_stream<VW>(a.init_mu + base + Map::vec_start(j, iv), mu);
        load_n_stream<VW>(a.init_I + base + Map::vec_start(j, iv), I);
#pragma unroll
        for (int e = 0; e < VW; ++e) {
          M[rr][iv * VW + e] = mu[e] * I[e];
          J[rr][iv * VW + e] = I[e] - Ip;
        }
      }
    }
  } else {
#pragma unroll
    for (int rr = 0; rr < RD; ++rr)
#pragma unroll
      for (int e = 0; e < NPL; ++e) { M[rr][e] = 0.f; J[rr][e] = 0.f; }
  }

  // Addresses of a token's rows = a wave-uniform pointer that moves by one token at a time + a constant 32-bit lane
  // offset, so that the per-token address work is a few scalar additions (a long token-serial run is bound by the
  // number of instructions one wave issues per token).
  const int Hq = a.Hq, hq = h / (H / Hq);
  const int64_t step_k = (int64_t)Hq * dk, step_v = (int64_t)H * dv;
  const TIn* qp = (const TIn*)a.q + (bos * Hq + hq) * dk;     // rows of the next token to request
  const TIn* kp = (const TIn*)a.k + (bos * Hq + hq) * dk;
  const TIn* vp = (const TIn*)a.v + (bos * H + h) * dv;
  const TIn* bp = (const TIn*)a.b + (bos * H + h) * dv;
  int64_t gt_i = bos * H + h;
  TIn* op = (TIn*)a.o + (bos * H + h) * dv;                   // output row of the token being processed
  int64_t var_i = (bos * H + h) * dv;
  int64_t go_i = gt_i;                                        // gate element of the token being processed
  unsigned lane_k[NV], lane_v[RD];   // byte offsets: base pointer in scalar registers + 32-bit lane offset
#pragma unroll
  for (int iv = 0; iv < NV; ++iv) lane_k[iv] = (unsigned)Map::vec_start(j, iv) * (unsigned)sizeof(TIn);
#pragma unroll
  for (int rr = 0; rr < RD; ++rr) lane_v[rr] = (unsigned)drow[rr] * (unsigned)sizeof(TIn);
  auto at = [](const TIn* base, unsigned bytes) { return (const TIn*)((const char*)base + bytes); };

  // request the rows of the token the pointers stand at and move them on one token (callers never request beyond the
  // last token of the sequence)
  auto request = [&](float* kk_, float* qq_, float* vv_, float* bb_, unsigned& gt_) {
#pragma unroll
    for (int iv = 0; iv < NV; ++iv) {
      load_n<VW>(at(kp, lane_k[iv]), kk_ + iv * VW);
      load_n<VW>(at(qp, lane_k[iv]), qq_ + iv * VW);
    }
#pragma unroll
    for (int rr = 0; rr < RD; ++rr) {
      vv_[rr] = to_f32(*at(vp, lane_v[rr]));
      bb_[rr] = to_f32(*at(bp, lane_v[rr]));
    }
    gt_ = load_gate_word(a.gt, gt_i, a.gate_bf16);
    kp += step_k; qp += step_k; vp += step_v; bp += step_v; gt_i += H;
  };
  // one token: state update and outputs from the token's rows
  auto token = [&](const float* kc, const float* qc, const float* vc, const float* bc, unsigned gt_word) {
    const float f = fast_exp2(-gate_value(gt_word, go_i, a.gate_bf16) * gh);
    go_i += H;
    float kk[NPL];
#pragma unroll
    for (int e = 0; e < NPL; ++e) kk[e] = kc[e] * kc[e];
#pragma unroll
    for (int rr = 0; rr < RD; ++rr) {
      float acc = 0.f, accv = 0.f;
#pragma unroll
      for (int e = 0; e < NPL; ++e) {
        M[rr][e] = fmaf(f, M[rr][e], vc[rr] * kc[e]);
        J[rr][e] = fmaf(f, J[rr][e], bc[rr] * kk[e]);
        const float rI = fast_rcp(J[rr][e] + Ip);
        acc = fmaf(M[rr][e] * rI, qc[e], acc);
        if constexpr (HAS_VAR) accv = fmaf(qc[e] * qc[e], rI, accv);
      }
      acc = row16_sum(acc) * scale;
      if (j == 0) *(TIn*)((char*)op + lane_v[rr]) = from_f32<TIn>(acc);
      if constexpr (HAS_VAR) {
        accv = row16_sum(accv) * scale;
        if (j == 0) store_rt(a.o_var, var_i + drow[rr], accv, a.var_bf16);
      }
    }
    op += step_v;
    var_i += step_v;
  };

  if constexpr (PF == 1) {
    float kc[NPL], qc[NPL], vc[RD], bc[RD];
    unsigned gtc = 0;
    if (T > 0) request(kc, qc, vc, bc, gtc);
    for (int t = 0; t < T; ++t) {
      float kn[NPL], qn[NPL], vn[RD], bn[RD];
      unsigned gtn = 0;
      const bool more = (t + 1 < T);
      if (more) request(kn, qn, vn, bn, gtn);
      token(kc, qc, vc, bc, gtc);
      if (more) {
#pragma unroll
        for (int e = 0; e < NPL; ++e) { kc[e] = kn[e]; qc[e] = qn[e]; }
#pragma unroll
        for (int rr = 0; rr < RD; ++rr) { vc[rr] = vn[rr]; bc[rr] = bn[rr]; }
        gtc = gtn;
      }
    }
  } else {
    // token t lives in register set t mod PF; it is processed from there and the set requested again for token t + PF
    float kb[PF][NPL], qb[PF][NPL], vb[PF][RD], bb[PF][RD];
    unsigned gb[PF];
#pragma unroll
    for (int u = 0; u < PF; ++u)
      if (u < T) request(kb[u], qb[u], vb[u], bb[u], gb[u]);
    // groups of PF tokens that all have a token PF ahead of them: straight-line code, no per-token conditions
    int t0 = 0;
    for (; t0 + 2 * PF <= T; t0 += PF) {
#pragma unroll
      for (int u = 0; u < PF; ++u) {
        token(kb[u], qb[u], vb[u], bb[u], gb[u]);
        request(kb[u], qb[u], vb[u], bb[u], gb[u]);
      }
    }
    // the last tokens (fewer than 2 PF): requests only while there is a token PF ahead
#pragma unroll
    for (int u = 0; u < 2 * PF; ++u) {
      const int t = t0 + u;
      if (t < T) {
        token(kb[u % PF], qb[u % PF], vb[u % PF], bb[u % PF], gb[u % PF]);
        if (t + PF < T) request(kb[u % PF], qb[u % PF], vb[u % PF], bb[u % PF], gb[u % PF]);
      }
    }
  }

  if (a.final_mu) {
#pragma unroll
    for (int rr = 0; rr < RD; ++rr) {
      const int64_t base = ((int64_t)nh * dv + drow[rr]) * dk;
#pragma unroll
      for (int iv = 0; iv < NV; ++iv) {
        float mu[VW], I[VW];
#pragma unroll
        for (int e = 0; e < VW; ++e) {
          I[e] = J[rr][iv * VW + e] + Ip;
          mu[e] = M[rr][iv * VW + e] * fast_rcp(I[e]);
        }
        if constexpr (mu16) store_n_stream<VW>((bf16_t*)a.final_mu + base + Map::vec_start(j, iv), mu);
        else store_n_stream<VW>(a.final_mu + base + Map::vec_start(j, iv), mu);
        store_n_stream<VW>(a.final_I + base + Map::vec_start(j, iv), I);
      }
    }
  }
}

template <typename TIn, int NPL>
static int launch_npl(const RecArgs& a, int rd, hipStream_t s) {
  const int64_t blocks = (int64_t)a.n_seqs * a.H * (a.dv / (4 * rd));
  if (blocks > 0x7fffffff) return PAL_E_DIM;
  // tokens in flight of a long run: as many as the registers of a wave take without cutting the occupancy it needs
  constexpr int PFL = NPL <= 4 ? 4 : (NPL <= 8 ? 3 : 2);
  const bool serial = a.T > 4;
  const bool var = a.flags & PAL_FLAG_HAS_VAR;
#define PAL_REC_LAUNCH(RD_, MU_, PF_)                                                                                     \
  do {                                                                                                                   \
    if (var) PAL_TIMED_LAUNCH(kKernRecurrentFwd, s, (recurrent_fwd_kernel<TIn, NPL, RD_, MU_, PF_, true>), dim3((unsigned)blocks), dim3(64), 0, s, a); \
    else PAL_TIMED_LAUNCH(kKernRecurrentFwd, s, (recurrent_fwd_kernel<TIn, NPL, RD_, MU_, PF_, false>), dim3((unsigned)blocks), dim3(64), 0, s, a); \
  } while (0)
  if (a.flags & PAL_FLAG_STATE_MU_BF16) {
    // the bf16 cache format of mu is a decode format: the small-wave mapping only
    PAL_REC_LAUNCH(1, true, 1);
  } else if (rd == 4) {
    PAL_REC_LAUNCH(4, false, PFL);
  } else if (serial) {
    PAL_REC_LAUNCH(1, false, PFL);
  } else {
    PAL_REC_LAUNCH(1, false, 1);
  }
#undef PAL_REC_LAUNCH
  PAL_HIP_LAUNCH_CHECK();
  return PAL_OK;
}

template <typename TIn>
static int launch_dtype(const RecArgs& a, int rd, hipStream_t s) {
  switch (a.dk / 16) {
    case 1: return launch_npl<TIn, 1>(a, rd, s);
    case 2: return launch_npl<TIn, 2>(a, rd, s);
    case 3: return launch_npl<TIn, 3>(a, rd, s);
    case 4: return launch_npl<TIn, 4>(a, rd, s);
    case 6: return launch_npl<TIn, 6>(a, rd, s);
    case 8: return launch_npl<TIn, 8>(a, rd, s);
    case 12: return launch_npl<TIn, 12>(a, rd, s);
    case 16: return launch_npl<TIn, 16>(a, rd, s);
    default: return PAL_E_HEADDIM;
  }
}

bool recurrent_dk_supported(int dk) {
  switch (dk) {
    case 16: case 32: case 48: case 64: case 96: case 128: case 192: case 256: return true;
    default: return false;
  }
}

}  // namespace pal

extern "C" int pal_recurrent_fwd(const PalDims* d, const PalFwdTensors* t, void* stream) {
  using namespace pal;
  if (!d) return PAL_E_NULL;
  PalDims dc = *d;
  dc.flags &= ~PAL_FLAG_STATE_MU_BF16;   // the one entry point that knows this flag
  int rc = check_fwd_common(&dc, t);
  if (rc) return rc;
  if (!recurrent_dk_supported(d->dk)) return PAL_E_HEADDIM;
  RecArgs a;
  a.q = t->q; a.k = t->k; a.v = t->v; a.b = t->b; a.gt = t->gt;
  a.g = t->g; a.Ip = t->Ip; a.o = t->o;
  a.o_var = (d->flags & PAL_FLAG_HAS_VAR) ? t->o_var : nullptr;
  a.init_mu = t->init_mu; a.init_I = t->init_I;
  a.final_mu = t->final_mu; a.final_I = t->final_I;
  a.cu_seqlens = t->cu_seqlens;
  a.T = d->seq_len; a.H = d->n_heads; a.dk = d->dk; a.dv = d->dv; a.n_seqs = d->n_seqs;
  a.Hq = d->n_qk_heads > 0 ? d->n_qk_heads : d->n_heads;
  a.gate_bf16 = d->gate_dtype == PAL_DTYPE_BF16;
  a.var_bf16 = d->var_dtype == PAL_DTYPE_BF16;
  a.flags = d->flags;
  a.scale = d->scale;
  // long scans: 16 value rows per wave once that still gives every SIMD of the chip two waves
  const int64_t waves16 = (int64_t)d->n_seqs * d->n_heads * (d->dv / 16);
  // decode (a handful of tokens) is pure state streaming: many small waves keep more loads in flight
  const int rd = (d->seq_len > 4 && waves16 >= 2048 && !(d->flags & PAL_FLAG_STATE_MU_BF16)) ? 4 : 1;
  hipStream_t s = (hipStream_t)stream;
  if (d->dtype == PAL_DTYPE_BF16) return launch_dtype<bf16_t>(a, rd, s);
  return launch_dtype<float>(a, rd, s);
}
