// Chunked Palimpsa forward: two kernels.
//
//  (1) chunk_state_kernel — one wave per (sequence, head, 16x16 tile of the
//      dv x dk state) walks the tiles of its sequence in order and applies
//        S <- F_C * S + (a o V)^T K          (a_s = decay from token s to tile end)
//      with bf16 MFMA contractions, fp32 state in registers.  It writes the
//      state at the START of every tile (what the reference stores as
//      intermediate_mu_state / intermediate_I_state,
//      chunk_palimpsa_forgetting_scalar.py:187-188) and the final state
//      (:214-218).  This is the only serial part of the forward.
//  (2) chunk_out_kernel — one workgroup per (tile, head), all tiles in
//      parallel.  Wave w owns key columns [16w, 16w+16).  For every value row d
//      it builds the operand X^T[n,s] = k_s[n] v_s[d] (and k_s[n]^2 b_s[d]),
//      multiplies by the decay matrix L^T on the matrix cores and finishes
//      M_t, I_t, 1/I_t, mu_t q_t in registers (the scan + division + output of
//      the reference kernel, :190-207).  Output orientation is [n, t] so the
//      sum over n stays inside a lane.
#include "chunk_common.h"
#include "pal_host.h"
#include "pal_profile.h"

namespace pal {

// ------------------------------------------------------------------ kernel 1
template <typename TIn>
__global__ __launch_bounds__(64) void chunk_state_kernel(ChunkArgs a) {
  __shared__ float sA[kC];
  const int lane = threadIdx.x, i = lane & 15, g = lane >> 4;
  const int NB = a.dk >> 4, ND = a.dv >> 4;
  int bid = blockIdx.x;
  const int nb = bid % NB; bid /= NB;
  const int dt = bid % ND; bid /= ND;
  const int h = bid % a.H;
  const int n = bid / a.H;
  const int H = a.H, dk = a.dk, dv = a.dv;
  int bos, len, cbase;
  seq_lookup(a, n, bos, len, cbase);
  const float Ip = a.Ip[h];
  const float gh = a.g[h] * kLog2e;

  // state tile in MFMA accumulator layout: rows d = 16dt + 4g + r, column n = 16nb + i
  f32x4 M = {0.f, 0.f, 0.f, 0.f}, J = {0.f, 0.f, 0.f, 0.f};
  const int64_t st_off = (((int64_t)n * H + h) * dv + 16 * dt + 4 * g) * dk + 16 * nb + i;
  if (a.init_mu) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const float mu = a.init_mu[st_off + (int64_t)r * dk];
      const float I = a.init_I[st_off + (int64_t)r * dk];
      M[r] = mu * I;
      J[r] = I - Ip;
    }
  }

  const TIn* kp = (const TIn*)a.k + (int64_t)h * dk + 16 * nb + i;
  const TIn* vp = (const TIn*)a.v + (int64_t)h * dv + 16 * dt + i;
  const TIn* bp = (const TIn*)a.b + (int64_t)h * dv + 16 * dt + i;

  const int nchunks = (len + kC - 1) / kC;
  float kr[2][8], vr[2][8], br[2][8], gtr;
  auto load_tile = [&](int c, float (&kx)[2][8], float (&vx)[2][8], float (&bx)[2][8], float& gx) {
    const int t0 = bos + c * kC;
    const int clen = min(kC, len - c * kC);
#pragma unroll
    for (int ks = 0; ks < 2; ++ks)
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int s = 8 * g + j + 32 * ks;
        const bool ok = s < clen;
        const int64_t tok = (int64_t)(t0 + (ok ? s : 0)) * H;
        const float kv = to_f32(kp[tok * dk]), vv = to_f32(vp[tok * dv]), bv = to_f32(bp[tok * dv]);
        kx[ks][j] = ok ? kv : 0.f;
        vx[ks][j] = ok ? vv : 0.f;
        bx[ks][j] = ok ? bv : 0.f;
      }
    gx = (lane < clen) ? load_gate(a.gt, (int64_t)(t0 + lane) * H + h, a.gate_bf16) : 0.f;
  };

  if (nchunks > 0) load_tile(0, kr, vr, br, gtr);
  for (int c = 0; c < nchunks; ++c) {
    // state at the start of this tile, in (mu, I) form
    {
      const int64_t co = (((int64_t)(cbase + c) * H + h) * dv + 16 * dt + 4 * g) * dk + 16 * nb + i;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float I = J[r] + Ip;
        a.chunk_mu[co + (int64_t)r * dk] = M[r] * fast_rcp(I);
        a.chunk_I[co + (int64_t)r * dk] = I;
      }
    }
    float kn[2][8], vn[2][8], bn[2][8], gtn = 0.f;
    const bool more = c + 1 < nchunks;
    if (more) load_tile(c + 1, kn, vn, bn, gtn);

    const float cs = wave_inclusive_scan(-gtr * gh, lane);
    const float tot = __shfl(cs, 63);
    __syncthreads();
    sA[lane] = fast_exp2(tot - cs);
    __syncthreads();
    const float FC = fast_exp2(tot);
    bf16x8 AM[2], AJ[2], BK[2], BKK[2];
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      const f32x4 a0 = *(const f32x4*)&sA[8 * g + 32 * ks];
      const f32x4 a1 = *(const f32x4*)&sA[8 * g + 32 * ks + 4];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float as = j < 4 ? a0[j & 3] : a1[j & 3];
        AM[ks][j] = (bf16_t)(as * vr[ks][j]);
        AJ[ks][j] = (bf16_t)(as * br[ks][j]);
        BK[ks][j] = (bf16_t)kr[ks][j];
        BKK[ks][j] = (bf16_t)(kr[ks][j] * kr[ks][j]);
      }
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) { M[r] *= FC; J[r] *= FC; }
    M = mfma16(AM[0], BK[0], M);
    J = mfma16(AJ[0], BKK[0], J);
    M = mfma16(AM[1], BK[1], M);
    J = mfma16(AJ[1], BKK[1], J);
    if (more) {
#pragma unroll
      for (int ks = 0; ks < 2; ++ks)
#pragma unroll
        for (int j = 0; j < 8; ++j) { kr[ks][j] = kn[ks][j]; vr[ks][j] = vn[ks][j]; br[ks][j] = bn[ks][j]; }
      gtr = gtn;
    }
  }
  if (a.final_mu) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const float I = J[r] + Ip;
      a.final_mu[st_off + (int64_t)r * dk] = M[r] * fast_rcp(I);
      a.final_I[st_off + (int64_t)r * dk] = I;
    }
  }
}

// ------------------------------------------------------------------ kernel 2
constexpr int kVS = 68;  // row stride (floats) of the transposed v/b staging tiles
constexpr int kDG = 16;  // value rows per staging group

// index of the L operand for (tb, ks): tb0,tb1 -> one K step; tb2,tb3 -> two
__device__ __forceinline__ constexpr int lidx(int tb, int ks) { return tb < 2 ? tb : 2 + 2 * (tb - 2) + ks; }

template <typename TIn, int NB, bool HAS_VAR>
__global__ __launch_bounds__(NB * 64) void chunk_out_kernel(ChunkArgs a) {
  extern __shared__ float smem[];
  float* sC = smem;                       // [64] running log2-decay inside the tile
  float* sV = sC + kC;                    // [16][kVS] v^T of the current value-row group
  float* sB = sV + kDG * kVS;             // [16][kVS]
  float* sO = sB + kDG * kVS;             // [NB][16][64] per-wave partial outputs
  float* sOv = sO + NB * kDG * kC;        // same for o_var
  constexpr int NT = NB * 64;
  const int tid = threadIdx.x, lane = tid & 63, nb = tid >> 6, i = lane & 15, g = lane >> 4;
  const int H = a.H, dk = a.dk, dv = a.dv;
  const int cidx = blockIdx.x / H, h = blockIdx.x % H;
  int seq, t0, clen, cis;
  chunk_lookup(a, cidx, seq, t0, clen, cis);
  const float Ip = a.Ip[h];
  const float gh = a.g[h] * kLog2e;

  if (nb == 0) {
    const float gt = (lane < clen) ? load_gate(a.gt, (int64_t)(t0 + lane) * H + h, a.gate_bf16) : 0.f;
    sC[lane] = wave_inclusive_scan(-gt * gh, lane);
  }
  // staging of v^T, b^T for one group of 16 value rows: work item = (token s, 4 rows)
  const TIn* vp = (const TIn*)a.v + ((int64_t)t0 * H + h) * dv;
  const TIn* bp = (const TIn*)a.b + ((int64_t)t0 * H + h) * dv;
  constexpr int NITEM = (kC * kDG / 4 + NT - 1) / NT;  // items per thread
  float vst[NITEM][4], bst[NITEM][4];
  auto stage_load = [&](int dg) {
#pragma unroll
    for (int it = 0; it < NITEM; ++it) {
      const int idx = tid + it * NT;
      const int s = idx >> 2, dq = idx & 3;
      if (idx < kC * kDG / 4 && s < clen) {
        load_vec<4>(vp + (int64_t)s * H * dv + dg * kDG + 4 * dq, vst[it]);
        load_vec<4>(bp + (int64_t)s * H * dv + dg * kDG + 4 * dq, bst[it]);
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) { vst[it][e] = 0.f; bst[it][e] = 0.f; }
      }
    }
  };
  auto stage_store = [&]() {
#pragma unroll
    for (int it = 0; it < NITEM; ++it) {
      const int idx = tid + it * NT;
      const int s = idx >> 2, dq = idx & 3;
      if (idx < kC * kDG / 4) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          sV[(4 * dq + e) * kVS + s] = vst[it][e];
          sB[(4 * dq + e) * kVS + s] = bst[it][e];
        }
      }
    }
  };
  stage_load(0);
  stage_store();
  __syncthreads();

  // ---- per-wave constants of this tile
  float F[4], Gi[4], ct[4];
#pragma unroll
  for (int tb = 0; tb < 4; ++tb) {
    ct[tb] = sC[16 * tb + i];
    F[tb] = fast_exp2(ct[tb]);
    Gi[tb] = (1.f - F[tb]) * Ip;
  }
  bf16x8 Lr[6];
  float kA[2][8], kk[2][8];
  {
    const TIn* kp = (const TIn*)a.k + ((int64_t)t0 * H + h) * dk + 16 * nb + i;
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      float cs[8];
      *(f32x4*)&cs[0] = *(const f32x4*)&sC[8 * g + 32 * ks];
      *(f32x4*)&cs[4] = *(const f32x4*)&sC[8 * g + 32 * ks + 4];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int s = 8 * g + j + 32 * ks;
        const bool ok = s < clen;
        const float kv = to_f32(kp[(int64_t)(ok ? s : 0) * H * dk]);
        kA[ks][j] = ok ? kv : 0.f;
        kk[ks][j] = kA[ks][j] * kA[ks][j];
#pragma unroll
        for (int tb = (ks ? 2 : 0); tb < 4; ++tb) {
          const int t = 16 * tb + i;
          const float lv = (s <= t) ? fast_exp2(ct[tb] - cs[j]) : 0.f;
          Lr[lidx(tb, ks)][j] = (bf16_t)lv;
        }
      }
    }
  }
  float qD[4][4];
  {
    const TIn* qp = (const TIn*)a.q + ((int64_t)t0 * H + h) * dk + 16 * nb + 4 * g;
#pragma unroll
    for (int tb = 0; tb < 4; ++tb) {
      const int t = 16 * tb + i;
      if (t < clen) {
        load_vec<4>(qp + (int64_t)t * H * dk, qD[tb]);
      } else {
#pragma unroll
        for (int r = 0; r < 4; ++r) qD[tb][r] = 0.f;
      }
    }
  }
  const float scale = a.scale;
  const float* cmu = a.chunk_mu + (((int64_t)cidx * H + h) * dv) * dk + 16 * nb + 4 * g;
  const float* cI = a.chunk_I + (((int64_t)cidx * H + h) * dv) * dk + 16 * nb + 4 * g;

  const int n_groups = dv / kDG;
  for (int dg = 0; dg < n_groups; ++dg) {
    if (dg + 1 < n_groups) stage_load(dg + 1);
#pragma unroll 2
    for (int dd = 0; dd < kDG; ++dd) {
      const int d = dg * kDG + dd;
      const f32x4 mu0 = *(const f32x4*)(cmu + (int64_t)d * dk);
      const f32x4 I0 = *(const f32x4*)(cI + (int64_t)d * dk);
      float M0[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) M0[r] = mu0[r] * I0[r];
      bf16x8 XM[2], XJ[2];
#pragma unroll
      for (int ks = 0; ks < 2; ++ks) {
        const f32x4 v0 = *(const f32x4*)&sV[dd * kVS + 8 * g + 32 * ks];
        const f32x4 v1 = *(const f32x4*)&sV[dd * kVS + 8 * g + 32 * ks + 4];
        const f32x4 b0 = *(const f32x4*)&sB[dd * kVS + 8 * g + 32 * ks];
        const f32x4 b1 = *(const f32x4*)&sB[dd * kVS + 8 * g + 32 * ks + 4];
#pragma unroll
        for (int j = 0; j < 8; j += 2) {
          const float va = j < 4 ? v0[j & 3] : v1[j & 3], vb = j < 4 ? v0[(j & 3) + 1] : v1[(j & 3) + 1];
          const float ba = j < 4 ? b0[j & 3] : b1[j & 3], bb = j < 4 ? b0[(j & 3) + 1] : b1[(j & 3) + 1];
          const bf16x2 pm = pack2(kA[ks][j] * va, kA[ks][j + 1] * vb);
          const bf16x2 pj = pack2(kk[ks][j] * ba, kk[ks][j + 1] * bb);
          XM[ks][j] = pm[0]; XM[ks][j + 1] = pm[1];
          XJ[ks][j] = pj[0]; XJ[ks][j + 1] = pj[1];
        }
      }
      float p[4], pv[4];
#pragma unroll
      for (int tb = 0; tb < 4; ++tb) {
        f32x4 accM = {0.f, 0.f, 0.f, 0.f};
        f32x4 accI = {Gi[tb], Gi[tb], Gi[tb], Gi[tb]};
        accM = mfma16(XM[0], Lr[lidx(tb, 0)], accM);
        accI = mfma16(XJ[0], Lr[lidx(tb, 0)], accI);
        if (tb >= 2) {
          accM = mfma16(XM[1], Lr[lidx(tb, 1)], accM);
          accI = mfma16(XJ[1], Lr[lidx(tb, 1)], accI);
        }
        float acc = 0.f, accv = 0.f;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const float Mf = fmaf(F[tb], M0[r], accM[r]);
          const float If = fmaf(F[tb], I0[r], accI[r]);
          const float rI = fast_rcp(If);
          acc = fmaf(Mf * rI, qD[tb][r], acc);
          if (HAS_VAR) accv = fmaf(qD[tb][r] * qD[tb][r], rI, accv);
        }
        p[tb] = acc;
        pv[tb] = accv;
      }
#pragma unroll
      for (int tb = 0; tb < 4; ++tb) {
        p[tb] = rows4_sum(p[tb]);
        if (HAS_VAR) pv[tb] = rows4_sum(pv[tb]);
      }
      if (g == 0) {
#pragma unroll
        for (int tb = 0; tb < 4; ++tb) {
          sO[(nb * kDG + dd) * kC + 16 * tb + i] = p[tb];
          if (HAS_VAR) sOv[(nb * kDG + dd) * kC + 16 * tb + i] = pv[tb];
        }
      }
    }
    __syncthreads();
    // flush the group's outputs: work item = (token t, 4 value rows)
    for (int idx = tid; idx < kC * kDG / 4; idx += NT) {
      const int t = idx >> 2, dq = idx & 3;
      if (t < clen) {
        float acc[4] = {0.f, 0.f, 0.f, 0.f}, accv[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int w = 0; w < NB; ++w)
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            acc[e] += sO[(w * kDG + 4 * dq + e) * kC + t];
            if (HAS_VAR) accv[e] += sOv[(w * kDG + 4 * dq + e) * kC + t];
          }
        const int64_t off = ((int64_t)(t0 + t) * H + h) * dv + dg * kDG + 4 * dq;
        TIn* op = (TIn*)a.o + off;
#pragma unroll
        for (int e = 0; e < 4; ++e) op[e] = from_f32<TIn>(acc[e] * scale);
        if (HAS_VAR) {
#pragma unroll
          for (int e = 0; e < 4; ++e) store_rt(a.o_var, off + e, accv[e] * scale, a.var_bf16);
        }
      }
    }
    if (dg + 1 < n_groups) stage_store();
    __syncthreads();
  }
}

template <typename TIn, int NB>
static int launch_out_nb(const ChunkArgs& a, hipStream_t s) {
  const bool var = a.flags & PAL_FLAG_HAS_VAR;
  const size_t lds = sizeof(float) * (kC + 2 * kDG * kVS + (var ? 2 : 1) * NB * kDG * kC);
  const int64_t blocks = (int64_t)a.total_chunks * a.H;
  if (blocks > 0x7fffffff) return PAL_E_DIM;
  if (lds > kMaxLds) return PAL_E_HEADDIM;
  if (var) {
    if (int rc = allow_lds((const void*)&chunk_out_kernel<TIn, NB, true>, lds)) return rc;
    PAL_TIMED_LAUNCH(kKernChunkOut, s, (chunk_out_kernel<TIn, NB, true>), dim3((unsigned)blocks), dim3(NB * 64), lds, s, a);
  } else {
    if (int rc = allow_lds((const void*)&chunk_out_kernel<TIn, NB, false>, lds)) return rc;
    PAL_TIMED_LAUNCH(kKernChunkOut, s, (chunk_out_kernel<TIn, NB, false>), dim3((unsigned)blocks), dim3(NB * 64), lds, s, a);
  }
  PAL_HIP_LAUNCH_CHECK();
  return PAL_OK;
}

template <typename TIn>
static int launch_out(const ChunkArgs& a, hipStream_t s) {
  switch (a.dk / 16) {
    case 1: return launch_out_nb<TIn, 1>(a, s);
    case 2: return launch_out_nb<TIn, 2>(a, s);
    case 3: return launch_out_nb<TIn, 3>(a, s);
    case 4: return launch_out_nb<TIn, 4>(a, s);
    case 5: return launch_out_nb<TIn, 5>(a, s);
    case 6: return launch_out_nb<TIn, 6>(a, s);
    case 7: return launch_out_nb<TIn, 7>(a, s);
    case 8: return launch_out_nb<TIn, 8>(a, s);
    case 9: return launch_out_nb<TIn, 9>(a, s);
    case 10: return launch_out_nb<TIn, 10>(a, s);
    case 11: return launch_out_nb<TIn, 11>(a, s);
    case 12: return launch_out_nb<TIn, 12>(a, s);
    case 13: return launch_out_nb<TIn, 13>(a, s);
    case 14: return launch_out_nb<TIn, 14>(a, s);
    case 15: return launch_out_nb<TIn, 15>(a, s);
    case 16: return launch_out_nb<TIn, 16>(a, s);
    default: return PAL_E_HEADDIM;
  }
}

void fill_chunk_args(ChunkArgs& a, const PalDims* d, const PalFwdTensors* t) {
  a.q = t->q; a.k = t->k; a.v = t->v; a.b = t->b; a.gt = t->gt;
  a.g = t->g; a.Ip = t->Ip; a.o = t->o;
  a.o_var = (d->flags & PAL_FLAG_HAS_VAR) ? t->o_var : nullptr;
  a.init_mu = t->init_mu; a.init_I = t->init_I;
  a.final_mu = t->final_mu; a.final_I = t->final_I;
  a.cu_seqlens = t->cu_seqlens;
  a.chunk_table = (d->flags & PAL_FLAG_VARLEN) ? t->chunk_table : nullptr;
  a.chunk_offsets = (d->flags & PAL_FLAG_VARLEN) ? t->chunk_offsets : nullptr;
  a.chunk_mu = t->chunk_mu; a.chunk_I = t->chunk_I;
  a.T = d->seq_len; a.H = d->n_heads; a.dk = d->dk; a.dv = d->dv;
  a.n_seqs = d->n_seqs; a.total_chunks = d->total_chunks;
  a.gate_bf16 = d->gate_dtype == PAL_DTYPE_BF16;
  a.var_bf16 = d->var_dtype == PAL_DTYPE_BF16;
  a.flags = d->flags;
  a.scale = d->scale;
}

}  // namespace pal

extern "C" int pal_chunk_fwd(const PalDims* d, const PalFwdTensors* t, void* stream) {
  using namespace pal;
  int rc = check_chunk_common(d, t);
  if (rc) return rc;
  ChunkArgs a;
  fill_chunk_args(a, d, t);
  hipStream_t s = (hipStream_t)stream;
  const int64_t waves = (int64_t)d->n_seqs * d->n_heads * (d->dv / 16) * (d->dk / 16);
  if (waves > 0x7fffffff) return PAL_E_DIM;
  if (d->dtype == PAL_DTYPE_BF16) PAL_TIMED_LAUNCH(kKernChunkState, s, (chunk_state_kernel<bf16_t>), dim3((unsigned)waves), dim3(64), 0, s, a);
  else PAL_TIMED_LAUNCH(kKernChunkState, s, (chunk_state_kernel<float>), dim3((unsigned)waves), dim3(64), 0, s, a);
  PAL_HIP_LAUNCH_CHECK();
  if (d->dtype == PAL_DTYPE_BF16) return launch_out<bf16_t>(a, s);
  return launch_out<float>(a, s);
}
