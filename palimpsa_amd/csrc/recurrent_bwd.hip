// Backward of the token-serial Palimpsa path, fp32 end to end.
//
// The reference has no such kernel (fused_recurrent_palimpsa.py:250-253 raises
// NotImplementedError); the gradients are those of the naive recurrence
// (chunk_palimpsa_forgetting_scalar.py:669-725):
//   G_t = scale do_t q_t^T,  dMloc_t = G_t/I_t,  dJloc_t = -G_t M_t/I_t^2 - scale dovar_t (q_t*q_t)^T/I_t^2
//   dM_t = dMloc_t + f_{t+1} dM_{t+1}  (same for J),  dq_t = scale mu_t^T do_t + 2 scale q_t*((1/I_t)^T dovar_t)
//   dv_t = dM_t k_t, db_t = dJ_t (k_t*k_t), dk_t = dM_t^T v_t + 2 k_t*(dJ_t^T b_t)
//   dlogf_t = <dM_t, f_t M_{t-1}> + <dJ_t, f_t J_{t-1}>,  dgt = -g dlogf, dg = -sum gt dlogf, dIp = sum dJloc
//
// Three kernels:
//  state   forward scan that only stores (M, J) every S tokens (S = 16, or 8 for dk > 128);
//  bwd     one wave per (sequence, head, 4 value rows), same lane mapping as the forward
//          (a state row on the 16 lanes of a DPP row).  Segments are walked backwards; inside a
//          segment the states *before* each token are recomputed once and stashed in LDS, then the
//          tokens are processed in reverse with dM, dJ in registers.  Sums over dk stay inside a
//          DPP row; sums over the value rows of other waves go to per-tile partial buffers;
//  reduce  adds the partials in a fixed order (deterministic, no atomics) and forms dgt, dg, dIp.
#include "pal_common.h"
#include "pal_host.h"
#include "pal_profile.h"

namespace pal {

bool recurrent_dk_supported(int dk);

struct RecBwdArgs {
  const void *q, *k, *v, *b, *gt, *d_o, *d_o_var;
  const float *g, *Ip, *init_mu, *init_I;
  const int32_t* cu_seqlens;
  void *g_dq, *g_dk, *g_dv, *g_db;
  float *dgt, *dg, *dIp, *d_init_mu, *d_init_I;
  // workspace
  int32_t* seg_off;      // [N+1] first segment of every sequence
  float *ckM, *ckJ;      // [segments, H, dv, dk]
  float *pdq, *pdk;      // [ND][tokens, H, dk]
  float* pdl;            // [ND][tokens, H]
  float* dl;             // [tokens, H] d log f
  float *pdIp, *pInit;   // [ND][N, H]
  double *dgPart, *dIpPart;  // [N, H]
  int32_t T, H, dk, dv, n_seqs, S, tokens, ND;
  int32_t seg_cap;       // segments the checkpoint buffers hold
  int32_t Hq;            // heads of q, k, dq, dk (H, or a divisor of it: a group of H / Hq value heads shares one)
  int32_t gate_bf16, var_bf16, out_bf16;
  uint32_t flags;
  float scale;
};

template <int NPL>
struct NMapB {
  static constexpr int VW = (NPL % 4 == 0) ? 4 : ((NPL % 2 == 0) ? 2 : 1);
  static constexpr int NV = NPL / VW;
  __device__ static __forceinline__ int vec_start(int j, int iv) { return 16 * VW * iv + VW * j; }
};

__device__ __forceinline__ void rec_seq(const RecBwdArgs& a, int n, int64_t& bos, int& len, int& segbase) {
  if (a.cu_seqlens) {
    int b0;
    packed_seq_bounds(a.cu_seqlens, n, a.T, b0, len);
    bos = b0;
    // the segments of a sequence stay inside the checkpoint buffers
    segbase = min(a.seg_off[n], a.seg_cap);
    len = min(len, (a.seg_cap - segbase) * a.S);
  } else {
    bos = (int64_t)n * a.T;
    len = a.T;
    segbase = n * ((a.T + a.S - 1) / a.S);
  }
}

__global__ void recurrent_bwd_segoff_kernel(RecBwdArgs a) {
  if (threadIdx.x != 0 || blockIdx.x != 0) return;
  int acc = 0;
  a.seg_off[0] = 0;
  for (int n = 0; n < a.n_seqs; ++n) {
    int b0, len;
    packed_seq_bounds(a.cu_seqlens, n, a.T, b0, len);
    acc += (len + a.S - 1) / a.S;
    a.seg_off[n + 1] = acc;
  }
}

// tokens whose rows are in flight in the token loops of the two kernels below (registers: 2 NPL + 5 per token)
template <int NPL>
constexpr int kRecBwdPrefetch = NPL <= 4 ? 3 : 2;

// ------------------------------------------------------------ state checkpoints
template <typename TIn, int NPL>
__global__ __launch_bounds__(64) void recurrent_bwd_state_kernel(RecBwdArgs a) {
  using Map = NMapB<NPL>;
  constexpr int VW = Map::VW, NV = Map::NV;
  const int lane = threadIdx.x, j = lane & 15, grp = lane >> 4;
  const int ND = a.ND;
  const int tile = blockIdx.x % ND, nh = blockIdx.x / ND, h = nh % a.H, n = nh / a.H;
  const int dk = a.dk, dv = a.dv, H = a.H, S = a.S;
  int64_t bos; int len, segbase;
  rec_seq(a, n, bos, len, segbase);
  const float gh = a.g[h] * kLog2e, Ip = a.Ip[h];
  const int drow = tile * 4 + grp;
  float M[NPL], J[NPL];
  if (a.init_mu) {
    const int64_t base = ((int64_t)nh * dv + drow) * dk;
#pragma unroll
    for (int iv = 0; iv < NV; ++iv) {
      float mu[VW], I[VW];
      load_vec<VW>(a.init_mu + base + Map::vec_start(j, iv), mu);
      load_vec<VW>(a.init_I + base + Map::vec_start(j, iv), I);
#pragma unroll
      for (int e = 0; e < VW; ++e) { M[iv * VW + e] = mu[e] * I[e]; J[iv * VW + e] = I[e] - Ip; }
    }
  } else {
#pragma unroll
    for (int e = 0; e < NPL; ++e) { M[e] = 0.f; J[e] = 0.f; }
  }
  const TIn* kp = (const TIn*)a.k + (bos * a.Hq + h / (H / a.Hq)) * dk;
  const TIn* vp = (const TIn*)a.v + (bos * H + h) * dv + drow;
  const TIn* bp = (const TIn*)a.b + (bos * H + h) * dv + drow;
  // the rows of PF tokens are in flight: a token is taken from its register set and the set reloaded at once with
  // the token PF ahead (always issued, clamped to the last token: the same number of requests in every iteration)
  constexpr int PF = kRecBwdPrefetch<NPL>;
  // (the gate is requested as the aligned word that holds it and decoded when the token is taken up: one kind of
  //  request for both storage types, so that no wait is forced where the two would meet)
  float kb[PF][NPL], vb[PF], bb_[PF];
  unsigned gb[PF];
  auto load_rows = [&](int t, float* kk, float& vv, float& bb, unsigned& gg) {
#pragma unroll
    for (int iv = 0; iv < NV; ++iv) load_vec<VW>(kp + (int64_t)t * a.Hq * dk + Map::vec_start(j, iv), kk + iv * VW);
    vv = to_f32(vp[(int64_t)t * H * dv]);
    bb = to_f32(bp[(int64_t)t * H * dv]);
    gg = load_gate_word(a.gt, (bos + t) * H + h, a.gate_bf16);
  };
  if (len > 0) {
#pragma unroll
    for (int u = 0; u < PF; ++u) load_rows(min(u, len - 1), kb[u], vb[u], bb_[u], gb[u]);
  }
  for (int t0 = 0; t0 < len; t0 += PF) {
#pragma unroll
    for (int u = 0; u < PF; ++u) {
      const int t = t0 + u;
      float kc[NPL];
#pragma unroll
      for (int e = 0; e < NPL; ++e) kc[e] = kb[u][e];
      const float vv = vb[u], bb = bb_[u];
      const unsigned gw = gb[u];
      load_rows(min(t + PF, len - 1), kb[u], vb[u], bb_[u], gb[u]);
      if (t < len) {
        const float gt = gate_value(gw, (bos + t) * H + h, a.gate_bf16);
        if (t % S == 0) {
          const int64_t co = (((int64_t)(segbase + t / S) * H + h) * dv + drow) * dk;
#pragma unroll
          for (int iv = 0; iv < NV; ++iv) {
            store_vec<VW>(a.ckM + co + Map::vec_start(j, iv), M + iv * VW);
            store_vec<VW>(a.ckJ + co + Map::vec_start(j, iv), J + iv * VW);
          }
        }
        const float f = fast_exp2(-gt * gh);
#pragma unroll
        for (int e = 0; e < NPL; ++e) {
          M[e] = fmaf(f, M[e], vv * kc[e]);
          J[e] = fmaf(f, J[e], bb * kc[e] * kc[e]);
        }
      }
    }
  }
}

// ------------------------------------------------------------------- backward
template <typename TIn, int NPL, bool HAS_VAR>
__global__ __launch_bounds__(64) void recurrent_bwd_kernel(RecBwdArgs a) {
  using Map = NMapB<NPL>;
  constexpr int VW = Map::VW, NV = Map::NV;
  extern __shared__ float stash[];   // [S][2*NPL][64]
  const int lane = threadIdx.x, j = lane & 15, grp = lane >> 4;
  const int ND = a.ND;
  const int tile = blockIdx.x % ND, nh = blockIdx.x / ND, h = nh % a.H, n = nh / a.H;
  const int dk = a.dk, dv = a.dv, H = a.H, S = a.S;
  int64_t bos; int len, segbase;
  rec_seq(a, n, bos, len, segbase);
  const float gval = a.g[h];
  const float gh = gval * kLog2e, Ip = a.Ip[h], scale = a.scale;
  constexpr bool has_var = HAS_VAR;
  const int drow = tile * 4 + grp;
  const TIn* qp = (const TIn*)a.q + (bos * a.Hq + h / (H / a.Hq)) * dk;
  const TIn* kp = (const TIn*)a.k + (bos * a.Hq + h / (H / a.Hq)) * dk;
  const int64_t vrow = (bos * H + h) * dv + drow;
  const TIn* vp = (const TIn*)a.v + vrow;
  const TIn* bp = (const TIn*)a.b + vrow;
  const TIn* dop = (const TIn*)a.d_o + vrow;
  constexpr int PF = kRecBwdPrefetch<NPL>;
  // gates and the gradient of the uncertainty output (element types chosen at run time) are requested as the aligned
  // word that holds them and decoded when the token is taken up: one kind of request for both storage types, so that
  // the rows of the tokens ahead stay in flight (a type branch at the request would be waited for on the spot)
  auto load_fwd_rows = [&](int t, float* kk, float& vv, float& bb, unsigned& gg) {
#pragma unroll
    for (int iv = 0; iv < NV; ++iv) load_vec<VW>(kp + (int64_t)t * a.Hq * dk + Map::vec_start(j, iv), kk + iv * VW);
    vv = to_f32(vp[(int64_t)t * H * dv]);
    bb = to_f32(bp[(int64_t)t * H * dv]);
    gg = load_gate_word(a.gt, (bos + t) * H + h, a.gate_bf16);
  };
  auto load_bwd_rows = [&](int t, float* kk, float* qq, float& vv, float& bb, float& dd, unsigned& dvar, unsigned& gg) {
#pragma unroll
    for (int iv = 0; iv < NV; ++iv) {
      load_vec<VW>(kp + (int64_t)t * a.Hq * dk + Map::vec_start(j, iv), kk + iv * VW);
      load_vec<VW>(qp + (int64_t)t * a.Hq * dk + Map::vec_start(j, iv), qq + iv * VW);
    }
    vv = to_f32(vp[(int64_t)t * H * dv]);
    bb = to_f32(bp[(int64_t)t * H * dv]);
    dd = to_f32(dop[(int64_t)t * H * dv]);
    dvar = 0u;
    if constexpr (HAS_VAR) dvar = load_gate_word(a.d_o_var, vrow + (int64_t)t * H * dv, a.var_bf16);
    gg = load_gate_word(a.gt, (bos + t) * H + h, a.gate_bf16);
  };
  float dMc[NPL], dJc[NPL];   // f_{t+1} dM_{t+1}: what flows into token t from the future
#pragma unroll
  for (int e = 0; e < NPL; ++e) { dMc[e] = 0.f; dJc[e] = 0.f; }
  float sig = 0.f;
  const int nseg = (len + S - 1) / S;
  for (int seg = nseg - 1; seg >= 0; --seg) {
    const int ts = seg * S, cnt = min(S, len - ts);
    float M[NPL], J[NPL];
    {
      const int64_t co = (((int64_t)(segbase + seg) * H + h) * dv + drow) * dk;
#pragma unroll
      for (int iv = 0; iv < NV; ++iv) {
        load_vec<VW>(a.ckM + co + Map::vec_start(j, iv), M + iv * VW);
        load_vec<VW>(a.ckJ + co + Map::vec_start(j, iv), J + iv * VW);
      }
    }
    // states before every token of the segment (rows of PF tokens in flight, see recurrent_bwd_state_kernel)
    {
      float kb[PF][NPL], vb[PF], bb_[PF];
      unsigned gb[PF];
#pragma unroll
      for (int u = 0; u < PF; ++u) load_fwd_rows(ts + min(u, cnt - 1), kb[u], vb[u], bb_[u], gb[u]);
      for (int j0 = 0; j0 < cnt; j0 += PF) {
#pragma unroll
        for (int u = 0; u < PF; ++u) {
          const int jj = j0 + u;
          float kc[NPL];
#pragma unroll
          for (int e = 0; e < NPL; ++e) kc[e] = kb[u][e];
          const float vv = vb[u], bb = bb_[u];
          const float gt = gate_value(gb[u], (bos + ts + min(jj, cnt - 1)) * H + h, a.gate_bf16);
          load_fwd_rows(ts + min(jj + PF, cnt - 1), kb[u], vb[u], bb_[u], gb[u]);
          if (jj < cnt) {
#pragma unroll
            for (int e = 0; e < NPL; ++e) {
              stash[(jj * 2 * NPL + e) * 64 + lane] = M[e];
              stash[(jj * 2 * NPL + NPL + e) * 64 + lane] = J[e];
            }
            if (jj + 1 < cnt) {
              const float f = fast_exp2(-gt * gh);
#pragma unroll
              for (int e = 0; e < NPL; ++e) {
                M[e] = fmaf(f, M[e], vv * kc[e]);
                J[e] = fmaf(f, J[e], bb * kc[e] * kc[e]);
              }
            }
          }
        }
      }
    }
    // reverse over the tokens of the segment, rows of PF tokens in flight (token cnt-1-r in round r)
    float rk[PF][NPL], rq[PF][NPL], rv[PF], rb[PF], rdo[PF];
    unsigned rdv[PF], rg[PF];
#pragma unroll
    for (int u = 0; u < PF; ++u) load_bwd_rows(ts + max(cnt - 1 - u, 0), rk[u], rq[u], rv[u], rb[u], rdo[u], rdv[u], rg[u]);
    for (int r0 = 0; r0 < cnt; r0 += PF) {
#pragma unroll
    for (int u = 0; u < PF; ++u) {
      const int jj = cnt - 1 - (r0 + u);
      float kc[NPL], qc[NPL];
#pragma unroll
      for (int e = 0; e < NPL; ++e) { kc[e] = rk[u][e]; qc[e] = rq[u][e]; }
      const float vv = rv[u], bb = rb[u], dov = scale * rdo[u];
      const int tl = ts + max(jj, 0);                       // the token this register set was requested for
      const float gt = gate_value(rg[u], (bos + tl) * H + h, a.gate_bf16);
      float dvv = 0.f;
      if constexpr (HAS_VAR) dvv = scale * gate_value(rdv[u], vrow + (int64_t)tl * H * dv, a.var_bf16);
      load_bwd_rows(ts + max(jj - PF, 0), rk[u], rq[u], rv[u], rb[u], rdo[u], rdv[u], rg[u]);
      if (jj < 0) continue;
      const int t = ts + jj;
      const float f = fast_exp2(-gt * gh);
      float dqp[NPL], dkp[NPL];
      float dvs = 0.f, dbs = 0.f, dls = 0.f;
#pragma unroll
      for (int e = 0; e < NPL; ++e) {
        const float Mp = f * stash[(jj * 2 * NPL + e) * 64 + lane];         // f_t M_{t-1}
        const float Jp = f * stash[(jj * 2 * NPL + NPL + e) * 64 + lane];
        const float kk = kc[e] * kc[e];
        const float Mt = fmaf(vv, kc[e], Mp);
        const float It = fmaf(bb, kk, Jp) + Ip;
        const float rI = fast_rcp(It);
        const float mu = Mt * rI;
        const float dMl = dov * qc[e] * rI;
        float dJl = -dMl * mu;
        float dq_e = mu * dov;
        if (has_var) {
          const float wq = dvv * qc[e];
          dJl = fmaf(-wq * qc[e] * rI, rI, dJl);
          dq_e = fmaf(2.f * wq, rI, dq_e);
        }
        sig += dJl;
        const float dMt = dMl + dMc[e];
        const float dJt = dJl + dJc[e];
        dqp[e] = dq_e;
        dkp[e] = fmaf(dMt, vv, 2.f * kc[e] * dJt * bb);
        dvs = fmaf(dMt, kc[e], dvs);
        dbs = fmaf(dJt, kk, dbs);
        dls = fmaf(dMt, Mp, dls);
        dls = fmaf(dJt, Jp, dls);
        dMc[e] = f * dMt;
        dJc[e] = f * dJt;
      }
      dvs = row16_sum(dvs);
      dbs = row16_sum(dbs);
      if (j == 0) {
        store_rt(a.g_dv, vrow + (int64_t)t * H * dv, dvs, a.out_bf16);
        store_rt(a.g_db, vrow + (int64_t)t * H * dv, dbs, a.out_bf16);
      }
      dls = wave_sum(dls);
      if (lane == 0) a.pdl[((int64_t)tile * a.tokens + bos + t) * H + h] = dls;
#pragma unroll
      for (int e = 0; e < NPL; ++e) { dqp[e] = rows4_sum(dqp[e]); dkp[e] = rows4_sum(dkp[e]); }
      if (grp == 0) {
        const int64_t po = (((int64_t)tile * a.tokens + bos + t) * H + h) * dk;
#pragma unroll
        for (int iv = 0; iv < NV; ++iv) {
          store_vec<VW>(a.pdq + po + Map::vec_start(j, iv), dqp + iv * VW);
          store_vec<VW>(a.pdk + po + Map::vec_start(j, iv), dkp + iv * VW);
        }
      }
    }
    }
  }
  // what reaches the initial state: dM_0 = f_1 dM_1
  float sinit = 0.f;
  if (a.init_mu) {
    const int64_t base = ((int64_t)nh * dv + drow) * dk;
#pragma unroll
    for (int iv = 0; iv < NV; ++iv) {
      float mu[VW], I[VW], gmu[VW], gI[VW];
      load_vec<VW>(a.init_mu + base + Map::vec_start(j, iv), mu);
      load_vec<VW>(a.init_I + base + Map::vec_start(j, iv), I);
#pragma unroll
      for (int e = 0; e < VW; ++e) {
        gmu[e] = dMc[iv * VW + e] * I[e];
        gI[e] = fmaf(dMc[iv * VW + e], mu[e], dJc[iv * VW + e]);
        sinit += dJc[iv * VW + e];
      }
      if (a.d_init_mu) {
        store_vec<VW>(a.d_init_mu + base + Map::vec_start(j, iv), gmu);
        store_vec<VW>(a.d_init_I + base + Map::vec_start(j, iv), gI);
      }
    }
  }
  sig = wave_sum(sig);
  sinit = wave_sum(sinit);
  if (lane == 0) {
    a.pdIp[(int64_t)tile * a.n_seqs * H + nh] = sig;
    a.pInit[(int64_t)tile * a.n_seqs * H + nh] = sinit;
  }
}

// --------------------------------------------------------------------- reduce
// dq, dk: one thread per (token, q/k head, n), summing the value-row tiles of every value head of the group in a
// fixed order; d log f and dgt: one thread per (token, head)
__global__ __launch_bounds__(256) void recurrent_bwd_reduce_kernel(RecBwdArgs a) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int64_t nqk = (int64_t)a.tokens * a.H * a.dk;       // entries of one partial buffer (one row per value head)
  const int64_t nout = (int64_t)a.tokens * a.Hq * a.dk;
  if (idx < nout) {
    const int rep = a.H / a.Hq;
    const int n = (int)(idx % a.dk);
    const int64_t row = idx / a.dk;                          // token * Hq + hq
    float sq = 0.f, sk = 0.f;
    for (int r = 0; r < rep; ++r) {
      const int64_t src = (row * rep + r) * a.dk + n;        // value head hq * rep + r of the same token
      for (int w = 0; w < a.ND; ++w) {
        sq += a.pdq[(int64_t)w * nqk + src];
        sk += a.pdk[(int64_t)w * nqk + src];
      }
    }
    store_rt(a.g_dq, idx, sq, a.out_bf16);
    store_rt(a.g_dk, idx, sk, a.out_bf16);
  }
  const int64_t nth = (int64_t)a.tokens * a.H;
  if (idx < nth) {
    float s = 0.f;
    for (int w = 0; w < a.ND; ++w) s += a.pdl[(int64_t)w * nth + idx];
    a.dl[idx] = s;
    a.dgt[idx] = -a.g[idx % a.H] * s;
  }
}

// one block per (sequence, head): dg partial and dIp partial
__global__ __launch_bounds__(256) void recurrent_bwd_seq_kernel(RecBwdArgs a) {
  __shared__ double sG[4];
  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  const int h = blockIdx.x % a.H, n = blockIdx.x / a.H;
  int64_t bos; int len, segbase;
  rec_seq(a, n, bos, len, segbase);
  double acc = 0.0;
  for (int t = tid; t < len; t += 256)
    acc -= (double)load_gate(a.gt, (bos + t) * a.H + h, a.gate_bf16) * (double)a.dl[(bos + t) * a.H + h];
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) acc += __shfl_xor(acc, off);
  if (lane == 0) sG[w] = acc;
  __syncthreads();
  if (tid == 0) {
    a.dgPart[(int64_t)n * a.H + h] = sG[0] + sG[1] + sG[2] + sG[3];
    double s = 0.0;
    for (int w2 = 0; w2 < a.ND; ++w2) {
      s += (double)a.pdIp[((int64_t)w2 * a.n_seqs + n) * a.H + h];
      if (a.init_mu) s -= (double)a.pInit[((int64_t)w2 * a.n_seqs + n) * a.H + h];
    }
    a.dIpPart[(int64_t)n * a.H + h] = s;
  }
}

__global__ void recurrent_bwd_head_kernel(RecBwdArgs a) {
  const int h = blockIdx.x * blockDim.x + threadIdx.x;
  if (h >= a.H) return;
  double sg = 0.0, si = 0.0;
  for (int n = 0; n < a.n_seqs; ++n) {
    sg += a.dgPart[(int64_t)n * a.H + h];
    si += a.dIpPart[(int64_t)n * a.H + h];
  }
  a.dg[h] = (float)sg;
  a.dIp[h] = (float)si;
}

// ------------------------------------------------------------------- host
struct RecBwdLayout {
  size_t oSeg, oCkM, oCkJ, oPdq, oPdk, oPdl, oDl, oPdIp, oPInit, oDg, oDIp, total;
  int S, ND;
  int64_t segments;
};

static size_t al256(size_t x) { return (x + 255) & ~(size_t)255; }

static RecBwdLayout rec_bwd_layout(const PalDims* d) {
  RecBwdLayout L;
  L.S = d->dk > 128 ? 8 : 16;
  L.ND = d->dv / 4;
  const size_t tokens = (size_t)d->batch * d->seq_len;
  const size_t E = (size_t)d->dv * d->dk;
  // upper bound on the number of segments: every sequence may end with a partial one
  L.segments = (int64_t)(tokens / L.S) + d->n_seqs;
  size_t o = 0;
  L.oSeg = o; o = al256(o + ((size_t)d->n_seqs + 1) * 4);
  L.oCkM = o; o = al256(o + (size_t)L.segments * d->n_heads * E * 4);
  L.oCkJ = o; o = al256(o + (size_t)L.segments * d->n_heads * E * 4);
  L.oPdq = o; o = al256(o + (size_t)L.ND * tokens * d->n_heads * d->dk * 4);
  L.oPdk = o; o = al256(o + (size_t)L.ND * tokens * d->n_heads * d->dk * 4);
  L.oPdl = o; o = al256(o + (size_t)L.ND * tokens * d->n_heads * 4);
  L.oDl = o; o = al256(o + tokens * d->n_heads * 4);
  L.oPdIp = o; o = al256(o + (size_t)L.ND * d->n_seqs * d->n_heads * 4);
  L.oPInit = o; o = al256(o + (size_t)L.ND * d->n_seqs * d->n_heads * 4);
  L.oDg = o; o = al256(o + (size_t)d->n_seqs * d->n_heads * 8);
  L.oDIp = o; o = al256(o + (size_t)d->n_seqs * d->n_heads * 8);
  L.total = o;
  return L;
}

template <typename TIn, int NPL>
static int launch_rec_bwd(const RecBwdArgs& a, hipStream_t s) {
  const int64_t blocks = (int64_t)a.n_seqs * a.H * a.ND;
  if (blocks > 0x7fffffff) return PAL_E_DIM;
  PAL_TIMED_LAUNCH(kKernRecurrentBwdFwdPass, s, (recurrent_bwd_state_kernel<TIn, NPL>), dim3((unsigned)blocks), dim3(64), 0, s, a);
  PAL_HIP_LAUNCH_CHECK();
  const size_t lds = (size_t)a.S * 2 * NPL * 64 * sizeof(float);
  if (a.flags & PAL_FLAG_HAS_VAR) {
    if (int rc = allow_lds((const void*)&recurrent_bwd_kernel<TIn, NPL, true>, lds)) return rc;
    PAL_TIMED_LAUNCH(kKernRecurrentBwd, s, (recurrent_bwd_kernel<TIn, NPL, true>), dim3((unsigned)blocks), dim3(64), lds, s, a);
  } else {
    if (int rc = allow_lds((const void*)&recurrent_bwd_kernel<TIn, NPL, false>, lds)) return rc;
    PAL_TIMED_LAUNCH(kKernRecurrentBwd, s, (recurrent_bwd_kernel<TIn, NPL, false>), dim3((unsigned)blocks), dim3(64), lds, s, a);
  }
  PAL_HIP_LAUNCH_CHECK();
  return PAL_OK;
}

template <typename TIn>
static int launch_rec_bwd_dtype(const RecBwdArgs& a, hipStream_t s) {
  switch (a.dk / 16) {
    case 1: return launch_rec_bwd<TIn, 1>(a, s);
    case 2: return launch_rec_bwd<TIn, 2>(a, s);
    case 3: return launch_rec_bwd<TIn, 3>(a, s);
    case 4: return launch_rec_bwd<TIn, 4>(a, s);
    case 6: return launch_rec_bwd<TIn, 6>(a, s);
    case 8: return launch_rec_bwd<TIn, 8>(a, s);
    case 12: return launch_rec_bwd<TIn, 12>(a, s);
    case 16: return launch_rec_bwd<TIn, 16>(a, s);
    default: return PAL_E_HEADDIM;
  }
}

}  // namespace pal

extern "C" size_t pal_recurrent_bwd_workspace_bytes(const PalDims* d) {
  if (pal_validate_dims(d) != PAL_OK || !pal::recurrent_dk_supported(d->dk)) return 0;
  return pal::rec_bwd_layout(d).total;
}

extern "C" int pal_recurrent_bwd(const PalDims* d, const PalFwdTensors* t, const PalBwdTensors* gr, void* workspace,
                                 size_t workspace_bytes, void* stream) {
  using namespace pal;
  if (!d || !t) return PAL_E_NULL;
  PalDims dd = *d;
  dd.flags &= ~PAL_FLAG_STORE_FINAL;
  PalFwdTensors tt = *t;
  tt.final_mu = tt.final_I = nullptr;
  if (!tt.o) tt.o = gr ? (void*)gr->d_o : nullptr;
  if ((dd.flags & PAL_FLAG_HAS_VAR) && !tt.o_var) tt.o_var = gr ? (void*)gr->d_o_var : nullptr;
  int rc = check_fwd_common(&dd, &tt);
  if (rc) return rc;
  if (!recurrent_dk_supported(dd.dk)) return PAL_E_HEADDIM;
  rc = check_bwd_common(&dd, gr);
  if (rc) return rc;
  const RecBwdLayout L = rec_bwd_layout(&dd);
  if (!workspace || workspace_bytes < L.total || !is_aligned16(workspace)) return PAL_E_WORKSPACE;
  RecBwdArgs a;
  a.q = tt.q; a.k = tt.k; a.v = tt.v; a.b = tt.b; a.gt = tt.gt;
  a.d_o = gr->d_o;
  a.d_o_var = (dd.flags & PAL_FLAG_HAS_VAR) ? gr->d_o_var : nullptr;
  a.g = tt.g; a.Ip = tt.Ip; a.init_mu = tt.init_mu; a.init_I = tt.init_I;
  a.cu_seqlens = tt.cu_seqlens;
  a.g_dq = gr->dq; a.g_dk = gr->dk; a.g_dv = gr->dv; a.g_db = gr->db;
  a.dgt = gr->dgt; a.dg = gr->dg; a.dIp = gr->dIp;
  a.d_init_mu = gr->d_init_mu; a.d_init_I = gr->d_init_I;
  char* ws = (char*)workspace;
  a.seg_off = (int32_t*)(ws + L.oSeg);
  a.ckM = (float*)(ws + L.oCkM); a.ckJ = (float*)(ws + L.oCkJ);
  a.pdq = (float*)(ws + L.oPdq); a.pdk = (float*)(ws + L.oPdk);
  a.pdl = (float*)(ws + L.oPdl); a.dl = (float*)(ws + L.oDl);
  a.pdIp = (float*)(ws + L.oPdIp); a.pInit = (float*)(ws + L.oPInit);
  a.dgPart = (double*)(ws + L.oDg); a.dIpPart = (double*)(ws + L.oDIp);
  a.T = dd.seq_len; a.H = dd.n_heads; a.dk = dd.dk; a.dv = dd.dv; a.n_seqs = dd.n_seqs;
  a.Hq = dd.n_qk_heads > 0 ? dd.n_qk_heads : dd.n_heads;
  a.S = L.S; a.tokens = dd.batch * dd.seq_len; a.ND = L.ND;
  a.seg_cap = (int32_t)(L.segments > 0x7fffffff ? 0x7fffffff : L.segments);
  a.gate_bf16 = dd.gate_dtype == PAL_DTYPE_BF16;
  a.var_bf16 = dd.var_dtype == PAL_DTYPE_BF16;
  a.out_bf16 = dd.dtype == PAL_DTYPE_BF16;
  a.flags = dd.flags;
  a.scale = dd.scale;
  hipStream_t s = (hipStream_t)stream;
  if (a.cu_seqlens) {
    hipLaunchKernelGGL(recurrent_bwd_segoff_kernel, dim3(1), dim3(64), 0, s, a);
    PAL_HIP_LAUNCH_CHECK();
  }
  rc = a.out_bf16 ? launch_rec_bwd_dtype<bf16_t>(a, s) : launch_rec_bwd_dtype<float>(a, s);
  if (rc) return rc;
  {
    const int64_t n = (int64_t)a.tokens * a.H * a.dk;
    hipLaunchKernelGGL(recurrent_bwd_reduce_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, a);
    PAL_HIP_LAUNCH_CHECK();
  }
  hipLaunchKernelGGL(recurrent_bwd_seq_kernel, dim3((unsigned)(a.n_seqs * a.H)), dim3(256), 0, s, a);
  PAL_HIP_LAUNCH_CHECK();
  hipLaunchKernelGGL(recurrent_bwd_head_kernel, dim3((a.H + 63) / 64), dim3(64), 0, s, a);
  PAL_HIP_LAUNCH_CHECK();
  return PAL_OK;
}
