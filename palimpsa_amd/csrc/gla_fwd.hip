// Chunked forward of scalar-gated linear attention: the Palimpsa recurrence without its precision
// state (b = 0, I = 1, so mu = M),
//     S_t = f_t S_{t-1} + v_t k_t^T ,   o_t = scale * S_t q_t ,   f_t = exp(-gt_t * g) .
// It is what the reference layer runs when metaplasticity is off (the simple_gla pair imported at
// palimpsa/layers/palimpsa.py:18 and called at :293-300).  Without the division by I_t the output of
// a tile is two plain matrix products,
//     O = ((Q K^T) o L) V + diag(F) Q S_0^T ,      L[t,s] = 2^{c_t - c_s} (s <= t),  F_t = 2^{c_t},
// so nothing of the [tokens x dv x dk] state has to be materialised per token: the tile-start states
// come from the same two kernels as in the Palimpsa forward (local contribution + serial scan, both
// without the J branch) and the kernel below does the rest on the matrix cores.
#include "chunk_common.h"
#include "pal_host.h"
#include "pal_profile.h"

namespace pal {

void fill_chunk_args(ChunkArgs& a, const PalDims* d, const PalFwdTensors* t);
int launch_tile_states(const ChunkArgs& a, int dtype, bool has_j, hipStream_t s);

constexpr int kVT = 72;  // row stride (bf16) of the transposed value tile

template <typename TIn>
__device__ __forceinline__ bf16x8 load_bf16x8(const TIn* p) {
  if constexpr (sizeof(TIn) == 2) {
    return *(const bf16x8*)p;
  } else {
    const f32x4 x = *(const f32x4*)p, y = *(const f32x4*)(p + 4);
    bf16x8 r;
#pragma unroll
    for (int e = 0; e < 4; ++e) { r[e] = (bf16_t)x[e]; r[4 + e] = (bf16_t)y[e]; }
    return r;
  }
}

// One workgroup of 4 waves per (tile, head); wave w owns the query tokens [16w, 16w+16).
//   P^T[s,t] = sum_n K[s,n] Q[t,n]            A = K rows (LDS), B = the wave's Q rows (registers); key blocks <= w only
//   P^T     *= L[t,s]                          in the accumulator layout (column t per lane, 4 rows s)
//   O^T[d,t] = F_t sum_n S_0[d,n] Q[t,n]       A = tile-start state rows (global fp32 -> bf16)
//            + sum_s V^T[d,s] P^T[s,t]         A = V^T rows (LDS), B = P^T straight from the accumulators:
// the contraction index of that last product is mapped to tokens as slot (g, j) -> s = 32p + 16(j/4) +
// 4g + j%4, which is where the accumulators of two neighbouring key blocks already sit, and V^T is read
// with the same map (two 8-byte LDS reads per operand).
// KS = ceil(dk / 32) contraction steps over the key dimension (operands zero padded to 32 KS).
template <typename TIn, int KS>
__global__ __launch_bounds__(256) void gla_out_kernel(ChunkArgs a) {
  extern __shared__ float smem[];
  const int H = a.H, dk = a.dk, dv = a.dv;
  constexpr int dkp = 32 * KS + 8;    // row stride (bf16) of the K tile
  float* sC = smem;                   // [64] running log2 decay inside the tile
  bf16_t* sK = (bf16_t*)(sC + kC);    // [64][dkp]
  bf16_t* sVT = sK + kC * dkp;        // [dv][kVT]
  const int tid = threadIdx.x, lane = tid & 63, i = lane & 15, g = lane >> 4;
  const int tb = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int cidx = blockIdx.x / H, h = blockIdx.x % H;
  int seq, t0, clen, cis;
  chunk_lookup(a, cidx, seq, t0, clen, cis);
  if (tb == 0) {
    const float gh = a.g[h] * kLog2e;
    const float gt = (lane < clen) ? load_gate(a.gt, (int64_t)(t0 + lane) * H + h, a.gate_bf16) : 0.f;
    sC[lane] = wave_inclusive_scan(-gt * gh, lane);
  }
  // the wave's 16 query rows as B operands (column t = 16 tb + i, contraction index n = 32 ks + 8 g + j)
  const int t = 16 * tb + i;
  bf16x8 Q[KS];
  {
    const TIn* qp = (const TIn*)a.q + ((int64_t)(t0 + t) * H + h) * dk + 8 * g;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      Q[ks] = bf16x8{0, 0, 0, 0, 0, 0, 0, 0};
      if (t < clen && 32 * ks + 8 * g < dk) Q[ks] = load_bf16x8(qp + 32 * ks);
    }
  }
  {
    // K rows, zero beyond the tile's tokens and beyond dk
    const TIn* kp = (const TIn*)a.k + ((int64_t)t0 * H + h) * dk;
    constexpr int groups = 4 * KS;
    for (int idx = tid; idx < kC * groups; idx += 256) {
      const int s = idx / groups, c8 = idx - s * groups;
      bf16x8 kx = {0, 0, 0, 0, 0, 0, 0, 0};
      if (s < clen && 8 * c8 < dk) kx = load_bf16x8(kp + (int64_t)s * H * dk + 8 * c8);
      *(bf16x8*)&sK[s * dkp + 8 * c8] = kx;
    }
    // V transposed (token index fastest), zero beyond the tile's tokens.  A work item is two consecutive
    // tokens by eight value columns: neighbouring lanes read neighbouring 16-byte pieces of a row, and a
    // pair of tokens goes to LDS as one 32-bit word per value column.
    const TIn* vp = (const TIn*)a.v + ((int64_t)t0 * H + h) * dv;
    const int vgroups = dv >> 3;
    for (int idx = tid; idx < (kC / 2) * vgroups; idx += 256) {
      const int sp = idx / vgroups, c8 = idx - sp * vgroups;
      bf16x8 v0 = {0, 0, 0, 0, 0, 0, 0, 0}, v1 = {0, 0, 0, 0, 0, 0, 0, 0};
      if (2 * sp < clen) v0 = load_bf16x8(vp + (int64_t)(2 * sp) * H * dv + 8 * c8);
      if (2 * sp + 1 < clen) v1 = load_bf16x8(vp + (int64_t)(2 * sp + 1) * H * dv + 8 * c8);
#pragma unroll
      for (int e = 0; e < 8; ++e) *(bf16x2*)&sVT[(8 * c8 + e) * kVT + 2 * sp] = bf16x2{v0[e], v1[e]};
    }
  }
  __syncthreads();

  const float ct = sC[16 * tb + i];
  const float Ft = fast_exp2(ct);

  // decayed, causally masked scores of the wave's 16 queries against key blocks 0..tb, as B operands
  bf16x8 P[2];
#pragma unroll
  for (int p = 0; p < 2; ++p) {
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      const int sb = 2 * p + half;
      f32x4 acc = {0.f, 0.f, 0.f, 0.f};
      if (sb <= tb) {
        const bf16_t* krow = sK + (16 * sb + i) * dkp + 8 * g;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) acc = mfma16(*(const bf16x8*)(krow + 32 * ks), Q[ks], acc);
        const f32x4 cs = *(const f32x4*)&sC[16 * sb + 4 * g];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const bool live = sb < tb || 4 * g + r <= i;
          acc[r] = live ? acc[r] * fast_exp2(ct - cs[r]) : 0.f;
        }
      }
#pragma unroll
      for (int r = 0; r < 4; ++r) P[p][4 * half + r] = (bf16_t)acc[r];
    }
  }

  const float scale = a.scale;
  const float* S0 = a.chunk_mu + ((int64_t)cidx * H + h) * dv * dk;
  TIn* orow = (TIn*)a.o + ((int64_t)(t0 + t) * H + h) * dv + 4 * g;
  const int n_db = dv >> 4;
  // four blocks of 16 value rows at a time, so that the loads of the tile-start state are in flight together
  for (int db0 = 0; db0 < n_db; db0 += 4) {
    f32x4 acc[4];
    const float* srow[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      acc[u] = f32x4{0.f, 0.f, 0.f, 0.f};
      srow[u] = S0 + (int64_t)(16 * min(db0 + u, n_db - 1) + i) * dk + 8 * g;   // a block past the end repeats the last one
    }
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const bf16x8 B = Q[ks];
      bf16x8 A[4];
      const bool ok = 32 * ks + 8 * g < dk;
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        A[u] = bf16x8{0, 0, 0, 0, 0, 0, 0, 0};
        if (ok) A[u] = load_bf16x8(srow[u] + 32 * ks);
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) acc[u] = mfma16(A[u], B, acc[u]);
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int db = min(db0 + u, n_db - 1);
#pragma unroll
      for (int r = 0; r < 4; ++r) acc[u][r] *= Ft;
      const bf16_t* vrow = sVT + (16 * db + i) * kVT + 4 * g;
#pragma unroll
      for (int p = 0; p < 2; ++p) {
        if (2 * p <= tb) {
          const bf16x4 lo = *(const bf16x4*)(vrow + 32 * p), hi = *(const bf16x4*)(vrow + 32 * p + 16);
          const bf16x8 A = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
          acc[u] = mfma16(A, P[p], acc[u]);
        }
      }
      if (t < clen && db0 + u < n_db) {
        const float out[4] = {acc[u][0] * scale, acc[u][1] * scale, acc[u][2] * scale, acc[u][3] * scale};
        store_vec<4>(orow + 16 * db, out);
      }
    }
  }
}

template <typename TIn, int KS>
static int launch_gla_out_ks(const ChunkArgs& a, hipStream_t s) {
  const size_t lds = sizeof(float) * kC + sizeof(bf16_t) * ((size_t)kC * (32 * KS + 8) + (size_t)a.dv * kVT);
  const int64_t blocks = (int64_t)a.total_chunks * a.H;
  if (blocks > 0x7fffffff) return PAL_E_DIM;
  if (lds > kMaxLds) return PAL_E_HEADDIM;
  if (int rc = allow_lds((const void*)&gla_out_kernel<TIn, KS>, lds)) return rc;
  PAL_TIMED_LAUNCH(kKernGlaOut, s, (gla_out_kernel<TIn, KS>), dim3((unsigned)blocks), dim3(256), lds, s, a);
  PAL_HIP_LAUNCH_CHECK();
  return PAL_OK;
}

template <typename TIn>
static int launch_gla_out(const ChunkArgs& a, hipStream_t s) {
  switch ((a.dk + 31) / 32) {
    case 1: return launch_gla_out_ks<TIn, 1>(a, s);
    case 2: return launch_gla_out_ks<TIn, 2>(a, s);
    case 3: return launch_gla_out_ks<TIn, 3>(a, s);
    case 4: return launch_gla_out_ks<TIn, 4>(a, s);
    case 5: return launch_gla_out_ks<TIn, 5>(a, s);
    case 6: return launch_gla_out_ks<TIn, 6>(a, s);
    case 7: return launch_gla_out_ks<TIn, 7>(a, s);
    case 8: return launch_gla_out_ks<TIn, 8>(a, s);
    default: return PAL_E_HEADDIM;
  }
}

}  // namespace pal

extern "C" int pal_gla_chunk_fwd(const PalDims* d, const PalFwdTensors* t, void* stream) {
  using namespace pal;
  int rc = pal_validate_dims(d);
  if (rc) return rc;
  if (!t) return PAL_E_NULL;
  if (!t->q || !t->k || !t->v || !t->gt || !t->g || !t->o || !t->chunk_mu) return PAL_E_NULL;
  if (d->flags & PAL_FLAG_HAS_VAR) return PAL_E_STATE;   // no precision state, no output variance
  if (((d->flags & PAL_FLAG_HAS_INIT) != 0) != (t->init_mu != nullptr)) return PAL_E_STATE;
  if (((d->flags & PAL_FLAG_STORE_FINAL) != 0) != (t->final_mu != nullptr)) return PAL_E_STATE;
  const bool varlen = d->flags & PAL_FLAG_VARLEN;
  if (varlen != (t->cu_seqlens != nullptr)) return PAL_E_CU_SEQLENS;
  if (varlen && (!t->chunk_table || !t->chunk_offsets)) return PAL_E_NULL;
  if (d->total_chunks <= 0) return PAL_E_CHUNK;
  {
    const int64_t per = ((int64_t)d->seq_len + PAL_CHUNK - 1) / PAL_CHUNK;
    if (varlen) {
      if (d->total_chunks < per || d->total_chunks > (int64_t)d->seq_len / PAL_CHUNK + d->n_seqs) return PAL_E_CHUNK;
    } else if ((int64_t)d->total_chunks != per * d->batch) {
      return PAL_E_CHUNK;
    }
  }
  const void* ptrs[] = {t->q, t->k, t->v, t->o, t->init_mu, t->final_mu, t->chunk_mu};
  for (const void* p : ptrs)
    if (p && !is_aligned16(p)) return PAL_E_ALIGN;
  // the shared argument block carries no precision tensors on this path
  PalFwdTensors tt = *t;
  tt.b = nullptr; tt.Ip = nullptr; tt.o_var = nullptr;
  tt.init_I = nullptr; tt.final_I = nullptr; tt.chunk_I = nullptr;
  ChunkArgs a;
  fill_chunk_args(a, d, &tt);
  hipStream_t s = (hipStream_t)stream;
  if (int rc2 = launch_tile_states(a, d->dtype, false, s)) return rc2;
  if (d->dtype == PAL_DTYPE_BF16) return launch_gla_out<bf16_t>(a, s);
  return launch_gla_out<float>(a, s);
}
