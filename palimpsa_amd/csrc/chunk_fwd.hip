// Chunked Palimpsa forward: three kernels.
//
//  (1) chunk_delta_kernel + chunk_scan_kernel — the state at the START of every
//      tile.  The first computes every tile's own contribution
//        Delta = (a o V)^T K                 (a_s = decay from token s to tile end)
//      with bf16 MFMA contractions, all tiles in parallel; the second runs the
//      recurrence S_c = F_C S_{c-1} + Delta_c over the tiles of a sequence as an
//      fp32 streaming scan (the only serial part of the forward) and leaves the
//      tile-start states and the final state in (mu, I) form.
//  (2) chunk_out_kernel — one workgroup per (tile, head), all tiles in
//      parallel.  Wave w owns key columns [16w, 16w+16).  For every value row d
//      it builds the operand X^T[n,s] = k_s[n] v_s[d] (and k_s[n]^2 b_s[d]),
//      multiplies by the decay matrix L^T on the matrix cores and finishes
//      M_t, I_t, 1/I_t, mu_t q_t in registers (the scan + division + output of
//      the reference kernel, :190-207).  Output orientation is [n, t] so the
//      sum over n stays inside a lane.
#include <atomic>
#include <type_traits>

#include "chunk_common.h"
#include "pal_host.h"
#include "pal_profile.h"

namespace pal {

// ------------------------------------------------------------------ kernel 1a
// Local contribution of one tile to the state: Delta = (a o V)^T K, with a_s the decay from token s
// to the end of the tile.  One workgroup of 4 waves per (tile, head), all tiles in parallel: the
// K, V, B rows of the tile are staged once through LDS (16-byte loads, stored transposed so that an
// MFMA operand is one contiguous run of tokens), then wave w produces the 16x16 blocks of the state
// whose key columns are [16w, 16w+16) (+64, ...).  The result is parked in the tile's slot of
// chunk_mu / chunk_I until the scan below replaces it.
// Row stride (elements) of the transposed staging tiles.  bf16 rows are staged as they are; fp32 rows in fp32
// tiles while those fit in LDS, else rounded to bf16 (the operands built from them are bf16 anyway).
template <typename TS>
struct StageStride { static constexpr int value = sizeof(TS) == 4 ? 68 : 72; };

template <typename TIn, typename TS>
__device__ __forceinline__ void stage_transposed(const TIn* src, int64_t row_stride, int width, int clen, TS* dst,
                                                 int tid) {
  // src: [64 tokens][width] rows -> dst[width][stride] (token index fastest), rows >= clen are zero
  constexpr int kTS = StageStride<TS>::value;
  const int groups = width >> 3;
  if constexpr (sizeof(TS) == 2) {
    // bf16 tiles: a work item is two consecutive tokens by eight columns, so that neighbouring lanes read
    // neighbouring 16-byte pieces of a row and a pair of tokens goes to LDS as one 32-bit word per column
    for (int idx = tid; idx < (kC / 2) * groups; idx += 256) {
      const int sp = idx / groups, c8 = idx - sp * groups;
      float x0[8], x1[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) { x0[e] = 0.f; x1[e] = 0.f; }
      if (2 * sp < clen) {
        load_vec<4>(src + (int64_t)(2 * sp) * row_stride + 8 * c8, x0);
        load_vec<4>(src + (int64_t)(2 * sp) * row_stride + 8 * c8 + 4, x0 + 4);
      }
      if (2 * sp + 1 < clen) {
        load_vec<4>(src + (int64_t)(2 * sp + 1) * row_stride + 8 * c8, x1);
        load_vec<4>(src + (int64_t)(2 * sp + 1) * row_stride + 8 * c8 + 4, x1 + 4);
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) *(bf16x2*)&dst[(8 * c8 + e) * kTS + 2 * sp] = pack2(x0[e], x1[e]);
    }
  } else {
    for (int idx = tid; idx < kC * groups; idx += 256) {
      const int s = idx & (kC - 1), c8 = idx >> 6;
      float x[8];
      if (s < clen) {
        load_vec<4>(src + (int64_t)s * row_stride + 8 * c8, x);
        load_vec<4>(src + (int64_t)s * row_stride + 8 * c8 + 4, x + 4);
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) x[e] = 0.f;
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) dst[(8 * c8 + e) * kTS + s] = x[e];
    }
  }
}

// eight consecutive staged elements (16-byte aligned) as fp32
__device__ __forceinline__ void staged8(const float* p, float* out) {
  *(f32x4*)&out[0] = *(const f32x4*)p;
  *(f32x4*)&out[4] = *(const f32x4*)(p + 4);
}
__device__ __forceinline__ void staged8(const bf16_t* p, float* out) {
  const bf16x8 x = *(const bf16x8*)p;
#pragma unroll
  for (int e = 0; e < 8; ++e) out[e] = (float)x[e];
}

// HAS_J = false drops the precision branch (b is not read, chunk_I is not written): the scalar-gated linear
// attention that the layer uses without its precision state.
// PREC (fp32 rows staged in fp32): operands split into two bf16 halves, three matrix instructions per product.
template <typename TIn, bool HAS_J, typename TS, bool PREC>
__global__ __launch_bounds__(256) void chunk_delta_kernel(ChunkArgs a, int dvn) {
  // blockIdx.y selects a piece of dvn value rows (dvn = dv: one piece; smaller where the staging tiles of all rows
  // would not fit the LDS)
  extern __shared__ float smem[];
  constexpr int kTS = StageStride<TS>::value;
  const int H = a.H, dk = a.dk, dv = a.dv;
  const int d0 = blockIdx.y * dvn, dn = min(dvn, dv - d0);
  float* sA = smem;                 // [64] decay from token s to the end of the tile
  TS* sKT = (TS*)(sA + kC);         // [dk][kTS]
  TS* sVT = sKT + dk * kTS;         // [dvn][kTS]
  TS* sBT = sVT + dvn * kTS;        // [dvn][kTS]
  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6, i = lane & 15, g = lane >> 4;
  const int NB = dk >> 4, ND = dn >> 4;
  const int cidx = blockIdx.x / H, h = blockIdx.x % H;
  int seq, t0, clen, cis;
  chunk_lookup(a, cidx, seq, t0, clen, cis);
  if (w == 0) {
    const float gh = a.g[h] * kLog2e;
    const float gt = (lane < clen) ? load_gate(a.gt, (int64_t)(t0 + lane) * H + h, a.gate_bf16) : 0.f;
    const float cs = wave_inclusive_scan(-gt * gh, lane);
    sA[lane] = fast_exp2((a.flags & kFlagDecayFromStart) ? cs : __shfl(cs, 63) - cs);
  }
  stage_transposed((const TIn*)a.k + qk_row(a, t0, h), qk_stride(a), dk, clen, sKT, tid);
  stage_transposed((const TIn*)a.v + ((int64_t)t0 * H + h) * dv + d0, (int64_t)H * dv, dn, clen, sVT, tid);
  if (HAS_J) stage_transposed((const TIn*)a.b + ((int64_t)t0 * H + h) * dv + d0, (int64_t)H * dv, dn, clen, sBT, tid);
  __syncthreads();
  float as[2][8];
#pragma unroll
  for (int ks = 0; ks < 2; ++ks) staged8(&sA[8 * g + 32 * ks], as[ks]);
  for (int nb = w; nb < NB; nb += 4) {
    bf16x8 BK[2], BKK[2], BKl[2], BKKl[2];   // the *l halves only exist with PREC
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      float kv[8];
      staged8(&sKT[(16 * nb + i) * kTS + 8 * g + 32 * ks], kv);
      if constexpr (PREC) {
        float kq[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) kq[j] = kv[j] * kv[j];
        split_bf16(kv, BK[ks], BKl[ks]);
        split_bf16(kq, BKK[ks], BKKl[ks]);
      } else {
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          BK[ks][j] = (bf16_t)kv[j];
          BKK[ks][j] = (bf16_t)(kv[j] * kv[j]);
        }
      }
    }
    for (int dt = 0; dt < ND; ++dt) {
      bf16x8 AM[2], AJ[2], AMl[2], AJl[2];
#pragma unroll
      for (int ks = 0; ks < 2; ++ks) {
        float vv[8], bb[8];
        staged8(&sVT[(16 * dt + i) * kTS + 8 * g + 32 * ks], vv);
        if (HAS_J) staged8(&sBT[(16 * dt + i) * kTS + 8 * g + 32 * ks], bb);
        if constexpr (PREC) {
#pragma unroll
          for (int j = 0; j < 8; ++j) { vv[j] *= as[ks][j]; if (HAS_J) bb[j] *= as[ks][j]; }
          split_bf16(vv, AM[ks], AMl[ks]);
          if (HAS_J) split_bf16(bb, AJ[ks], AJl[ks]);
        } else {
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            AM[ks][j] = (bf16_t)(as[ks][j] * vv[j]);
            if (HAS_J) AJ[ks][j] = (bf16_t)(as[ks][j] * bb[j]);
          }
        }
      }
      // the products are taken transposed (K as the row operand) so that a lane ends up with four consecutive
      // key columns of one value row: rows n = 16nb + 4g + r, column d = 16dt + i, one 16-byte store per lane
      f32x4 M = {0.f, 0.f, 0.f, 0.f}, J = {0.f, 0.f, 0.f, 0.f};
      if constexpr (PREC) {
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
          M = mfma16_split(BK[ks], BKl[ks], AM[ks], AMl[ks], M);
          if (HAS_J) J = mfma16_split(BKK[ks], BKKl[ks], AJ[ks], AJl[ks], J);
        }
      } else {
      M = mfma16(BK[0], AM[0], M);
      if (HAS_J) J = mfma16(BKK[0], AJ[0], J);
      M = mfma16(BK[1], AM[1], M);
      if (HAS_J) J = mfma16(BKK[1], AJ[1], J);
      }
      const int64_t co = (((int64_t)cidx * H + h) * dv + d0 + 16 * dt + i) * dk + 16 * nb + 4 * g;
      *(f32x4*)&a.chunk_mu[co] = M;
      if (HAS_J) *(f32x4*)&a.chunk_I[co] = J;
    }
  }
}

// ------------------------------------------------------------------ kernel 1b
// Serial part of the forward: S_c = F_c S_{c-1} + Delta_c per state entry, fp32, pure streaming.
// One thread per four consecutive state entries of a (sequence, head), 1024 entries per block.  Each slot of
// chunk_mu / chunk_I is overwritten with the state at the START of its tile in (mu, I) form
// (what the reference stores as intermediate_*_state, chunk_palimpsa_forgetting_scalar.py:187-188);
// the state after the last tile goes to final_mu / final_I (:214-218).
__global__ __launch_bounds__(256) void chunk_scan_kernel(ChunkArgs a) {
  __shared__ float sF[kScanTiles];
  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  const int64_t E = (int64_t)a.dv * a.dk;
  const int nblk = (int)((E + 1023) / 1024);     // four consecutive entries per thread
  const int blk = blockIdx.x % nblk;
  const int nh = blockIdx.x / nblk;
  const int h = nh % a.H, n = nh / a.H;
  const int64_t e = ((int64_t)blk * 256 + tid) * 4;
  const bool on = e < E;
  int bos, len, cbase;
  seq_lookup(a, n, bos, len, cbase);
  const int nchunks = (len + kC - 1) / kC;
  const float Ip = a.Ip[h];
  const float gh = a.g[h] * kLog2e;
  f32x4 SM = {0.f, 0.f, 0.f, 0.f}, SJ = {0.f, 0.f, 0.f, 0.f};
  const int64_t so = (int64_t)nh * E + e;
  if (a.init_mu && on) {
    const f32x4 mu = *(const f32x4*)(a.init_mu + so), I = *(const f32x4*)(a.init_I + so);
#pragma unroll
    for (int x = 0; x < 4; ++x) { SM[x] = mu[x] * I[x]; SJ[x] = I[x] - Ip; }
  }
  // the slot of a tile: its Delta is read, the state at its start (mu, I) written, the state advanced
  auto advance = [&](int64_t off, const f32x4& dM, const f32x4& dJ, float F) {
    f32x4 mu, I;
#pragma unroll
    for (int x = 0; x < 4; ++x) {
      I[x] = SJ[x] + Ip;
      mu[x] = SM[x] * fast_rcp(I[x]);
      SM[x] = fmaf(F, SM[x], dM[x]);
      SJ[x] = fmaf(F, SJ[x], dJ[x]);
    }
    *(f32x4*)(a.chunk_mu + off) = mu;
    *(f32x4*)(a.chunk_I + off) = I;
  };
  for (int c0 = 0; c0 < nchunks; c0 += kScanTiles) {
    const int cn = min(kScanTiles, nchunks - c0);
    __syncthreads();
    for (int c = w; c < cn; c += 4) {
      const int t = (c0 + c) * kC + lane;
      const float gt = (t < len) ? load_gate(a.gt, (int64_t)(bos + t) * a.H + h, a.gate_bf16) : 0.f;
      const float tot = wave_sum(-gt * gh);
      if (lane == 0) sF[c] = fast_exp2(tot);
    }
    __syncthreads();
    if (!on) continue;
    int c = 0;
    for (; c + 4 <= cn; c += 4) {
      f32x4 dM[4], dJ[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int64_t off = ((int64_t)(cbase + c0 + c + u) * a.H + h) * E + e;
        dM[u] = *(const f32x4*)(a.chunk_mu + off);
        dJ[u] = *(const f32x4*)(a.chunk_I + off);
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) advance(((int64_t)(cbase + c0 + c + u) * a.H + h) * E + e, dM[u], dJ[u], sF[c + u]);
    }
    for (; c < cn; ++c) {
      const int64_t off = ((int64_t)(cbase + c0 + c) * a.H + h) * E + e;
      const f32x4 dM = *(const f32x4*)(a.chunk_mu + off), dJ = *(const f32x4*)(a.chunk_I + off);
      advance(off, dM, dJ, sF[c]);
    }
  }
  if (a.final_mu && on) {
    f32x4 mu, I;
#pragma unroll
    for (int x = 0; x < 4; ++x) { I[x] = SJ[x] + Ip; mu[x] = SM[x] * fast_rcp(I[x]); }
    *(f32x4*)(a.final_mu + so) = mu;
    *(f32x4*)(a.final_I + so) = I;
  }
}

// The same scan without the precision state: S_c = F_c S_{c-1} + Delta_c with Delta_c read from chunk_mu (fp32).
// The state at the start of every tile is written in bf16 (what its readers feed to the matrix cores) to the
// buffer handed over in the chunk_I slot; the running state stays fp32 and its last value goes to final_mu.
__global__ __launch_bounds__(256) void gla_scan_kernel(ChunkArgs a) {
  bf16_t* tile_S = (bf16_t*)a.chunk_I;
  __shared__ float sF[kScanTiles];
  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  const int64_t E = (int64_t)a.dv * a.dk;
  const int nblk = (int)((E + 1023) / 1024);     // four consecutive entries per thread
  const int blk = blockIdx.x % nblk;
  const int nh = blockIdx.x / nblk;
  const int h = nh % a.H, n = nh / a.H;
  const int64_t e = ((int64_t)blk * 256 + tid) * 4;
  const bool on = e < E;
  int bos, len, cbase;
  seq_lookup(a, n, bos, len, cbase);
  const int nchunks = (len + kC - 1) / kC;
  const float gh = a.g[h] * kLog2e;
  const int64_t so = (int64_t)nh * E + e;
  f32x4 S = {0.f, 0.f, 0.f, 0.f};
  if (a.init_mu && on) S = *(const f32x4*)(a.init_mu + so);
  for (int c0 = 0; c0 < nchunks; c0 += kScanTiles) {
    const int cn = min(kScanTiles, nchunks - c0);
    __syncthreads();
    for (int c = w; c < cn; c += 4) {
      const int t = (c0 + c) * kC + lane;
      const float gt = (t < len) ? load_gate(a.gt, (int64_t)(bos + t) * a.H + h, a.gate_bf16) : 0.f;
      const float tot = wave_sum(-gt * gh);
      if (lane == 0) sF[c] = fast_exp2(tot);
    }
    __syncthreads();
    if (!on) continue;
    int c = 0;
    for (; c + 4 <= cn; c += 4) {
      f32x4 dS[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) dS[u] = *(const f32x4*)(a.chunk_mu + ((int64_t)(cbase + c0 + c + u) * a.H + h) * E + e);
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        store_vec<4>(tile_S + ((int64_t)(cbase + c0 + c + u) * a.H + h) * E + e, (const float*)&S);
        const float F = sF[c + u];
#pragma unroll
        for (int x = 0; x < 4; ++x) S[x] = fmaf(F, S[x], dS[u][x]);
      }
    }
    for (; c < cn; ++c) {
      const int64_t off = ((int64_t)(cbase + c0 + c) * a.H + h) * E + e;
      const f32x4 dS = *(const f32x4*)(a.chunk_mu + off);
      store_vec<4>(tile_S + off, (const float*)&S);
      const float F = sF[c];
#pragma unroll
      for (int x = 0; x < 4; ++x) S[x] = fmaf(F, S[x], dS[x]);
    }
  }
  if (a.final_mu && on) *(f32x4*)(a.final_mu + so) = S;
}

// ------------------------------------------------------------------ kernel 2
constexpr int kVH = 72;  // row stride (f16) of the transposed, block-scaled v/b staging tiles of chunk_out_kernel
constexpr int kDG = 16;  // value rows per staging group

// Adds the tile-start state (already under the block exponents; zero in the lanes that do not hold token 0) to the
// first element of the operands of tokens 0..7: the first pair becomes a packed multiply-add instead of a multiply.
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ void fold_state_pairs(f16x8& XM, f16x8& XJ, f16x8 kA, f16x8 vv, f16x8 kk, f16x8 bb, f16x2 am,
                                                 f16x2 aj) {
  const f16x2 xm = __builtin_elementwise_fma(kA.xy, vv.xy, am), xj = __builtin_elementwise_fma(kk.xy, bb.xy, aj);
  XM[0] = xm[0]; XM[1] = xm[1];
  XJ[0] = xj[0]; XJ[1] = xj[1];
}
__device__ __forceinline__ void fold_state(f16x8& XM, f16x8& XJ, f16x8 kA, f16x8 vv, f16x8 kk, f16x8 bb, float m0, float i0) {
  const f16x2 am = {(f16_t)m0, (f16_t)0.f}, aj = {(f16_t)i0, (f16_t)0.f};
  fold_state_pairs(XM, XJ, kA, vv, kk, bb, am, aj);
}
// chunk_out_kernel keeps the workgroup's tile-start state in LDS (f16) where it is small: at most four column blocks
// (and, at run time, at most 64 value rows); floats of LDS that takes per (tile, head)
__host__ __device__ constexpr bool out_state_cache(int NB, bool prec) { return !prec && NB <= 4; }
__host__ __device__ constexpr int out_state_cache_floats(int NB, bool prec) {
  return out_state_cache(NB, prec) ? (2 * 64 * 16 * NB * 2) / 4 + 4 : 0;
}

// index of the L operand for (tb, ks): tb0,tb1 -> one K step; tb2,tb3 -> two
__device__ __forceinline__ constexpr int lidx(int tb, int ks) { return tb < 2 ? tb : 2 + 2 * (tb - 2) + ks; }

// RS > 1 splits the value rows of a group among RS waves per column block (wave = (column block, rows dd = rs mod RS)).
// The hardware puts wave i of a workgroup on SIMD i mod 4, so a workgroup of 5, 6 or 7 waves loads the SIMDs 2:1:1:1 or
// 2:2:1:1 and this kernel, which is bound by vector issue, then runs at the pace of the busiest SIMD (measured: the same
// time for 5, 6, 7 and 8 column blocks).  With two waves per column block the waves spread evenly.
// TS > 1 gives a workgroup TS (tile, head) pairs, each with its own NB * RS waves and its own piece of LDS (they only
// share the barriers), so that a workgroup of two waves becomes one of four and covers all four SIMDs.
// PREC (fp32 rows): the rows are staged in fp32, the operands X and L are formed in fp32 and split into two bf16
// halves each, three matrix instructions per product (no block exponents: bf16 has the range of fp32).
// (the second launch bound caps the register budget at 256 per lane: the matrix results then stay in ordinary vector
// registers instead of being copied out of accumulation registers, 32 copies per value row in this kernel)
template <typename TIn, int NB, bool HAS_VAR, int RS, int TS, bool PREC>
__global__ __launch_bounds__(NB * RS * TS * 64, 2) void chunk_out_kernel(ChunkArgs a) {
  extern __shared__ float smem[];
  using TSt = std::conditional_t<PREC, float, f16_t>;   // element type of the staged v, b rows
  constexpr int NT = NB * RS * 64;        // threads per (tile, head)
  // CACHE (f16 operands, at most four column blocks, at most 64 value rows): the workgroup's tile-start state is read
  // once, for the maxima that the block exponents need, and then kept in LDS as the f16 numbers that the first
  // token's operands take (M_0 f_0 2^-(ek+ev), I_0 f_0 2^-(2ek+eb)), followed by a zero word for the lanes that add nothing
  constexpr bool CACHE = out_state_cache(NB, PREC);
  constexpr int kCacheFloats = out_state_cache_floats(NB, PREC);
  constexpr int kTileFloats = kC + (HAS_VAR ? 2 : 1) * NB * kDG * kC + (4 * kDG * kVH * (int)sizeof(TSt)) / 4 + kCacheFloats;
  const int sub = TS == 1 ? 0 : (int)threadIdx.x / NT;
  const int tid = (int)threadIdx.x - sub * NT;
  const int64_t n_items = (int64_t)a.total_chunks * a.H;
  const int64_t item_raw = (int64_t)blockIdx.x * TS + sub;
  const bool valid = item_raw < n_items;          // a spare group of the last workgroup repeats the last item, unstored
  const int64_t item = valid ? item_raw : n_items - 1;
  float* sC = smem + sub * kTileFloats;   // [64] running log2-decay inside the tile
  TSt* sV = (TSt*)(sC + kC);              // [2][16][kVH] v^T 2^-E of the current and the next value-row group
  TSt* sB = sV + 2 * kDG * kVH;           // [2][16][kVH] b^T 2^-E
  float* sO = (float*)(sB + 2 * kDG * kVH);   // [NB][16][64] per-wave partial outputs
  float* sOv = sO + NB * kDG * kC;        // same for o_var
  f16_t* sStM = (f16_t*)(sC + (kTileFloats - kCacheFloats));   // [dv <= 64][dk] CACHE: see above
  f16_t* sStI = sStM + 64 * 16 * NB;
  f16_t* sZero = sStI + 64 * 16 * NB;
  const int lane = tid & 63, i = lane & 15, g = lane >> 4;
  const int nb = RS == 1 ? (tid >> 6) : (tid >> 6) % NB, rs = RS == 1 ? 0 : (tid >> 6) / NB;
  const int H = a.H, dk = a.dk, dv = a.dv;
  const int cidx = (int)(item / H), h = (int)(item % H);
  int seq, t0, clen, cis;
  chunk_lookup(a, cidx, seq, t0, clen, cis);
  const float Ip = a.Ip[h];
  const float gh = a.g[h] * kLog2e;

  if (tid < 64) {
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
  // the wave's k column and q rows are requested first so that their latency overlaps the block-exponent pass
  float kraw[2][8];
  {
    const TIn* kp = (const TIn*)a.k + qk_row(a, t0, h) + 16 * nb + i;
#pragma unroll
    for (int ks = 0; ks < 2; ++ks)
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int s = 8 * g + j + 32 * ks;
        const bool ok = s < clen;
        const float kv = to_f32(kp[(int64_t)(ok ? s : 0) * qk_stride(a)]);
        kraw[ks][j] = ok ? kv : 0.f;
      }
  }
  float qD[4][4];
  {
    const TIn* qp = (const TIn*)a.q + qk_row(a, t0, h) + 16 * nb + 4 * g;
#pragma unroll
    for (int tb = 0; tb < 4; ++tb) {
      const int t = 16 * tb + i;
      if (t < clen) {
        load_vec<4>(qp + (int64_t)t * qk_stride(a), qD[tb]);
      } else {
#pragma unroll
        for (int r = 0; r < 4; ++r) qD[tb][r] = 0.f;
      }
    }
  }
  stage_load(0);
  // block exponents of the f16 operands (see tile_block_exponents); sO doubles as its scratch
  // FOLD (f16 operands): the tile-start state rides in the operands of the tile's first token, X'_0 = X_0 + f_0 (M_0, I_0)
  // under the block exponents (F_t = L[t,0] f_0, and I_t = (1 - F_t) Ip + F_t I_0 + J-sum has no negative term), so the
  // prefix products yield M_t and I_t without two multiply-adds per state entry; the exponents make room for the state.
  constexpr bool FOLD = !PREC;
  const float* st_mu = a.chunk_mu + (((int64_t)cidx * H + h) * dv) * dk;
  const float* st_I = a.chunk_I + (((int64_t)cidx * H + h) * dv) * dk;
  const bool cache = CACHE && dv <= 64;
  float stm[CACHE ? 16 : 1], sti[CACHE ? 16 : 1];   // CACHE: the thread's share of the state, M_0 = mu_0 I_0 and I_0
  float mm0 = 0.f, im0 = 0.f;
  if constexpr (CACHE) {
    if (cache) {
#pragma unroll
      for (int p = 0; p < 4; ++p) {
        const int idx = tid + p * NT;
        f32x4 m = {0.f, 0.f, 0.f, 0.f}, y = {0.f, 0.f, 0.f, 0.f};
        if (idx < dv * dk / 4) {
          m = *(const f32x4*)(st_mu + 4 * (int64_t)idx);
          y = *(const f32x4*)(st_I + 4 * (int64_t)idx);
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          stm[4 * p + e] = m[e] * y[e];
          sti[4 * p + e] = y[e];
          mm0 = fmaxf(mm0, fabsf(stm[4 * p + e]));
          im0 = fmaxf(im0, fabsf(y[e]));
        }
      }
    }
  }
  TileExponents bexp = {0, 0, 0};
  if constexpr (!PREC)
    bexp = tile_block_exponents((const TIn*)a.k + qk_row(a, t0, h), vp, bp, a.Hq, H, dk, dv, clen, tid, NT, sO, 0, 0,
                                cache ? nullptr : st_mu, st_I, dv * dk / 4, mm0, im0);
  const float down_k = __builtin_amdgcn_exp2f(-(float)bexp.ek);
  const float down_v = __builtin_amdgcn_exp2f(-(float)bexp.ev);
  const float down_b = __builtin_amdgcn_exp2f(-(float)bexp.eb);
  auto stage_store = [&](int buf) {
#pragma unroll
    for (int it = 0; it < NITEM; ++it) {
      const int idx = tid + it * NT;
      const int s = idx >> 2, dq = idx & 3;
      if (idx < kC * kDG / 4) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          sV[(buf * kDG + 4 * dq + e) * kVH + s] = (TSt)(vst[it][e] * down_v);
          sB[(buf * kDG + 4 * dq + e) * kVH + s] = (TSt)(bst[it][e] * down_b);
        }
      }
    }
  };
  stage_store(0);
  if constexpr (CACHE) {
    if (cache) {
      const float f0u = fast_exp2(sC[0]);   // written before the barriers of the exponent pass
      const float cm = (f0u * down_k) * down_v, cj = ((f0u * down_k) * down_k) * down_b;
#pragma unroll
      for (int p = 0; p < 4; ++p) {
        const int idx = tid + p * NT;
        if (idx < dv * dk / 4) {
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            sStM[4 * idx + e] = (f16_t)(cm * stm[4 * p + e]);
            sStI[4 * idx + e] = (f16_t)(cj * sti[4 * p + e]);
          }
        }
      }
      if (tid == 0) { sZero[0] = (f16_t)0.f; sZero[1] = (f16_t)0.f; }
    }
  }
  __syncthreads();

  // ---- per-wave constants of this tile
  // the sums hold M 2^-(ek+ev) and J 2^-(2ek+eb): the tile-start state and the prior enter with the same factors
  // (two steps each, so that no factor leaves the fp32 range where the rows themselves do not)
  float Fm[4], Fj[4], Gi[4], ct[4];
#pragma unroll
  for (int tb = 0; tb < 4; ++tb) {
    ct[tb] = sC[16 * tb + i];
    const float F = fast_exp2(ct[tb]);
    Fm[tb] = (F * down_k) * down_v;
    Fj[tb] = ((F * down_k) * down_k) * down_b;
    Gi[tb] = ((((1.f - F) * Ip) * down_k) * down_k) * down_b;
  }
  f16x8 Lr[6];            // decay operand
  f16x8 kA[2], kk[2];     // k and k*k of the wave's key column for the 64 tokens, operand layout
  // the same with PREC: the decay operand as two bf16 halves, k and k*k in fp32 (the products are split per row)
  bf16x8 Lh[PREC ? 6 : 1], Ll[PREC ? 6 : 1];
  float kf[PREC ? 2 : 1][8], kkf[PREC ? 2 : 1][8];
  {
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      float cs[8];
      *(f32x4*)&cs[0] = *(const f32x4*)&sC[8 * g + 32 * ks];
      *(f32x4*)&cs[4] = *(const f32x4*)&sC[8 * g + 32 * ks + 4];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int s = 8 * g + j + 32 * ks;
        const float ksc = kraw[ks][j] * down_k;
        if constexpr (PREC) {
          kf[ks][j] = ksc;
          kkf[ks][j] = ksc * ksc;
        } else {
          kA[ks][j] = (f16_t)ksc;
          kk[ks][j] = (f16_t)(ksc * ksc);
        }
#pragma unroll
        for (int tb = (ks ? 2 : 0); tb < 4; ++tb) {
          const int t = 16 * tb + i;
          const float lv = (s <= t) ? fast_exp2(ct[tb] - cs[j]) : 0.f;
          if constexpr (PREC) {
            const bf16_t hi = (bf16_t)lv;
            Lh[lidx(tb, ks)][j] = hi;
            Ll[lidx(tb, ks)][j] = (bf16_t)(lv - (float)hi);
          } else {
            Lr[lidx(tb, ks)][j] = (f16_t)lv;
          }
        }
      }
    }
  }
  // mu = M / I comes out times 2^(ek+eb-ev) and 1 / I times 2^(2ek+eb): put right once per output
  const float scale = ((a.scale * __builtin_amdgcn_exp2f((float)bexp.ev)) * down_k) * down_b;
  const float scale_var = ((a.scale * down_k) * down_k) * down_b;
  const float* cmu = st_mu + 16 * nb + 4 * g;
  const float* cI = st_I + 16 * nb + 4 * g;
  // FOLD: the entry of the wave's own key column i instead (operand layout); the lanes that hold token 0 of the
  // operands (g = 0) carry the factor f_0 2^-(ek+ev) resp. f_0 2^-(2ek+eb), the others zero
  const float* cmu1 = st_mu + 16 * nb + i;
  const float* cI1 = st_I + 16 * nb + i;
  const float f0 = (FOLD && g == 0) ? fast_exp2(sC[0]) : 0.f;
  const float c0m = (f0 * down_k) * down_v, c0j = ((f0 * down_k) * down_k) * down_b;

  // tile-start state of the next value row is fetched one iteration ahead
  f32x4 mu0_n = {0.f, 0.f, 0.f, 0.f}, I0_n = {0.f, 0.f, 0.f, 0.f};
  float mu1_n = 0.f, I1_n = 0.f;
  // CACHE: the lanes of token 0 walk the cached state by rows, the others stay on the zero word
  const f16_t* chM = (g == 0) ? sStM + 16 * nb + i : sZero;
  const f16_t* chI = (g == 0) ? sStI + 16 * nb + i : sZero;
  const int ch_stride = (g == 0) ? dk : 0;
  if constexpr (FOLD) {
    if (!cache) {
      mu1_n = cmu1[(int64_t)rs * dk];
      I1_n = cI1[(int64_t)rs * dk];
    }
  } else {
    mu0_n = *(const f32x4*)(cmu + (int64_t)rs * dk);
    I0_n = *(const f32x4*)(cI + (int64_t)rs * dk);
  }
  const int n_groups = dv / kDG;
  for (int dg = 0; dg < n_groups; ++dg) {
    const int buf = dg & 1;
    for (int dd = rs; dd < kDG; dd += RS) {
      const int d = dg * kDG + dd;
      if (dd - rs == kDG / 2 && dg + 1 < n_groups) {
        // rows of the next group go to the other buffer mid-group (read only after the barriers below)
        stage_load(dg + 1);
        stage_store(buf ^ 1);
      }
      const f32x4 mu0 = mu0_n, I0 = I0_n;
      const float mu1 = mu1_n, I1 = I1_n;
      {
        const int64_t dn = (int64_t)min(d + RS, dv - 1) * dk;
        if constexpr (FOLD) {
          if (!cache) {
            mu1_n = cmu1[dn];
            I1_n = cI1[dn];
          }
        } else {
          mu0_n = *(const f32x4*)(cmu + dn);
          I0_n = *(const f32x4*)(cI + dn);
        }
      }
      float M0[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) M0[r] = mu0[r] * I0[r];
      f16x8 XM[2], XJ[2];
      bf16x8 XMh[PREC ? 2 : 1], XMl[PREC ? 2 : 1], XJh[PREC ? 2 : 1], XJl[PREC ? 2 : 1];
#pragma unroll
      for (int ks = 0; ks < 2; ++ks) {
        if constexpr (PREC) {
          float xv[8], xb[8];
          staged8((const float*)&sV[(buf * kDG + dd) * kVH + 8 * g + 32 * ks], xv);
          staged8((const float*)&sB[(buf * kDG + dd) * kVH + 8 * g + 32 * ks], xb);
#pragma unroll
          for (int j = 0; j < 8; ++j) { xv[j] *= kf[ks][j]; xb[j] *= kkf[ks][j]; }
          split_bf16(xv, XMh[ks], XMl[ks]);
          split_bf16(xb, XJh[ks], XJl[ks]);
        } else {
          // 8 consecutive tokens of the row: one 16-byte LDS read each; packed f16 products are the operands
          const f16x8 vv = *(const f16x8*)&sV[(buf * kDG + dd) * kVH + 8 * g + 32 * ks];
          const f16x8 bb = *(const f16x8*)&sB[(buf * kDG + dd) * kVH + 8 * g + 32 * ks];
          XM[ks] = kA[ks] * vv;
          XJ[ks] = kk[ks] * bb;
          if (FOLD && ks == 0) {
            if (cache) {
              // a 16-bit read leaves {value, 0} in the register: the addend pair as it is
              const f16x2 am = __builtin_bit_cast(f16x2, (uint32_t)*(const unsigned short*)(chM + d * ch_stride));
              const f16x2 aj = __builtin_bit_cast(f16x2, (uint32_t)*(const unsigned short*)(chI + d * ch_stride));
              fold_state_pairs(XM[0], XJ[0], kA[0], vv, kk[0], bb, am, aj);
            } else {
              fold_state(XM[0], XJ[0], kA[0], vv, kk[0], bb, (c0m * mu1) * I1, c0j * I1);
            }
          }
        }
      }
      float p[4], pv[4];
#pragma unroll
      for (int tb = 0; tb < 4; ++tb) {
        f32x4 accM = {0.f, 0.f, 0.f, 0.f};
        f32x4 accI = {Gi[tb], Gi[tb], Gi[tb], Gi[tb]};
        if constexpr (PREC) {
          accM = mfma16_split(XMh[0], XMl[0], Lh[lidx(tb, 0)], Ll[lidx(tb, 0)], accM);
          accI = mfma16_split(XJh[0], XJl[0], Lh[lidx(tb, 0)], Ll[lidx(tb, 0)], accI);
          if (tb >= 2) {
            accM = mfma16_split(XMh[1], XMl[1], Lh[lidx(tb, 1)], Ll[lidx(tb, 1)], accM);
            accI = mfma16_split(XJh[1], XJl[1], Lh[lidx(tb, 1)], Ll[lidx(tb, 1)], accI);
          }
        } else {
        accM = mfma16h(XM[0], Lr[lidx(tb, 0)], accM);
        accI = mfma16h(XJ[0], Lr[lidx(tb, 0)], accI);
        if (tb >= 2) {
          accM = mfma16h(XM[1], Lr[lidx(tb, 1)], accM);
          accI = mfma16h(XJ[1], Lr[lidx(tb, 1)], accI);
        }
        }
        float acc = 0.f, accv = 0.f;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const float Mf = FOLD ? accM[r] : fmaf(Fm[tb], M0[r], accM[r]);
          const float If = FOLD ? accI[r] : fmaf(Fj[tb], I0[r], accI[r]);
          const float rI = fast_rcp(If);
          acc = fmaf(Mf * rI, qD[tb][r], acc);
          if (HAS_VAR) accv = fmaf(qD[tb][r] * qD[tb][r], rI, accv);
        }
        p[tb] = acc;
        pv[tb] = accv;
      }
      // sum over the four rows of 16 lanes (key columns 4g..4g+3 of every row): transposing reduction,
      // after which the lanes of row g hold the total of token block g
      sO[(nb * kDG + dd) * kC + 16 * g + i] = rows4_sum_x4(p[0], p[1], p[2], p[3]);
      if (HAS_VAR) sOv[(nb * kDG + dd) * kC + 16 * g + i] = rows4_sum_x4(pv[0], pv[1], pv[2], pv[3]);
    }
    __syncthreads();
    // flush the group's outputs: work item = (token t, 4 value rows)
    for (int idx = tid; idx < kC * kDG / 4; idx += NT) {
      const int t = idx >> 2, dq = idx & 3;
      if (t < clen && valid) {
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
          for (int e = 0; e < 4; ++e) store_rt(a.o_var, off + e, accv[e] * scale_var, a.var_bf16);
        }
      }
    }
    __syncthreads();
  }
}

// The same outputs with the work of a (tile, head) laid out by value rows instead of by key columns: four waves, wave w
// owns the value rows d = w mod 4 and walks over all column blocks of its rows, so a workgroup is four waves whatever
// the head dim and every SIMD of a unit carries the same load.  A workgroup takes a slice of at most 64 value rows
// (blockIdx.y), which keeps three workgroups on a compute unit.  v^T and b^T of the slice stay in LDS (f16,
// block-scaled by the maxima of the slice); the k columns (scaled, with their squares) and the q rows of the next column
// block are staged by the whole workgroup while the rows of the current one are processed (two buffers, one barrier per
// column block), and the outputs are summed over the column blocks in an LDS tile that only the owning wave touches.
// bf16 rows only.  Three waves per SIMD: 168 registers per lane, matrix results in ordinary vector registers.
constexpr int kKH = 72;   // row stride (f16) of the staged k columns

template <bool HAS_VAR>
__global__ __launch_bounds__(256, 3) void chunk_out_rows_kernel(ChunkArgs a, int dvs) {
  extern __shared__ float smem[];
  using TIn = bf16_t;
  const int tid = (int)threadIdx.x, lane = tid & 63, w = tid >> 6, i = lane & 15, g = lane >> 4;
  const int H = a.H, dk = a.dk, dv = a.dv;
  const int cidx = (int)(blockIdx.x / H), h = (int)(blockIdx.x % H);
  const int r0 = (int)blockIdx.y * dvs, rn = min(dvs, dv - r0);   // value rows [r0, r0 + rn) of this workgroup
  int seq, t0, clen, cis;
  chunk_lookup(a, cidx, seq, t0, clen, cis);
  float* sC = smem;                        // [64] running log2-decay inside the tile
  f16_t* sV = (f16_t*)(sC + kC);           // [dvs][kVH] v^T 2^-ev
  f16_t* sB = sV + dvs * kVH;              // [dvs][kVH] b^T 2^-eb
  f16_t* sK = sB + dvs * kVH;              // [2][16][kKH] k^T 2^-ek of a column block
  f16_t* sKK = sK + 2 * 16 * kKH;          // [2][16][kKH] its squares
  bf16_t* sQ = (bf16_t*)(sKK + 2 * 16 * kKH);   // [2][64][16] q rows of a column block
  float* sO = (float*)(sQ + 2 * kC * 16);  // [dvs][64] outputs summed over the column blocks
  float* sOv = sO + dvs * kC;              // same for o_var
  const float Ip = a.Ip[h];
  const float gh = a.g[h] * kLog2e;
  if (tid < 64) {
    const float gt = (lane < clen) ? load_gate(a.gt, (int64_t)(t0 + lane) * H + h, a.gate_bf16) : 0.f;
    sC[lane] = wave_inclusive_scan(-gt * gh, lane);
  }
  const TIn* vp = (const TIn*)a.v + ((int64_t)t0 * H + h) * dv + r0;
  const TIn* bp = (const TIn*)a.b + ((int64_t)t0 * H + h) * dv + r0;
  const TIn* kbase = (const TIn*)a.k + qk_row(a, t0, h);
  const TIn* qbase = (const TIn*)a.q + qk_row(a, t0, h);
  // staging work item of this thread, for v, b (16 value rows per step) and for k, q (one column block per step):
  // (token ss, 4 consecutive rows or columns sq)
  const int ss = tid >> 2, sq = tid & 3;
  const bool s_ok = ss < clen;
  const unsigned kq_off = (unsigned)(s_ok ? ss : 0) * (unsigned)qk_stride(a) + 4u * sq;   // a tile spans < 2^31 elements
  bf16x4 k_next, q_next;   // the thread's share of the next column block, as loaded
  auto request = [&](int nb) {
    k_next = *(const bf16x4*)(kbase + 16 * nb + kq_off);
    q_next = *(const bf16x4*)(qbase + 16 * nb + kq_off);
  };
  request(0);
  // the tile-start state rides in the operands of the first token, see FOLD in chunk_out_kernel
  const float* st_mu = a.chunk_mu + (((int64_t)cidx * H + h) * dv + r0) * dk;
  const float* st_I = a.chunk_I + (((int64_t)cidx * H + h) * dv + r0) * dk;
  const TileExponents bexp = tile_block_exponents(kbase, vp - r0, bp - r0, a.Hq, H, dk, dv, clen, tid, 256, sO, r0, rn,
                                                  st_mu, st_I, rn * dk / 4);
  const float down_k = __builtin_amdgcn_exp2f(-(float)bexp.ek);
  const float down_v = __builtin_amdgcn_exp2f(-(float)bexp.ev);
  const float down_b = __builtin_amdgcn_exp2f(-(float)bexp.eb);
  auto deposit = [&](int buf) {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const float ksc = s_ok ? (float)k_next[e] * down_k : 0.f;
      sK[(buf * 16 + 4 * sq + e) * kKH + ss] = (f16_t)ksc;
      sKK[(buf * 16 + 4 * sq + e) * kKH + ss] = (f16_t)(ksc * ksc);
    }
    *(bf16x4*)&sQ[(buf * kC + ss) * 16 + 4 * sq] = q_next;
  };
  deposit(0);
  {
    const int n_groups = rn / kDG;
#pragma unroll 2
    for (int dg = 0; dg < n_groups; ++dg) {
      float x[4] = {0.f, 0.f, 0.f, 0.f}, y[4] = {0.f, 0.f, 0.f, 0.f};
      if (s_ok) {
        load_vec<4>(vp + (int64_t)ss * H * dv + dg * kDG + 4 * sq, x);
        load_vec<4>(bp + (int64_t)ss * H * dv + dg * kDG + 4 * sq, y);
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        sV[(dg * kDG + 4 * sq + e) * kVH + ss] = (f16_t)(x[e] * down_v);
        sB[(dg * kDG + 4 * sq + e) * kVH + ss] = (f16_t)(y[e] * down_b);
      }
    }
  }
  __syncthreads();

  // per-wave constants of the tile (see chunk_out_kernel)
  float Gi[4], ct[4];
#pragma unroll
  for (int tb = 0; tb < 4; ++tb) {
    ct[tb] = sC[16 * tb + i];
    const float F = fast_exp2(ct[tb]);
    Gi[tb] = ((((1.f - F) * Ip) * down_k) * down_k) * down_b;
  }
  f16x8 Lr[6];
#pragma unroll
  for (int ks = 0; ks < 2; ++ks) {
    float cs[8];
    *(f32x4*)&cs[0] = *(const f32x4*)&sC[8 * g + 32 * ks];
    *(f32x4*)&cs[4] = *(const f32x4*)&sC[8 * g + 32 * ks + 4];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int s = 8 * g + j + 32 * ks;
#pragma unroll
      for (int tb = (ks ? 2 : 0); tb < 4; ++tb) {
        const int t = 16 * tb + i;
        Lr[lidx(tb, ks)][j] = (f16_t)((s <= t) ? fast_exp2(ct[tb] - cs[j]) : 0.f);
      }
    }
  }
  const float scale = ((a.scale * __builtin_amdgcn_exp2f((float)bexp.ev)) * down_k) * down_b;
  const float scale_var = ((a.scale * down_k) * down_k) * down_b;

  const int n_blocks = dk >> 4;
  const float* cmu0 = st_mu + i;   // the entry of the lane's key column i of a block (operand layout)
  const float* cI0 = st_I + i;
  const float f0 = (g == 0) ? fast_exp2(sC[0]) : 0.f;   // lanes that hold token 0 of the operands
  const float c0m = (f0 * down_k) * down_v, c0j = ((f0 * down_k) * down_k) * down_b;
  float mu1_n = cmu0[(int64_t)w * dk], I1_n = cI0[(int64_t)w * dk];
#pragma unroll 1
  for (int nb = 0; nb < n_blocks; ++nb) {
    const int buf = nb & 1;
    const bool more = nb + 1 < n_blocks;
    f16x8 kA[2], kk[2];
    float qD[4][4];
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      kA[ks] = *(const f16x8*)&sK[(buf * 16 + i) * kKH + 8 * g + 32 * ks];
      kk[ks] = *(const f16x8*)&sKK[(buf * 16 + i) * kKH + 8 * g + 32 * ks];
    }
#pragma unroll
    for (int tb = 0; tb < 4; ++tb) {
      const bf16x4 x = *(const bf16x4*)&sQ[(buf * kC + 16 * tb + i) * 16 + 4 * g];
#pragma unroll
      for (int r = 0; r < 4; ++r) qD[tb][r] = (float)x[r];
    }
    if (more) request(nb + 1);
    const float* cmu = cmu0 + 16 * nb;
    const float* cI = cI0 + 16 * nb;
#pragma unroll 1
    for (int d = w; d < rn; d += 4) {
      const float mu1 = mu1_n, I1 = I1_n;
      {
        // the state row of the next iteration: the wave's next row, or its first row of the next column block
        const bool last = d + 4 >= rn;
        const int64_t dn = last ? (int64_t)w * dk + (more ? 16 : 0) : (int64_t)(d + 4) * dk;
        mu1_n = cmu[dn];
        I1_n = cI[dn];
      }
      float* so = sO + d * kC + 16 * g + i;
      float* sov = sOv + d * kC + 16 * g + i;
      float prev = 0.f, prevv = 0.f;
      if (nb) {
        prev = *so;
        if (HAS_VAR) prevv = *sov;
      }
      f16x8 XM[2], XJ[2];
#pragma unroll
      for (int ks = 0; ks < 2; ++ks) {
        const f16x8 vv = *(const f16x8*)&sV[d * kVH + 8 * g + 32 * ks];
        const f16x8 bb = *(const f16x8*)&sB[d * kVH + 8 * g + 32 * ks];
        XM[ks] = kA[ks] * vv;
        XJ[ks] = kk[ks] * bb;
        if (ks == 0) fold_state(XM[0], XJ[0], kA[0], vv, kk[0], bb, (c0m * mu1) * I1, c0j * I1);
      }
      float p[4], pv[4];
#pragma unroll
      for (int tb = 0; tb < 4; ++tb) {
        f32x4 accM = {0.f, 0.f, 0.f, 0.f};
        f32x4 accI = {Gi[tb], Gi[tb], Gi[tb], Gi[tb]};
        accM = mfma16h(XM[0], Lr[lidx(tb, 0)], accM);
        accI = mfma16h(XJ[0], Lr[lidx(tb, 0)], accI);
        if (tb >= 2) {
          accM = mfma16h(XM[1], Lr[lidx(tb, 1)], accM);
          accI = mfma16h(XJ[1], Lr[lidx(tb, 1)], accI);
        }
        float acc = 0.f, accv = 0.f;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const float rI = fast_rcp(accI[r]);
          acc = fmaf(accM[r] * rI, qD[tb][r], acc);
          if (HAS_VAR) accv = fmaf(qD[tb][r] * qD[tb][r], rI, accv);
        }
        p[tb] = acc;
        pv[tb] = accv;
      }
      *so = prev + rows4_sum_x4(p[0], p[1], p[2], p[3]);
      if (HAS_VAR) *sov = prevv + rows4_sum_x4(pv[0], pv[1], pv[2], pv[3]);
    }
    if (more) deposit(buf ^ 1);
    // the other buffer is complete for the next column block (it was last read before the previous barrier); after
    // the last block: the outputs are complete
    __syncthreads();
  }
  // outputs: work item = (token ss, 4 value rows sq)
  if (s_ok) {
    const int n_groups = rn / kDG;
    for (int dg = 0; dg < n_groups; ++dg) {
      const int64_t off = ((int64_t)(t0 + ss) * H + h) * dv + r0 + dg * kDG + 4 * sq;
      TIn* op = (TIn*)a.o + off;
#pragma unroll
      for (int e = 0; e < 4; ++e) op[e] = from_f32<TIn>(sO[(dg * kDG + 4 * sq + e) * kC + ss] * scale);
      if (HAS_VAR) {
#pragma unroll
        for (int e = 0; e < 4; ++e) store_rt(a.o_var, off + e, sOv[(dg * kDG + 4 * sq + e) * kC + ss] * scale_var, a.var_bf16);
      }
    }
  }
}

// value rows per workgroup of chunk_out_rows_kernel: equal slices (multiples of 16) of at most 64 rows, 48 with o_var,
// so that three workgroups fit the LDS of a compute unit
static int out_rows_slice(int dv, bool var) {
  const int cap = var ? 48 : 64;
  const int n = (dv + cap - 1) / cap;
  return ((dv / 16 + n - 1) / n) * 16;
}
static size_t out_rows_lds_bytes(int dv, bool var) {
  const size_t dvs = out_rows_slice(dv, var);
  return sizeof(float) * kC + 2 * sizeof(f16_t) * dvs * kVH + 4 * sizeof(f16_t) * 16 * kKH + 2 * sizeof(bf16_t) * kC * 16 +
         sizeof(float) * dvs * kC * (var ? 2 : 1);
}
static int launch_out_rows(const ChunkArgs& a, hipStream_t s) {
  const bool var = a.flags & PAL_FLAG_HAS_VAR;
  const size_t lds = out_rows_lds_bytes(a.dv, var);
  const int64_t blocks = (int64_t)a.total_chunks * a.H;
  if (blocks > 0x7fffffff) return PAL_E_DIM;
  if (lds > kMaxLds) return PAL_E_HEADDIM;
  const int dvs = out_rows_slice(a.dv, var);
  const dim3 grid((unsigned)blocks, (unsigned)((a.dv + dvs - 1) / dvs));
  if (var) {
    if (int rc = allow_lds((const void*)&chunk_out_rows_kernel<true>, lds)) return rc;
    PAL_TIMED_LAUNCH(kKernChunkOut, s, (chunk_out_rows_kernel<true>), grid, dim3(256), lds, s, a, dvs);
  } else {
    if (int rc = allow_lds((const void*)&chunk_out_rows_kernel<false>, lds)) return rc;
    PAL_TIMED_LAUNCH(kKernChunkOut, s, (chunk_out_rows_kernel<false>), grid, dim3(256), lds, s, a, dvs);
  }
  PAL_HIP_LAUNCH_CHECK();
  return PAL_OK;
}

template <typename TIn, int NB, bool PREC>
static int launch_out_nb_p(const ChunkArgs& a, hipStream_t s) {
  const bool var = a.flags & PAL_FLAG_HAS_VAR;
  const size_t lds = sizeof(float) * (kC + (var ? 2 : 1) * NB * kDG * kC + out_state_cache_floats(NB, PREC)) +
                     4 * (PREC ? sizeof(float) : sizeof(f16_t)) * kDG * kVH;
  const int64_t blocks = (int64_t)a.total_chunks * a.H;
  if (blocks > 0x7fffffff) return PAL_E_DIM;
  if (lds > kMaxLds) return PAL_E_HEADDIM;
  // waves per column block, see chunk_out_kernel (7 blocks x 2 would need 128 VGPRs per wave and spills; with 1-3
  // blocks several workgroups share a compute unit and the repeated per-wave set-up costs more than the balance gains)
  constexpr int RS = (!PREC && (NB == 5 || NB == 6)) ? 2 : 1;
  // (tile, head) pairs per workgroup, see chunk_out_kernel (measured: +9 % at two column blocks, nothing at one or three)
  constexpr int TS = (!PREC && NB == 2) ? 2 : 1;
  const size_t lds_all = lds * TS;
  const unsigned grid = (unsigned)((blocks + TS - 1) / TS);
  if (var) {
    if (int rc = allow_lds((const void*)&chunk_out_kernel<TIn, NB, true, RS, TS, PREC>, lds_all)) return rc;
    PAL_TIMED_LAUNCH(kKernChunkOut, s, (chunk_out_kernel<TIn, NB, true, RS, TS, PREC>), dim3(grid), dim3(NB * RS * TS * 64), lds_all, s, a);
  } else {
    if (int rc = allow_lds((const void*)&chunk_out_kernel<TIn, NB, false, RS, TS, PREC>, lds_all)) return rc;
    PAL_TIMED_LAUNCH(kKernChunkOut, s, (chunk_out_kernel<TIn, NB, false, RS, TS, PREC>), dim3(grid), dim3(NB * RS * TS * 64), lds_all, s, a);
  }
  PAL_HIP_LAUNCH_CHECK();
  return PAL_OK;
}

// fp32 rows take the fp32-accurate variant unless PAL_FLAG_FP32_FAST asks for single bf16/f16 operands
template <typename TIn, int NB>
static int launch_out_nb(const ChunkArgs& a, hipStream_t s) {
  if constexpr (sizeof(TIn) == 4) {
    if (!(a.flags & PAL_FLAG_FP32_FAST)) return launch_out_nb_p<TIn, NB, true>(a, s);
  }
  return launch_out_nb_p<TIn, NB, false>(a, s);
}

template <typename TIn>
static int launch_out(const ChunkArgs& a, hipStream_t s) {
  if constexpr (std::is_same_v<TIn, bf16_t>) {
    // bf16 rows: the layout by value rows (chunk_out_rows_kernel) unless a workgroup of the layout by key columns is
    // exactly two or four waves on at most 64 value rows (measured: 3-7 % faster there, 3-25 % slower elsewhere)
    const int nbk = a.dk / 16;
    const bool by_columns = a.dv <= 64 && (nbk == 2 || nbk == 4);
    if (!by_columns && out_rows_lds_bytes(a.dv, a.flags & PAL_FLAG_HAS_VAR) <= kMaxLds) return launch_out_rows(a, s);
  }
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
  a.Hq = d->n_qk_heads > 0 ? d->n_qk_heads : d->n_heads;
  a.n_seqs = d->n_seqs; a.total_chunks = d->total_chunks;
  a.gate_bf16 = d->gate_dtype == PAL_DTYPE_BF16;
  a.var_bf16 = d->var_dtype == PAL_DTYPE_BF16;
  a.flags = d->flags;
  a.scale = d->scale;
}

}  // namespace pal

namespace pal {

// the one-pass form of chunk_states.hip
bool state_pass_applies(const ChunkArgs& a, int dtype, bool has_j);
int launch_state_pass(const ChunkArgs& a, bool has_j, void* tiles_a, float* tiles_b, const float* init_a,
                      const float* init_b, float* fin_a, float* fin_b, bool reverse, float fin_scale, int kern_id,
                      hipStream_t s);

// Local contribution of every tile to the state, into chunk_mu (and chunk_I when has_j).
template <typename TIn, bool HAS_J, typename TS, bool PREC>
static int launch_tile_delta_t(const ChunkArgs& a, hipStream_t s) {
  const int64_t blocks = (int64_t)a.total_chunks * a.H;
  if (blocks > 0x7fffffff) return PAL_E_DIM;
  // value rows per workgroup: all of them, or the largest multiple of 16 whose staging tiles fit the LDS
  int pieces = 1, dvn = a.dv;
  size_t lds = 0;
  for (;; ++pieces) {
    dvn = ((a.dv / 16 + pieces - 1) / pieces) * 16;
    lds = sizeof(float) * kC + sizeof(TS) * (size_t)(a.dk + (HAS_J ? 2 : 1) * dvn) * StageStride<TS>::value;
    if (lds <= kMaxLds || dvn == 16) break;
  }
  if (lds > kMaxLds) return PAL_E_HEADDIM;
  pieces = (a.dv + dvn - 1) / dvn;
  if (int rc = allow_lds((const void*)&chunk_delta_kernel<TIn, HAS_J, TS, PREC>, lds)) return rc;
  PAL_TIMED_LAUNCH(kKernChunkState, s, (chunk_delta_kernel<TIn, HAS_J, TS, PREC>), dim3((unsigned)blocks, (unsigned)pieces),
                   dim3(256), lds, s, a, dvn);
  PAL_HIP_LAUNCH_CHECK();
  return PAL_OK;
}

// fp32 rows take the fp32-accurate variant (fp32 staging, operands split into two bf16 halves) unless
// PAL_FLAG_FP32_FAST asks for single bf16 operands.
template <typename TIn, bool HAS_J>
static int launch_tile_delta_j(const ChunkArgs& a, hipStream_t s) {
  if constexpr (sizeof(TIn) == 4) {
    if (!(a.flags & PAL_FLAG_FP32_FAST)) return launch_tile_delta_t<TIn, HAS_J, float, true>(a, s);
    const size_t lds_f32 = sizeof(float) * (kC + (size_t)(a.dk + (HAS_J ? 2 : 1) * a.dv) * StageStride<float>::value);
    if (lds_f32 <= kMaxLds) return launch_tile_delta_t<TIn, HAS_J, float, false>(a, s);
  }
  return launch_tile_delta_t<TIn, HAS_J, bf16_t, false>(a, s);
}

int launch_tile_delta(const ChunkArgs& a, int dtype, bool has_j, hipStream_t s) {
  if (dtype == PAL_DTYPE_BF16)
    return has_j ? launch_tile_delta_j<bf16_t, true>(a, s) : launch_tile_delta_j<bf16_t, false>(a, s);
  return has_j ? launch_tile_delta_j<float, true>(a, s) : launch_tile_delta_j<float, false>(a, s);
}

// Tile-start states: local contributions, then the serial scan over the tiles of each sequence.
// has_j = false leaves the precision state out (b, Ip, chunk_I, init_I, final_I are not touched).
int launch_tile_states(const ChunkArgs& a, int dtype, bool has_j, hipStream_t s) {
  if (state_pass_applies(a, dtype, has_j))
    return launch_state_pass(a, has_j, has_j ? (void*)a.chunk_mu : (void*)a.chunk_I, has_j ? a.chunk_I : nullptr, a.init_mu,
                             a.init_I, a.final_mu, a.final_I, false, 1.f, kKernChunkStates, s);
  if (int rc = launch_tile_delta(a, dtype, has_j, s)) return rc;
  {
    const int64_t E = (int64_t)a.dv * a.dk;
    const int64_t blocks = (int64_t)a.n_seqs * a.H * ((E + 1023) / 1024);
    if (blocks > 0x7fffffff) return PAL_E_DIM;
    if (has_j) PAL_TIMED_LAUNCH(kKernChunkScan, s, chunk_scan_kernel, dim3((unsigned)blocks), dim3(256), 0, s, a);
    else PAL_TIMED_LAUNCH(kKernChunkScan, s, gla_scan_kernel, dim3((unsigned)blocks), dim3(256), 0, s, a);
    PAL_HIP_LAUNCH_CHECK();
  }
  return PAL_OK;
}

}  // namespace pal

// ------------------------------------------------------------ forward on the library's own scratch
// The tile-start states of pal_chunk_fwd_static live here instead of in caller memory.  Every GPU the library runs on
// holds its own copy of this array (at its own address) until the process ends.
static __device__ __align__(256) float scratch[PAL_STATIC_SCRATCH_BYTES / sizeof(float)];

namespace pal {

// Device address of `scratch` on the current device.  In host code the array's name is only a handle of the symbol,
// not memory a kernel can touch: the address is asked for once per device (with that device current) and kept.
constexpr int kMaxDevices = 64;
static std::atomic<float*> g_scratch_ptr[kMaxDevices];

static int static_scratch(float** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return (int)e;
  if (dev < 0 || dev >= kMaxDevices) return PAL_E_DIM;
  float* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (!p) {
    void* addr = nullptr;
    e = hipGetSymbolAddress(&addr, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return (int)e;
    if (!addr) return (int)hipErrorInvalidSymbol;
    p = (float*)addr;
    g_scratch_ptr[dev].store(p, std::memory_order_release);   // two threads racing here store the same address
  }
  *out = p;
  return PAL_OK;
}

}  // namespace pal

extern "C" int pal_chunk_fwd_static(const PalDims* d, const PalFwdTensors* t, void* stream) {
  using namespace pal;
  if (!d || !t) return PAL_E_NULL;
  if (t->chunk_mu || t->chunk_I) return PAL_E_STATE;   // the states live in the library's scratch on this path
  PalFwdTensors tt = *t;
  // any aligned non-null value passes the pointer checks; the real addresses follow once the size is known to fit
  tt.chunk_mu = tt.chunk_I = (float*)(uintptr_t)256;
  int rc = check_chunk_common(d, &tt);
  if (rc) return rc;
  const uint64_t entries = (uint64_t)d->total_chunks * (uint64_t)d->n_heads * (uint64_t)d->dv * (uint64_t)d->dk;
  if (entries > PAL_STATIC_SCRATCH_BYTES / (2 * sizeof(float))) return PAL_E_SCRATCH;
  float* base = nullptr;
  rc = static_scratch(&base);
  if (rc) return rc;
  tt.chunk_mu = base;
  tt.chunk_I = base + PAL_STATIC_SCRATCH_BYTES / (2 * sizeof(float));
  ChunkArgs a;
  fill_chunk_args(a, d, &tt);
  hipStream_t s = (hipStream_t)stream;
  // every slot the output kernel reads is written by the state kernels of this call first: nothing has to start at zero
  if (int rc2 = launch_tile_states(a, d->dtype, true, s)) return rc2;
  if (d->dtype == PAL_DTYPE_BF16) return launch_out<bf16_t>(a, s);
  return launch_out<float>(a, s);
}

extern "C" int pal_chunk_fwd(const PalDims* d, const PalFwdTensors* t, void* stream) {
  using namespace pal;
  if (d && t && (d->flags & PAL_FLAG_STATES_ONLY)) {
    // tile-start states only: the outputs are not touched and need not exist
    PalDims dd = *d;
    dd.flags &= ~(uint32_t)(PAL_FLAG_STATES_ONLY | PAL_FLAG_HAS_VAR);
    PalFwdTensors tt = *t;
    tt.o = (void*)(uintptr_t)256;   // passes the pointer checks, never dereferenced
    tt.o_var = nullptr;
    int rc = check_chunk_common(&dd, &tt);
    if (rc) return rc;
    ChunkArgs a;
    fill_chunk_args(a, &dd, &tt);
    return launch_tile_states(a, dd.dtype, true, (hipStream_t)stream);
  }
  int rc = check_chunk_common(d, t);
  if (rc) return rc;
  ChunkArgs a;
  fill_chunk_args(a, d, t);
  hipStream_t s = (hipStream_t)stream;
  if (int rc2 = launch_tile_states(a, d->dtype, true, s)) return rc2;
  if (d->dtype == PAL_DTYPE_BF16) return launch_out<bf16_t>(a, s);
  return launch_out<float>(a, s);
}
