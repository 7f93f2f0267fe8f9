// Pieces shared by the chunked forward and backward kernels.
//
// Chunked form of the recurrence (one sequence, one head, a tile of C = 64
// tokens; c_t = running sum of log2 f inside the tile, F_t = 2^{c_t},
// L[t,s] = 2^{c_t - c_s} for s <= t, else 0):
//   M_t = sum_s L[t,s] v_s k_s^T + F_t M_0          (the associative scan of the
//   I_t = sum_s L[t,s] b_s (k_s*k_s)^T + F_t (I_0 - Ip) + Ip    reference,
//                                     chunk_palimpsa_forgetting_scalar.py:190-195)
// The sums over s are bf16 MFMA contractions with fp32 accumulation; M_0, I_0
// are the fp32 states at the start of the tile.
#pragma once
#include "pal_common.h"

namespace pal {

constexpr int kC = PAL_CHUNK;  // tokens per tile
constexpr int kScanTiles = 1024;   // per-tile decays a scan kernel keeps in LDS at a time

// internal bit of ChunkArgs::flags (above the PAL_FLAG_* bits): chunk_delta_kernel weights token s with the decay
// from the start of the tile up to s instead of from s to the end of the tile
constexpr uint32_t kFlagDecayFromStart = 1u << 30;

struct ChunkArgs {
  const void *q, *k, *v, *b, *gt;
  const float *g, *Ip;
  void *o, *o_var;
  const float *init_mu, *init_I;
  float *final_mu, *final_I;
  const int32_t *cu_seqlens, *chunk_table, *chunk_offsets;
  float *chunk_mu, *chunk_I;
  int32_t T, H, dk, dv, n_seqs, total_chunks;
  int32_t Hq;   // heads of q and k: H, or a divisor of it when a group of H / Hq value heads shares one q/k head
  int32_t gate_bf16, var_bf16;
  uint32_t flags;
  float scale;
};

// q and k rows of value head h: element offset of token t's row, and the token stride, in a [tokens, Hq, dk] tensor
__device__ __forceinline__ int64_t qk_row(const ChunkArgs& a, int64_t t, int h) {
  return (t * a.Hq + h / (a.H / a.Hq)) * a.dk;
}
__device__ __forceinline__ int64_t qk_stride(const ChunkArgs& a) { return (int64_t)a.Hq * a.dk; }

// tile c -> (sequence, first token in the packed/batched token axis, tokens in tile, index in sequence)
__device__ __forceinline__ void chunk_lookup(const ChunkArgs& a, int c, int& seq, int& t0, int& clen, int& cis) {
  if (a.chunk_table) {
    const int32_t* row = a.chunk_table + 4 * (int64_t)c;
    seq = min(max(row[0], 0), a.n_seqs - 1);
    cis = row[3];
    // a tile stays inside the packed token axis whatever the table holds (its first token always exists:
    // masked lanes still address it)
    t0 = min(max(row[1], 0), a.T - 1);
    clen = min(max(row[2], 0), min(kC, a.T - t0));
  } else {
    const int per = (a.T + kC - 1) / kC;
    seq = c / per;
    cis = c - seq * per;
    t0 = seq * a.T + cis * kC;
    clen = min(kC, a.T - cis * kC);
  }
}

// sequence n -> (first token, length, index of its first tile)
__device__ __forceinline__ void seq_lookup(const ChunkArgs& a, int n, int& bos, int& len, int& cbase) {
  if (a.cu_seqlens) {
    packed_seq_bounds(a.cu_seqlens, n, a.T, bos, len);
    // the tiles of a sequence stay inside the per-tile buffers
    cbase = min(max(a.chunk_offsets[n], 0), a.total_chunks);
    len = min(len, (a.total_chunks - cbase) * kC);
  } else {
    bos = n * a.T;
    len = a.T;
    cbase = n * ((a.T + kC - 1) / kC);
  }
}

// Block exponents of a tile for the f16 operands of the prefix products.  The operands
//   X^M = (k 2^-ek)(v 2^-ev)  and  X^J = (k 2^-ek)^2 (b 2^-eb)
// are built with packed f16 multiplies from f16 copies of the scaled rows; ek, ev, eb bring the largest |k| of the
// tile to [1, 2) and the largest |v|, |b| to [2^11, 2^12), so that the operands use the top of the f16 range whatever
// the magnitude of the rows (entries more than 2^26 below the largest of their tensor in the tile lose bits, which
// is an absolute error far below that of the bf16 rows).  The sums then hold M 2^-(ek+ev) and J 2^-(2ek+eb); the
// tile-start state enters with the same factors and mu = M / I is put right once per output by 2^(ev-ek-eb), so the
// scaling costs nothing per state entry.  A tensor that is all zero (or holds inf/nan) gets exponent 0.
// With st_mu, st_I (the sn4 groups of four consecutive entries of the tile-start state that the workgroup uses, as
// (mu, I)) the exponents also make room for the state, which the caller adds to the operands of the tile's first
// token: ev and eb are raised until |M_0| 2^-(ek+ev) and I_0 2^-(2ek+eb) stay below 2^14 (the rows then sit lower in
// the f16 range; what they lose is small against the state they are added to).
// Every thread of the workgroup calls this (it synchronises); sMax is LDS scratch of 5 floats per wave.
struct TileExponents { int ek, ev, eb; };

__device__ __forceinline__ int block_exponent_of(float m, int target) {
  // m is a maximum of absolute values: zero, inf and nan keep exponent 0 (the arithmetic then yields what fp32 would)
  return (m > 0.f && m < __builtin_inff()) ? ilogbf(m) - target : 0;
}

// vn > 0 restricts the maxima of v and b to the value rows [v0, v0 + vn) (a workgroup that only forms products of those)
template <typename TIn>
__device__ __forceinline__ TileExponents tile_block_exponents(const TIn* kt, const TIn* vt, const TIn* bt, int Hq, int H,
                                                              int dk, int dv, int clen, int tid, int nthreads,
                                                              float* sMax, int v0 = 0, int vn = 0,
                                                              const float* st_mu = nullptr, const float* st_I = nullptr,
                                                              int sn4 = 0, float mm0 = 0.f, float im0 = 0.f) {
  // (mm0, im0: the thread's maxima of |M_0| and I_0 where the caller has read its share of the state already)
  float km = 0.f, vm = 0.f, bm = 0.f, mm = mm0, im = im0;
  if (st_mu) {
#pragma unroll 4
    for (int idx = tid; idx < sn4; idx += nthreads) {
      const f32x4 m = *(const f32x4*)(st_mu + 4 * (int64_t)idx), y = *(const f32x4*)(st_I + 4 * (int64_t)idx);
#pragma unroll
      for (int e = 0; e < 4; ++e) { mm = fmaxf(mm, fabsf(m[e] * y[e])); im = fmaxf(im, fabsf(y[e])); }
    }
  }
  const int gk = dk >> 3, gv = (vn > 0 ? vn : dv) >> 3;
  vt += v0;
  bt += v0;
  for (int idx = tid; idx < kC * gk; idx += nthreads) {
    const int s = idx / gk, c = idx - s * gk;
    if (s < clen) {
      float x[8];
      load_vec<4>(kt + (int64_t)s * Hq * dk + 8 * c, x);
      load_vec<4>(kt + (int64_t)s * Hq * dk + 8 * c + 4, x + 4);
#pragma unroll
      for (int e = 0; e < 8; ++e) km = fmaxf(km, fabsf(x[e]));
    }
  }
  for (int idx = tid; idx < kC * gv; idx += nthreads) {
    const int s = idx / gv, c = idx - s * gv;
    if (s < clen) {
      float x[8], y[8];
      load_vec<4>(vt + (int64_t)s * H * dv + 8 * c, x);
      load_vec<4>(vt + (int64_t)s * H * dv + 8 * c + 4, x + 4);
      load_vec<4>(bt + (int64_t)s * H * dv + 8 * c, y);
      load_vec<4>(bt + (int64_t)s * H * dv + 8 * c + 4, y + 4);
#pragma unroll
      for (int e = 0; e < 8; ++e) { vm = fmaxf(vm, fabsf(x[e])); bm = fmaxf(bm, fabsf(y[e])); }
    }
  }
  km = wave_max(km);
  vm = wave_max(vm);
  bm = wave_max(bm);
  mm = wave_max(mm);
  im = wave_max(im);
  const int w = tid >> 6, nw = (nthreads + 63) >> 6;
  if ((tid & 63) == 0) {
    sMax[5 * w] = km; sMax[5 * w + 1] = vm; sMax[5 * w + 2] = bm; sMax[5 * w + 3] = mm; sMax[5 * w + 4] = im;
  }
  __syncthreads();
  km = 0.f; vm = 0.f; bm = 0.f; mm = 0.f; im = 0.f;
  for (int x = 0; x < nw; ++x) {
    km = fmaxf(km, sMax[5 * x]); vm = fmaxf(vm, sMax[5 * x + 1]); bm = fmaxf(bm, sMax[5 * x + 2]);
    mm = fmaxf(mm, sMax[5 * x + 3]); im = fmaxf(im, sMax[5 * x + 4]);
  }
  __syncthreads();
  TileExponents e;
  e.ek = block_exponent_of(km, 0);
  e.ev = block_exponent_of(vm, 11);
  e.eb = block_exponent_of(bm, 11);
  if (mm > 0.f && mm < __builtin_inff()) e.ev = max(e.ev, ilogbf(mm) - 13 - e.ek);
  if (im > 0.f && im < __builtin_inff()) e.eb = max(e.eb, ilogbf(im) - 13 - 2 * e.ek);
  return e;
}

// inclusive prefix sum over the 64 lanes of a wave: four shifted adds inside each row of 16 lanes (DPP
// row_shr with zero fill), then the totals of the rows before (lane 15 of each, read as scalars)
template <int N>
__device__ __forceinline__ float row_shr_zero(float x) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x110 + N, 0xf, 0xf, true));
}
__device__ __forceinline__ float wave_inclusive_scan(float x, int lane) {
  x += row_shr_zero<1>(x);
  x += row_shr_zero<2>(x);
  x += row_shr_zero<4>(x);
  x += row_shr_zero<8>(x);
  const float t0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, x), 15));
  const float t1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, x), 31));
  const float t2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, x), 47));
  const int row = lane >> 4;
  return x + (row == 0 ? 0.f : row == 1 ? t0 : row == 2 ? t0 + t1 : (t0 + t1) + t2);
}

}  // namespace pal
