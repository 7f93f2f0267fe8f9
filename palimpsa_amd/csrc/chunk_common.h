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

struct ChunkArgs {
  const void *q, *k, *v, *b, *gt;
  const float *g, *Ip;
  void *o, *o_var;
  const float *init_mu, *init_I;
  float *final_mu, *final_I;
  const int32_t *cu_seqlens, *chunk_table, *chunk_offsets;
  float *chunk_mu, *chunk_I;
  int32_t T, H, dk, dv, n_seqs, total_chunks;
  int32_t gate_bf16, var_bf16;
  uint32_t flags;
  float scale;
};

// tile c -> (sequence, first token in the packed/batched token axis, tokens in tile, index in sequence)
__device__ __forceinline__ void chunk_lookup(const ChunkArgs& a, int c, int& seq, int& t0, int& clen, int& cis) {
  if (a.chunk_table) {
    const int32_t* row = a.chunk_table + 4 * (int64_t)c;
    seq = row[0]; t0 = row[1]; clen = row[2]; cis = row[3];
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
    bos = a.cu_seqlens[n];
    len = a.cu_seqlens[n + 1] - bos;
    cbase = a.chunk_offsets[n];
  } else {
    bos = n * a.T;
    len = a.T;
    cbase = n * ((a.T + kC - 1) / kC);
  }
}

// inclusive prefix sum over the 64 lanes of a wave
__device__ __forceinline__ float wave_inclusive_scan(float x, int lane) {
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    float y = __shfl_up(x, off);
    if (lane >= off) x += y;
  }
  return x;
}

}  // namespace pal
