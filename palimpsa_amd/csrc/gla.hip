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
int launch_tile_delta(const ChunkArgs& a, int dtype, bool has_j, hipStream_t s);
int launch_group_sum(const void* src_q, const void* src_k, void* dst_q, void* dst_k, int64_t tokens, int Hq, int rep, int dk,
                     int dtype, hipStream_t s);
bool state_pass_applies(const ChunkArgs& a, int dtype, bool has_j);
int launch_state_pass(const ChunkArgs& a, bool has_j, void* tiles_a, float* tiles_b, const float* init_a,
                      const float* init_b, float* fin_a, float* fin_b, bool reverse, float fin_scale, int kern_id,
                      hipStream_t s);

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

// Arguments of gla_tile_kernel: the shared tile/gate bookkeeping plus the roles of the three row tensors.
struct GlaTileArgs {
  ChunkArgs c;            // T, H, tiles, gate (gt, g), scale
  const void *X, *Y;      // rows [token][H][dc]: X plays the query, Y the key of the scores
  const void* Z;          // rows [token][H][de]: what the scores mix
  const bf16_t* St;       // per-tile states [tile][H][dv][dk], bf16
  void* out;              // rows [token][H][de]
  const void* W;          // optional rows [token][H][de]: dot[token] = sum_e W out (fp32, before rounding)
  float* dot;             // [H][tokens] (head-major, so that the gate kernel reads contiguous rows) or null
  int64_t n_tokens;       // tokens in the batch (row length of dot)
  int32_t dc, de;         // contraction width of the scores, width of the output rows
  // heads in X, Y, Z and W (H, or the number of shared q/k heads where the tensor is q or k: value head h then reads
  // the rows of head h / (H / heads)); out always has one row per value head
  int32_t hX, hY, hZ, hW;
};

// One kernel for the tile-parallel part of the forward and of the three input gradients.  For the 64
// tokens of a tile, with x the token of the output row and y the tokens it attends to,
//     out[x, e] = scale * ( w_x sum_c St[e, c] X[x, c]  +  sum_y  (X[x,:] . Y[y,:]) L(x, y) Z[y, e] )
//   forward (REVERSE = false):  y <= x,  L = 2^{c_x - c_y},  w_x = 2^{c_x}         (decay since the tile start)
//   reverse (REVERSE = true):   y >= x,  L = 2^{c_y - c_x},  w_x = 2^{c_end - c_x} (decay up to the tile end)
//   o   : X = q,  Y = k,  Z = v,  St = tile-start state S [dv][dk]
//   dq  : X = dO, Y = v,  Z = k,  St = S read transposed (STATE_T)
//   dv  : X = k,  Y = q,  Z = dO, St = gradient of the tile-end state G [dv][dk],      reverse
//   dk  : X = v,  Y = dO, Z = q,  St = G read transposed,                              reverse
// One workgroup of 4 waves per (tile, head), two phases.
//  (1) Scores: wave w owns the tokens x in [16w, 16w+16).
//        P^T[y,x] = sum_c Y[y,c] X[x,c]        A = Y rows (LDS), B = the wave's X rows (LDS)
//        P^T     *= L(x,y), masked             in the accumulator layout (column x per lane, 4 rows y)
//      The accumulators of two neighbouring y blocks, rounded to bf16, ARE a B operand of the second
//      product when its contraction index is mapped to tokens as slot (g, j) -> y = 32p + 16(j/4) + 4g + j%4;
//      they are parked in LDS so that every wave can use the scores of all 64 tokens.
//  (2) Output: wave w owns the blocks of 16 output columns [w EB, (w+1) EB) for all 64 tokens.
//        out^T[e,x] = w_x sum_c St[e,c] X[x,c]  A = state rows (global, bf16), loaded once and used
//                                               for the four token blocks, B = X rows (LDS)
//                   + sum_y Z^T[e,y] P^T[y,x]   A = Z^T rows (LDS, read with the token map above)
//      so every state entry is read by exactly one wave of the workgroup.
// EB = ceil(de / 64) column blocks per wave.
// (second launch bound: at most 256 registers per lane, so matrix results stay in ordinary vector registers)
template <typename TIn, int EB, bool REVERSE, bool STATE_T>
__global__ __launch_bounds__(256, 2) void gla_tile_kernel(GlaTileArgs A) {
  extern __shared__ float smem[];
  const ChunkArgs& a = A.c;
  const int H = a.H, dc = A.dc, de = A.de;
  const int KS = (dc + 31) >> 5;      // contraction steps of the scores and of the state term
  const int dcp = 32 * KS + 16;       // row stride (bf16) of the X and Y tiles: 32 bytes more than a multiple of 64 (no bank conflicts)
  float* sC = smem;                   // [64] running log2 decay inside the tile
  float* sDot = sC + kC;              // [4][64] partial dot products of the waves
  bf16x8* sP = (bf16x8*)(sDot + 4 * kC);   // [4 token blocks][2][64 lanes] score operands
  bf16_t* sY = (bf16_t*)(sP + 4 * 2 * 64); // [64][dcp]
  bf16_t* sX = sY + kC * dcp;         // [64][dcp]
  bf16_t* sZT = sX + kC * dcp;        // [de][kVT]
  const int tid = threadIdx.x, lane = tid & 63, i = lane & 15, g = lane >> 4;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int cidx = blockIdx.x / H, h = blockIdx.x % H;
  int seq, t0, clen, cis;
  chunk_lookup(a, cidx, seq, t0, clen, cis);
  if (w == 0) {
    const float gh = a.g[h] * kLog2e;
    const float gt = (lane < clen) ? load_gate(a.gt, (int64_t)(t0 + lane) * H + h, a.gate_bf16) : 0.f;
    sC[lane] = wave_inclusive_scan(-gt * gh, lane);
  }
  // head of this workgroup's rows in each tensor, and the tensors' token strides in heads
  const int hsX = A.hX, hsY = A.hY, hsZ = A.hZ, hsW = A.hW;
  const int hx = h / (H / hsX), hy = h / (H / hsY), hz = h / (H / hsZ), hw = h / (H / hsW);
  // X rows of token block xb as a B operand (column x = 16 xb + i, contraction index c = 32 ks + 8 g + j), from LDS
  auto x_operand = [&](int xb, int ks) { return *(const bf16x8*)(sX + (16 * xb + i) * dcp + 8 * g + 32 * ks); };
  // State operands of this wave: blocks of 16 output columns [w EB, (w+1) EB), rows e = 16 eb + i, contraction
  // index c = 32 ks + 8 g + j.  The first step is requested before the staging below so that its latency
  // overlaps the staging's, every further step one step ahead of its use.
  const bf16_t* St = A.St + ((int64_t)cidx * H + h) * dc * de;
  const int n_eb = de >> 4;
  const bf16_t* srow[EB];
#pragma unroll
  for (int el = 0; el < EB; ++el) {
    const int e = 16 * min(w * EB + el, n_eb - 1) + i;   // a block past the end repeats the last one (not stored)
    srow[el] = STATE_T ? St + (int64_t)(8 * g) * de + e : St + (int64_t)e * dc + 8 * g;
  }
  bf16x8 raw[EB];
  auto fetch_state = [&](int ks) {
    const bool ok = 32 * ks + 8 * g < dc;
#pragma unroll
    for (int el = 0; el < EB; ++el) {
      raw[el] = bf16x8{0, 0, 0, 0, 0, 0, 0, 0};
      if (ok) {
        if constexpr (STATE_T) {
          // the state is stored [c][e]: eight rows apart, neighbouring lanes read neighbouring columns
#pragma unroll
          for (int j = 0; j < 8; ++j) raw[el][j] = srow[el][(int64_t)(32 * ks + j) * de];
        } else {
          raw[el] = *(const bf16x8*)(srow[el] + 32 * ks);
        }
      }
    }
  };
  fetch_state(0);
  {
    // Y rows, zero beyond the tile's tokens and beyond dc
    const TIn* yp = (const TIn*)A.Y + ((int64_t)t0 * hsY + hy) * dc;
    const int groups = 4 * KS;
    for (int idx = tid; idx < kC * groups; idx += 256) {
      const int s = idx / groups, c8 = idx - s * groups;
      bf16x8 yx = {0, 0, 0, 0, 0, 0, 0, 0}, xx = {0, 0, 0, 0, 0, 0, 0, 0};
      if (s < clen && 8 * c8 < dc) {
        yx = load_bf16x8(yp + (int64_t)s * hsY * dc + 8 * c8);
        xx = load_bf16x8((const TIn*)A.X + ((int64_t)(t0 + s) * hsX + hx) * dc + 8 * c8);
      }
      *(bf16x8*)&sY[s * dcp + 8 * c8] = yx;
      *(bf16x8*)&sX[s * dcp + 8 * c8] = xx;
    }
    // Z transposed (token index fastest), zero beyond the tile's tokens.  A work item is two consecutive
    // tokens by eight columns: neighbouring lanes read neighbouring 16-byte pieces of a row, and a
    // pair of tokens goes to LDS as one 32-bit word per column.
    const TIn* zp = (const TIn*)A.Z + ((int64_t)t0 * hsZ + hz) * de;
    const int zgroups = de >> 3;
    for (int idx = tid; idx < (kC / 2) * zgroups; idx += 256) {
      const int sp = idx / zgroups, c8 = idx - sp * zgroups;
      bf16x8 z0 = {0, 0, 0, 0, 0, 0, 0, 0}, z1 = {0, 0, 0, 0, 0, 0, 0, 0};
      if (2 * sp < clen) z0 = load_bf16x8(zp + (int64_t)(2 * sp) * hsZ * de + 8 * c8);
      if (2 * sp + 1 < clen) z1 = load_bf16x8(zp + (int64_t)(2 * sp + 1) * hsZ * de + 8 * c8);
#pragma unroll
      for (int e = 0; e < 8; ++e) *(bf16x2*)&sZT[(8 * c8 + e) * kVT + 2 * sp] = bf16x2{z0[e], z1[e]};
    }
  }
  __syncthreads();

  // ---- phase 1: decayed, masked scores of token block w against the blocks on its causal side
  {
    const int tb = w;
    f32x4 accS[4];
#pragma unroll
    for (int yb = 0; yb < 4; ++yb) accS[yb] = f32x4{0.f, 0.f, 0.f, 0.f};
    for (int ks = 0; ks < KS; ++ks) {
      const bf16x8 Xo = x_operand(tb, ks);
#pragma unroll
      for (int yb = 0; yb < 4; ++yb)
        if (REVERSE ? yb >= tb : yb <= tb)
          accS[yb] = mfma16(*(const bf16x8*)(sY + (16 * yb + i) * dcp + 8 * g + 32 * ks), Xo, accS[yb]);
    }
    const float cx = sC[16 * tb + i];
#pragma unroll
    for (int p = 0; p < 2; ++p) {
      bf16x8 P;
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        const int yb = 2 * p + half;
        const f32x4 cy = *(const f32x4*)&sC[16 * yb + 4 * g];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const bool side = REVERSE ? yb >= tb : yb <= tb;
          const bool live = side && (yb != tb || (REVERSE ? 4 * g + r >= i : 4 * g + r <= i));
          const float val = live ? accS[yb][r] * fast_exp2(REVERSE ? cy[r] - cx : cx - cy[r]) : 0.f;
          P[4 * half + r] = (bf16_t)val;
        }
      }
      sP[(tb * 2 + p) * 64 + lane] = P;
    }
  }
  __syncthreads();

  // ---- phase 2: output columns of this wave for all four token blocks
  const float scale = a.scale;
  float wx[4];
#pragma unroll
  for (int xb = 0; xb < 4; ++xb) {
    const float cx = sC[16 * xb + i];
    wx[xb] = fast_exp2(REVERSE ? sC[kC - 1] - cx : cx);
  }
  f32x4 acc[EB][4];
#pragma unroll
  for (int el = 0; el < EB; ++el)
#pragma unroll
    for (int xb = 0; xb < 4; ++xb) acc[el][xb] = f32x4{0.f, 0.f, 0.f, 0.f};
  bf16x8 Xn[4];
#pragma unroll
  for (int xb = 0; xb < 4; ++xb) Xn[xb] = x_operand(xb, 0);
  for (int ks = 0; ks < KS; ++ks) {
    bf16x8 Sa[EB], Xo[4];
#pragma unroll
    for (int el = 0; el < EB; ++el) Sa[el] = raw[el];
#pragma unroll
    for (int xb = 0; xb < 4; ++xb) Xo[xb] = Xn[xb];
    if (ks + 1 < KS) {                         // next step's operands in flight while this step's products run
      fetch_state(ks + 1);
#pragma unroll
      for (int xb = 0; xb < 4; ++xb) Xn[xb] = x_operand(xb, ks + 1);
    }
#pragma unroll
    for (int el = 0; el < EB; ++el)
#pragma unroll
      for (int xb = 0; xb < 4; ++xb) acc[el][xb] = mfma16(Sa[el], Xo[xb], acc[el][xb]);
  }
  bf16x8 P[4][2];
#pragma unroll
  for (int xb = 0; xb < 4; ++xb)
#pragma unroll
    for (int p = 0; p < 2; ++p) P[xb][p] = sP[(xb * 2 + p) * 64 + lane];
  float dot[4] = {0.f, 0.f, 0.f, 0.f};
  const bool has_dot = A.dot != nullptr;
#pragma unroll
  for (int el = 0; el < EB; ++el) {
    const int eb = min(w * EB + el, n_eb - 1);
    const bool valid = w * EB + el < n_eb;
    const bf16_t* zrow = sZT + (16 * eb + i) * kVT + 4 * g;
    bf16x8 Za[2];
#pragma unroll
    for (int p = 0; p < 2; ++p) {
      const bf16x4 lo = *(const bf16x4*)(zrow + 32 * p), hi = *(const bf16x4*)(zrow + 32 * p + 16);
      Za[p] = bf16x8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    }
#pragma unroll
    for (int xb = 0; xb < 4; ++xb) {
#pragma unroll
      for (int r = 0; r < 4; ++r) acc[el][xb][r] *= wx[xb];
#pragma unroll
      for (int p = 0; p < 2; ++p)
        if ((REVERSE ? 2 * p + 1 >= xb : 2 * p <= xb)) acc[el][xb] = mfma16(Za[p], P[xb][p], acc[el][xb]);
      // finished block: scale, and take the dot product with W while the values are still fp32
      const int x = 16 * xb + i;
#pragma unroll
      for (int r = 0; r < 4; ++r) acc[el][xb][r] *= scale;
      if (has_dot && valid && x < clen) {
        float wv[4];
        load_vec<4>((const TIn*)A.W + ((int64_t)(t0 + x) * hsW + hw) * de + 16 * eb + 4 * g, wv);
#pragma unroll
        for (int r = 0; r < 4; ++r) dot[xb] = fmaf(wv[r], acc[el][xb][r], dot[xb]);
      }
    }
  }
  if (has_dot) {
    // rows g of a wave hold different output columns of the same token: sum them, then the four waves
    const float tot = rows4_sum_x4(dot[0], dot[1], dot[2], dot[3]);   // lanes of row g: token block g
    sDot[w * kC + lane] = tot;                                        // lane = 16 g + i = token
  }
  // The results go out through LDS (the staging tiles are dead once every wave has its products): a lane holds
  // four columns of one token, which would make 8-byte pieces of rows; from the tile in LDS each row is written
  // as one contiguous run of 16-byte accesses.
  __syncthreads();
  TIn* sOut = (TIn*)sP;               // [64][de + 8 / sizeof-ratio] over the score, Y and Z tiles
  const int ostride = de + (16 / (int)sizeof(TIn));
#pragma unroll
  for (int el = 0; el < EB; ++el) {
    const int ebn = w * EB + el;
    if (ebn < n_eb) {
#pragma unroll
      for (int xb = 0; xb < 4; ++xb) store_vec<4>(sOut + (16 * xb + i) * ostride + 16 * ebn + 4 * g, (const float*)&acc[el][xb]);
    }
  }
  if (has_dot && w == 0 && lane < clen)
    A.dot[(int64_t)h * A.n_tokens + t0 + lane] = (sDot[lane] + sDot[kC + lane]) + (sDot[2 * kC + lane] + sDot[3 * kC + lane]);
  __syncthreads();
  {
    constexpr int VEC = 16 / (int)sizeof(TIn);   // elements per 16-byte access
    const int per_row = de / VEC;
    TIn* obase = (TIn*)A.out + ((int64_t)t0 * H + h) * de;
    for (int idx = tid; idx < clen * per_row; idx += 256) {
      const int x = idx / per_row, c = idx - x * per_row;
      *(f32x4*)(obase + (int64_t)x * H * de + VEC * c) = *(const f32x4*)(sOut + x * ostride + VEC * c);
    }
  }
}

enum GlaRole { kGlaOut = 0, kGlaDq, kGlaDv, kGlaDk };

template <typename TIn, int EB, bool REVERSE, bool STATE_T>
static int launch_gla_tile_eb(const GlaTileArgs& A, int kern_id, hipStream_t s) {
  const int KS = (A.dc + 31) / 32;
  const size_t lds_head = sizeof(float) * (kC + 4 * kC);
  const size_t lds_stage = 16 * 4 * 2 * 64 + sizeof(bf16_t) * (2 * (size_t)kC * (32 * KS + 16) + (size_t)A.de * kVT);
  const size_t lds_out = (size_t)kC * (A.de * sizeof(TIn) + 16);   // the output tile reuses the staging area
  const size_t lds = lds_head + (lds_stage > lds_out ? lds_stage : lds_out);
  const int64_t blocks = (int64_t)A.c.total_chunks * A.c.H;
  if (blocks > 0x7fffffff) return PAL_E_DIM;
  if (lds > kMaxLds) return PAL_E_HEADDIM;
  if (int rc = allow_lds((const void*)&gla_tile_kernel<TIn, EB, REVERSE, STATE_T>, lds)) return rc;
  PAL_TIMED_LAUNCH(kern_id, s, (gla_tile_kernel<TIn, EB, REVERSE, STATE_T>), dim3((unsigned)blocks), dim3(256), lds, s, A);
  PAL_HIP_LAUNCH_CHECK();
  return PAL_OK;
}

template <typename TIn, bool REVERSE, bool STATE_T>
static int launch_gla_tile_rs(const GlaTileArgs& A, int kern_id, hipStream_t s) {
  switch ((A.de + 63) / 64) {
    case 1: return launch_gla_tile_eb<TIn, 1, REVERSE, STATE_T>(A, kern_id, s);
    case 2: return launch_gla_tile_eb<TIn, 2, REVERSE, STATE_T>(A, kern_id, s);
    case 3: return launch_gla_tile_eb<TIn, 3, REVERSE, STATE_T>(A, kern_id, s);
    case 4: return launch_gla_tile_eb<TIn, 4, REVERSE, STATE_T>(A, kern_id, s);
    default: return PAL_E_HEADDIM;
  }
}

template <typename TIn>
static int launch_gla_tile(const GlaTileArgs& A, GlaRole role, hipStream_t s) {
  switch (role) {
    case kGlaOut: return launch_gla_tile_rs<TIn, false, false>(A, kKernGlaOut, s);
    case kGlaDq: return launch_gla_tile_rs<TIn, false, true>(A, kKernGlaDq, s);
    case kGlaDv: return launch_gla_tile_rs<TIn, true, false>(A, kKernGlaDv, s);
    default: return launch_gla_tile_rs<TIn, true, true>(A, kKernGlaDk, s);
  }
}

static int launch_gla_tile_dt(const GlaTileArgs& A, int dtype, GlaRole role, hipStream_t s) {
  return dtype == PAL_DTYPE_BF16 ? launch_gla_tile<bf16_t>(A, role, s) : launch_gla_tile<float>(A, role, s);
}

// ------------------------------------------------------------------ the three input gradients in one kernel
// For head dims up to 64 and bf16 rows the tiles of q, k, v, dO of a (tile, head) and its two states fit into LDS
// together (76 KB, two workgroups per compute unit), so one workgroup forms dq, dv and dk in turn with the products
// of gla_tile_kernel (same roles, same operand maps) from one copy of the rows: 48 KB read and 24 KB written per
// (tile, head) instead of 3 x 41 KB moved by three launches, and the tile states are read as 16-byte pieces and
// transposed on their way out of LDS instead of by 2-byte requests to memory.  The rows W of the two dot
// products (q for q.dq, k for k.dk) come from the same tiles.
struct GlaBwdTileArgs {
  ChunkArgs c;                  // T, H, tiles, gate (gt, g), scale, dk, dv
  const void *q, *k, *v, *d_o;  // rows [token][H][dv] (v, dO), [token][Hq][dk] (q, k: c.Hq heads)
  const bf16_t *S, *G;          // tile-start states and gradients of the tile-end states, [tile][H][dv][dk]
  void *dq, *dk, *dv;
  float *qdq, *kdk;             // [H][tokens]
  int64_t n_tokens;
};

constexpr int kFR = 80;   // row stride (bf16) of the row and state tiles of the fused kernel (rows of up to 64 entries):
                          // 16-byte reads by lanes (row i, piece g) are free of bank conflicts when the rows are
                          // 32 bytes more than a multiple of 64 bytes apart (measured; 144-byte rows cost twice the time)
constexpr int kFZ = 68;   // row stride (bf16) of its transposed tile and of its output tile: both are accessed in 8-byte
                          // pieces by 16 lanes on 16 rows at a time, which 34 words per row spread over the 32 banks
// Place of entry (row, col) in a state tile.  The tile is read along its rows (16-byte pieces) by one role and along
// its columns (2-byte pieces, eight rows apart between the lane groups) by the others; eight rows are a multiple of
// the 32 LDS banks apart, so the groups of 16 columns are exchanged between the groups of eight rows.
constexpr int kFS = 72;   // row stride (bf16) of the state tiles (read along rows by one role only; 80 would not leave room for
                          // two workgroups per compute unit)
__device__ __forceinline__ int state_tile_at(int row, int col) { return row * kFS + (col ^ (((row >> 3) & 3) << 4)); }

// Eight waves per workgroup (four per SIMD with two workgroups on a compute unit): a role's scores are formed by two
// waves per token block (one per half of the score operand), its output by two waves per block of 16 columns (token
// blocks {0, 2} and {1, 3}: the same number of matrix instructions in both causal directions).
// DKC, DVC: the head dims when they are known at compile time (loops unrolled, index arithmetic folded), else 0.
template <typename TIn, int DKC, int DVC>
__global__ __launch_bounds__(512, 4) void gla_bwd_tile_kernel(GlaBwdTileArgs A) {
  static_assert(sizeof(TIn) == 2, "bf16 rows");
  extern __shared__ float smem[];
  const ChunkArgs& a = A.c;
  const int H = a.H, dk = DKC ? DKC : a.dk, dv = DVC ? DVC : a.dv;
  float* sC = smem;                          // [64] running log2 decay inside the tile
  float* sDot = sC + kC;                     // [8][64] partial dot products of the waves
  bf16_t* sQ = (bf16_t*)(sDot + 8 * kC);     // row tiles [64 tokens][kFR], zero beyond the tile's tokens and widths
  bf16_t* sK = sQ + kC * kFR;
  bf16_t* sV = sK + kC * kFR;
  bf16_t* sDo = sV + kC * kFR;
  bf16_t* sS = sDo + kC * kFR;               // state tiles [64 value rows][kFS], zero beyond dv x dk
  bf16_t* sG = sS + kC * kFS;
  bf16_t* sZT = sG + kC * kFS;               // [64 columns][kFZ]: the mixed rows of the current role, token index fastest
  bf16x8* sP = (bf16x8*)(sZT + kC * kFZ);    // [4 token blocks][2][64 lanes] score operands; then the output tile [64][kFZ]
  TIn* sOut = (TIn*)sP;
  const int tid = threadIdx.x, lane = tid & 63, i = lane & 15, g = lane >> 4;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  // A workgroup walks over (tile, head) items; the rows and states of the next item are requested into registers
  // before the products of the current one start, so that their latency is covered by that work.
  // Waves 0-3: tokens 2 sp, 2 sp + 1, columns [8 c8, 8 c8 + 8) of q and k and two rows of S; waves 4-7: of v, dO and G.
  const int sp = (tid & 255) >> 3, c8 = tid & 7;
  const bool upper = w >= 4;
  const int64_t n_items = (int64_t)a.total_chunks * H;
  bf16x8 ra[2], rb[2], rc[2];
  unsigned gate_n = 0u;   // the token's gate as stored (wave 0)
  float gh_n = 0.f;       // the head's decay rate g (wave 0)
  // (tile, head) of an item and the tile's place in the token axis.  With a tile table the two words are requested
  // one item before they are needed (meta_request) and range-checked when they are (meta_finish, as chunk_lookup).
  struct Meta { int cidx, h, t0, clen; };
  // A load from an address that is the same in every lane is turned into a scalar value right behind the load, which
  // makes the wave wait for it there (and for every request issued before it).  The loads that are meant to stay in
  // flight get an offset of zero that the compiler cannot see through; their values are made scalar where they are used.
  int lane_zero = 0;
  asm volatile("" : "+v"(lane_zero));
  int tab_t0 = 0, tab_clen = 0;   // words of the tile table for the item after the next (written by loads only)
  int cidx_nn = 0, h_nn = 0;
  auto meta_request = [&](int64_t item) {
    // the item is the same for every lane
    cidx_nn = __builtin_amdgcn_readfirstlane((int)(item / H));
    h_nn = __builtin_amdgcn_readfirstlane((int)(item - (int64_t)cidx_nn * H));
    if (a.chunk_table) {
      const int32_t* row = a.chunk_table + 4 * (int64_t)cidx_nn;
      tab_t0 = row[1 + lane_zero];
      tab_clen = row[2 + lane_zero];
    }
  };
  auto meta_finish = [&](Meta& m) {
    m.cidx = cidx_nn;
    m.h = h_nn;
    if (a.chunk_table) {
      m.t0 = min(max(__builtin_amdgcn_readfirstlane(tab_t0), 0), a.T - 1);
      m.clen = min(max(__builtin_amdgcn_readfirstlane(tab_clen), 0), min(kC, a.T - m.t0));
    } else {
      const int per = (a.T + kC - 1) / kC;
      const int seq = m.cidx / per, cis = m.cidx - seq * per;
      m.t0 = seq * a.T + cis * kC;
      m.clen = min(kC, a.T - cis * kC);
    }
  };
  auto request = [&](const Meta& m) {
    const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
    const TIn* pa = (const TIn*)(upper ? A.v : A.q);
    const TIn* pb = (const TIn*)(upper ? A.d_o : A.k);
    const bf16_t* pc = upper ? A.G : A.S;
    const int d = upper ? dv : dk;
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int s = 2 * sp + u;
      const bool on = s < m.clen && 8 * c8 < d;
      // q and k may carry fewer heads than v and dO (a group of value heads shares one)
      const int hn = upper ? H : a.Hq, hh = upper ? m.h : m.h / (H / a.Hq);
      const int64_t row = ((int64_t)(m.t0 + (on ? s : 0)) * hn + hh) * d + (on ? 8 * c8 : 0);
      ra[u] = on ? *(const bf16x8*)(pa + row) : zero;
      rb[u] = on ? *(const bf16x8*)(pb + row) : zero;
      const bool ons = s < dv && 8 * c8 < dk;
      const int64_t so = ((int64_t)m.cidx * H + m.h) * dv * dk + (int64_t)(ons ? s : 0) * dk + (ons ? 8 * c8 : 0);
      rc[u] = ons ? *(const bf16x8*)(pc + so) : zero;
    }
    if (w == 0) {
      if (lane < m.clen) gate_n = load_gate_word(a.gt, (int64_t)(m.t0 + lane) * H + m.h, a.gate_bf16);
      gh_n = a.g[m.h + lane_zero];
    }
  };
  int64_t item = blockIdx.x;
  const int64_t stride = gridDim.x;
  if (item >= n_items) return;
  Meta m_next;
  meta_request(item);
  meta_finish(m_next);
  request(m_next);
  if (item + stride < n_items) meta_request(item + stride);
  for (;;) {
  // the requested item becomes the current one: its tiles go to LDS (every read of the previous item's is behind a barrier)
  const int h = m_next.h, t0 = m_next.t0, clen = m_next.clen;
  if (w == 0) {
    const float gt = (lane < clen) ? gate_value(gate_n, (int64_t)(t0 + lane) * H + h, a.gate_bf16) : 0.f;
    sC[lane] = wave_inclusive_scan(-gt * (gh_n * kLog2e), lane);
  }
  {
    bf16_t* ta = upper ? sV : sQ;
    bf16_t* tb = upper ? sDo : sK;
    bf16_t* tc = upper ? sG : sS;
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int o = (2 * sp + u) * kFR + 8 * c8;
      *(bf16x8*)&ta[o] = ra[u];
      *(bf16x8*)&tb[o] = rb[u];
      *(bf16x8*)&tc[state_tile_at(2 * sp + u, 8 * c8)] = rc[u];
    }
    if (!upper) {   // first role (dq) mixes the rows of k: token pair sp, one 32-bit word per column
#pragma unroll
      for (int e = 0; e < 8; ++e) *(bf16x2*)&sZT[(8 * c8 + e) * kFZ + 2 * sp] = bf16x2{rb[0][e], rb[1][e]};
    }
  }
  __syncthreads();
  const bool more = item + stride < n_items;
  if (more) {
    meta_finish(m_next);
    request(m_next);
    if (item + 2 * stride < n_items) meta_request(item + 2 * stride);
  }

  const float scale = a.scale;
  // One role of gla_tile_kernel on the tiles in LDS.  sX, sY: rows of the scores (width dc); sSt: state tile read
  // straight (rows = output columns) or transposed; sW: rows of the dot product or null; zn: rows the NEXT role mixes.
  auto role = [&](auto rev_c, auto st_c, const bf16_t* sX, const bf16_t* sY, const bf16_t* sSt, const bf16_t* sW,
                  const bf16_t* zn, int dc, int de, void* out, float* dot_out) {
    constexpr bool REVERSE = decltype(rev_c)::value, STATE_T = decltype(st_c)::value;
    const int KS = (dc + 31) >> 5, n_eb = de >> 4;
    auto x_operand = [&](int xb, int ks) { return *(const bf16x8*)(sX + (16 * xb + i) * kFR + 8 * g + 32 * ks); };
    // ---- scores of token block w / 2 against the blocks yb = 2 p + (w & 1) on its causal side: one half of each of
    //      the block's two score operands
    {
      const int tb = w >> 1, half = w & 1;
      f32x4 accS[2];
#pragma unroll
      for (int p = 0; p < 2; ++p) accS[p] = f32x4{0.f, 0.f, 0.f, 0.f};
      for (int ks = 0; ks < KS; ++ks) {
        const bf16x8 Xo = x_operand(tb, ks);
#pragma unroll
        for (int p = 0; p < 2; ++p) {
          const int yb = 2 * p + half;
          if (REVERSE ? yb >= tb : yb <= tb)
            accS[p] = mfma16(*(const bf16x8*)(sY + (16 * yb + i) * kFR + 8 * g + 32 * ks), Xo, accS[p]);
        }
      }
      const float cx = sC[16 * tb + i];
#pragma unroll
      for (int p = 0; p < 2; ++p) {
        const int yb = 2 * p + half;
        const f32x4 cy = *(const f32x4*)&sC[16 * yb + 4 * g];
        float val[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const bool side = REVERSE ? yb >= tb : yb <= tb;
          const bool live = side && (yb != tb || (REVERSE ? 4 * g + r >= i : 4 * g + r <= i));
          val[r] = live ? accS[p][r] * fast_exp2(REVERSE ? cy[r] - cx : cx - cy[r]) : 0.f;
        }
        store_vec<4>((bf16_t*)&sP[(tb * 2 + p) * 64 + lane] + 4 * half, val);
      }
    }
    __syncthreads();
    // ---- output columns [16 (w / 2), 16 (w / 2) + 16) for the token blocks xh, xh + 2 (xh = w & 1)
    const int eb = min(w >> 1, n_eb - 1);          // a wave past the last block repeats it (not stored)
    const bool valid = (w >> 1) < n_eb;
    const int xh = w & 1;
    f32x4 acc[2];
#pragma unroll
    for (int u = 0; u < 2; ++u) acc[u] = f32x4{0.f, 0.f, 0.f, 0.f};
    for (int ks = 0; ks < KS; ++ks) {
      bf16x8 Sa;
      if constexpr (STATE_T) {
#pragma unroll
        for (int j = 0; j < 8; ++j) Sa[j] = sSt[state_tile_at(32 * ks + 8 * g + j, 16 * eb + i)];
      } else {
        Sa = *(const bf16x8*)(sSt + state_tile_at(16 * eb + i, 32 * ks + 8 * g));
      }
#pragma unroll
      for (int u = 0; u < 2; ++u) acc[u] = mfma16(Sa, x_operand(xh + 2 * u, ks), acc[u]);
    }
    const bf16_t* zrow = sZT + (16 * eb + i) * kFZ + 4 * g;
    bf16x8 Za[2];
#pragma unroll
    for (int p = 0; p < 2; ++p) {
      const bf16x4 lo = *(const bf16x4*)(zrow + 32 * p), hi = *(const bf16x4*)(zrow + 32 * p + 16);
      Za[p] = bf16x8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    }
    float dot[2] = {0.f, 0.f};
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int xb = xh + 2 * u;
      const float cx = sC[16 * xb + i];
      const float wx = fast_exp2(REVERSE ? sC[kC - 1] - cx : cx);
#pragma unroll
      for (int r = 0; r < 4; ++r) acc[u][r] *= wx;
#pragma unroll
      for (int p = 0; p < 2; ++p)
        if ((REVERSE ? 2 * p + 1 >= xb : 2 * p <= xb)) acc[u] = mfma16(Za[p], sP[(xb * 2 + p) * 64 + lane], acc[u]);
#pragma unroll
      for (int r = 0; r < 4; ++r) acc[u][r] *= scale;
      if (sW && valid) {
        const bf16x4 wv = *(const bf16x4*)(sW + (16 * xb + i) * kFR + 16 * eb + 4 * g);
#pragma unroll
        for (int r = 0; r < 4; ++r) dot[u] = fmaf((float)wv[r], acc[u][r], dot[u]);
      }
    }
    __syncthreads();   // every wave has its scores and mixed rows: the two areas are free
    if (sW) {
      // lanes of row g get the sum over the four rows of argument g: token block g of this wave, or zero
      const float d0 = dot[0], d1 = dot[1];
      sDot[w * kC + lane] = rows4_sum_x4(xh ? 0.f : d0, xh ? d0 : 0.f, xh ? 0.f : d1, xh ? d1 : 0.f);   // lane = token
    }
    if (valid) {
#pragma unroll
      for (int u = 0; u < 2; ++u)
        store_vec<4>(sOut + (16 * (xh + 2 * u) + i) * kFZ + 16 * eb + 4 * g, (const float*)&acc[u]);
    }
    if (zn) {
      // token pair zp, columns [8 zc + 4 ze, 8 zc + 4 ze + 4) of the next role's mixed rows
      const int zp = tid >> 4, zc = (tid >> 1) & 7, ze = tid & 1;
      const bf16x4 z0 = *(const bf16x4*)(zn + (2 * zp) * kFR + 8 * zc + 4 * ze);
      const bf16x4 z1 = *(const bf16x4*)(zn + (2 * zp + 1) * kFR + 8 * zc + 4 * ze);
#pragma unroll
      for (int e = 0; e < 4; ++e) *(bf16x2*)&sZT[(8 * zc + 4 * ze + e) * kFZ + 2 * zp] = bf16x2{z0[e], z1[e]};
    }
    __syncthreads();
    if (sW && w == 0 && lane < clen) {
      float tot = 0.f;
#pragma unroll
      for (int x = 0; x < 8; ++x) tot += sDot[x * kC + lane];
      dot_out[(int64_t)h * A.n_tokens + t0 + lane] = tot;
    }
    {
      const int per_row = de >> 3;
      TIn* obase = (TIn*)out + ((int64_t)t0 * H + h) * de;
      for (int idx = tid; idx < clen * per_row; idx += 512) {
        const int x = idx / per_row, c = idx - x * per_row;
        const bf16x4 lo = *(const bf16x4*)(sOut + x * kFZ + 8 * c), hi = *(const bf16x4*)(sOut + x * kFZ + 8 * c + 4);
        *(bf16x8*)(obase + (int64_t)x * H * de + 8 * c) = bf16x8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
      }
    }
    __syncthreads();   // the output tile has been read: the next role may write its scores
  };
  using T_ = std::true_type;
  using F_ = std::false_type;
  // dq: X = dO, Y = v, mixes k, tile-start state transposed, q . dq on the side; then the rows of dO for dv
  role(F_{}, T_{}, sDo, sV, sS, sQ, sDo, dv, dk, A.dq, A.qdq);
  // dv: X = k, Y = q, mixes dO, gradient of the tile-end state, reverse; then the rows of q for dk
  role(T_{}, F_{}, sK, sQ, sG, (const bf16_t*)nullptr, sQ, dk, dv, A.dv, (float*)nullptr);
  // dk: X = v, Y = dO, mixes q, gradient of the tile-end state transposed, reverse, k . dk on the side
  role(T_{}, T_{}, sV, sDo, sG, sK, (const bf16_t*)nullptr, dv, dk, A.dk, A.kdk);
  if (!more) break;
  item += stride;
  }
}

static bool gla_bwd_tile_applies(const PalDims* d) {
  return d->dtype == PAL_DTYPE_BF16 && d->dk <= 64 && d->dv <= 64;
}

static int launch_gla_bwd_tile(const GlaBwdTileArgs& A, hipStream_t s) {
  const size_t lds = sizeof(float) * (kC + 8 * kC) + sizeof(bf16_t) * (size_t)kC * (4 * kFR + 2 * kFS + kFZ + 72);
  const int64_t items = (int64_t)A.c.total_chunks * A.c.H;
  int dev = 0, cus = 0;
  if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess ||
      cus <= 0)
    cus = 256;
  const int64_t resident = 2 * (int64_t)cus;   // two workgroups per compute unit, each walks its items
  const int64_t blocks = items < resident ? items : resident;
  if (A.c.dk == 64 && A.c.dv == 64) {
    if (int rc = allow_lds((const void*)&gla_bwd_tile_kernel<bf16_t, 64, 64>, lds)) return rc;
    PAL_TIMED_LAUNCH(kKernGlaBwdTile, s, (gla_bwd_tile_kernel<bf16_t, 64, 64>), dim3((unsigned)blocks), dim3(512), lds, s, A);
  } else {
    if (int rc = allow_lds((const void*)&gla_bwd_tile_kernel<bf16_t, 0, 0>, lds)) return rc;
    PAL_TIMED_LAUNCH(kKernGlaBwdTile, s, (gla_bwd_tile_kernel<bf16_t, 0, 0>), dim3((unsigned)blocks), dim3(512), lds, s, A);
  }
  PAL_HIP_LAUNCH_CHECK();
  return PAL_OK;
}

// argument checks shared by the forward and the backward entry points
static int check_gla(const PalDims* d, const PalFwdTensors* t) {
  int rc = pal_validate_dims(d);
  if (rc) return rc;
  if (!t) return PAL_E_NULL;
  if (!t->q || !t->k || !t->v || !t->gt || !t->g || !t->o || !t->chunk_I) return PAL_E_NULL;
  if (d->flags & PAL_FLAG_HAS_VAR) return PAL_E_STATE;   // no precision state, no output variance
  if (d->flags & PAL_FLAG_STATE_MU_BF16) return PAL_E_STATE;
  if (((d->flags & PAL_FLAG_HAS_INIT) != 0) != (t->init_mu != nullptr)) return PAL_E_STATE;
  if (((d->flags & PAL_FLAG_STORE_FINAL) != 0) != (t->final_mu != nullptr)) return PAL_E_STATE;
  const bool varlen = d->flags & PAL_FLAG_VARLEN;
  if (varlen != (t->cu_seqlens != nullptr)) return PAL_E_CU_SEQLENS;
  if (varlen && (!t->chunk_table || !t->chunk_offsets)) return PAL_E_NULL;
  if (d->total_chunks <= 0) return PAL_E_CHUNK;
  const int64_t per = ((int64_t)d->seq_len + PAL_CHUNK - 1) / PAL_CHUNK;
  if (varlen) {
    if (d->total_chunks < per || d->total_chunks > (int64_t)d->seq_len / PAL_CHUNK + d->n_seqs) return PAL_E_CHUNK;
  } else if ((int64_t)d->total_chunks != per * d->batch) {
    return PAL_E_CHUNK;
  }
  const void* ptrs[] = {t->q, t->k, t->v, t->o, t->init_mu, t->final_mu, t->chunk_mu, t->chunk_I};
  for (const void* p : ptrs)
    if (p && !is_aligned16(p)) return PAL_E_ALIGN;
  if (!is_aligned4(t->gt)) return PAL_E_ALIGN;   // gates are fetched as the aligned 32-bit word that holds them
  return PAL_OK;
}

// the shared argument block carries no precision tensors on this path
static void fill_gla_args(ChunkArgs& a, const PalDims* d, const PalFwdTensors* t) {
  PalFwdTensors tt = *t;
  tt.b = nullptr; tt.Ip = nullptr; tt.o_var = nullptr;
  tt.init_I = nullptr; tt.final_I = nullptr;
  fill_chunk_args(a, d, &tt);
}

// ------------------------------------------------------------------ backward
// Gradient of the state at the END of every tile, G_c = F_{c+1} G_{c+1} + D_{c+1}, from the tiles' own
// contributions D_c = sum_t F_t dO_t q_t^T parked in buf by chunk_delta_kernel: the forward scan run
// backwards.  One thread per (sequence, head, state entry); slot c of g_tiles gets G_c in bf16 (the running
// value stays fp32).  What is left after the first tile, times scale, is the gradient of the initial state.
__global__ __launch_bounds__(256) void gla_bwd_scan_kernel(ChunkArgs a, const float* buf, bf16_t* g_tiles, float* d_init) {
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
  f32x4 G = {0.f, 0.f, 0.f, 0.f};
  for (int c_hi = nchunks; c_hi > 0; c_hi -= kScanTiles) {
    const int c0 = max(0, c_hi - kScanTiles), cn = c_hi - c0;
    __syncthreads();
    for (int c = w; c < cn; c += 4) {
      const int t = (c0 + c) * kC + lane;
      const float gt = (t < len) ? load_gate(a.gt, (int64_t)(bos + t) * a.H + h, a.gate_bf16) : 0.f;
      const float tot = wave_sum(-gt * gh);
      if (lane == 0) sF[c] = fast_exp2(tot);
    }
    __syncthreads();
    if (!on) continue;
    int c = cn;
    for (; c >= 4; c -= 4) {
      f32x4 D[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) D[u] = *(const f32x4*)(buf + ((int64_t)(cbase + c0 + c - 1 - u) * a.H + h) * E + e);
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        store_vec<4>(g_tiles + ((int64_t)(cbase + c0 + c - 1 - u) * a.H + h) * E + e, (const float*)&G);
        const float F = sF[c - 1 - u];
#pragma unroll
        for (int x = 0; x < 4; ++x) G[x] = fmaf(F, G[x], D[u][x]);
      }
    }
    for (; c >= 1; --c) {
      const int64_t off = ((int64_t)(cbase + c0 + c - 1) * a.H + h) * E + e;
      const f32x4 D = *(const f32x4*)(buf + off);
      store_vec<4>(g_tiles + off, (const float*)&G);
      const float F = sF[c - 1];
#pragma unroll
      for (int x = 0; x < 4; ++x) G[x] = fmaf(F, G[x], D[x]);
    }
  }
  if (d_init && on) {
    const f32x4 r = {a.scale * G[0], a.scale * G[1], a.scale * G[2], a.scale * G[3]};
    *(f32x4*)(d_init + (int64_t)nh * E + e) = r;
  }
}

// Gate gradients.  With C_t the running sum of the log decay l_t = -gt_t g over a sequence, q_t enters
// the output only as q_t e^{C_t} and k_t only as k_t e^{-C_t}, so dC_t = q_t . dq_t - k_t . dk_t (the two
// dot products come from the dq and dk kernels in fp32) and dl_t is the sum of dC over the tokens from t
// to the end of the sequence.  One workgroup per (sequence, head) walks the sequence from its end in
// pieces of 1024 tokens: four consecutive tokens per thread, a suffix scan over the lanes of each wave,
// the four wave totals through LDS.  dgt_t = -g dl_t, and the workgroup's share of
// dg = -sum_t gt_t dl_t goes to dg_part[seq][head].
constexpr int kGateTok = 4;                    // consecutive tokens per thread
constexpr int kGatePiece = 256 * kGateTok;     // tokens per step of a workgroup

__global__ __launch_bounds__(256) void gla_bwd_gate_kernel(ChunkArgs a, const float* qdq, const float* kdk, float* dgt,
                                                           float* dg_part, int64_t n_tokens) {
  __shared__ float sTot[2][4];
  __shared__ float sAcc[4];
  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  const int h = blockIdx.x % a.H, n = blockIdx.x / a.H;
  int bos, len, cbase;
  seq_lookup(a, n, bos, len, cbase);
  const float gh = a.g[h];
  float carry = 0.f, acc = 0.f;
  int it = 0;
  for (int base = ((len - 1) / kGatePiece) * kGatePiece; base >= 0; base -= kGatePiece, ++it) {
    const int tf = base + kGateTok * tid;
    float x[kGateTok];
#pragma unroll
    for (int j = 0; j < kGateTok; ++j) {
      const int64_t off = (int64_t)h * n_tokens + bos + tf + j;      // the dot products are stored head-major
      x[j] = (tf + j < len) ? qdq[off] - kdk[off] : 0.f;
    }
    // suffix sums inside the thread, then over the lanes of the wave (exclusive of the thread itself)
#pragma unroll
    for (int j = kGateTok - 2; j >= 0; --j) x[j] += x[j + 1];
    float s = x[0];
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      const float y = __shfl_down(s, d);
      if (lane + d < 64) s += y;
    }
    const float wave_tot = __shfl(s, 0);
    const float after = s - x[0];             // tokens of later lanes of this wave
    if (lane == 0) sTot[it & 1][w] = wave_tot;
    __syncthreads();
    float later = carry, piece = 0.f;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const float tu = sTot[it & 1][u];
      piece += tu;
      if (u > w) later += tu;
    }
    carry += piece;
#pragma unroll
    for (int j = 0; j < kGateTok; ++j) {
      if (tf + j < len) {
        const int64_t off = (int64_t)(bos + tf + j) * a.H + h;
        const float dl = x[j] + after + later;
        dgt[off] = -gh * dl;
        acc = fmaf(load_gate(a.gt, off, a.gate_bf16), dl, acc);
      }
    }
  }
  acc = wave_sum(acc);
  if (lane == 0) sAcc[w] = acc;
  __syncthreads();
  if (tid == 0) dg_part[(int64_t)n * a.H + h] = -(sAcc[0] + sAcc[1] + sAcc[2] + sAcc[3]);
}

// dg[h] = sum over the sequences, in a fixed order
__global__ void gla_bwd_head_reduce_kernel(const float* dg_part, float* dg, int n_seqs, int H) {
  const int h = blockIdx.x * blockDim.x + threadIdx.x;
  if (h >= H) return;
  float s = 0.f;
  for (int n = 0; n < n_seqs; ++n) s += dg_part[(int64_t)n * H + h];
  dg[h] = s;
}

// workspace of the backward: per-tile contributions D (fp32), G tiles (bf16), the two dot-product rows,
// per-sequence shares of dg
struct GlaBwdWorkspace {
  size_t d_tiles, g_tiles, qdq, kdk, dg_part, dq_full, dk_full, total;
};
static GlaBwdWorkspace gla_bwd_layout(const PalDims* d) {
  auto up = [](size_t x) { return (x + 255) & ~(size_t)255; };
  GlaBwdWorkspace w;
  const size_t tokens = (size_t)d->batch * d->seq_len;
  const size_t entries = (size_t)d->total_chunks * d->n_heads * d->dv * d->dk;
  w.d_tiles = 0;
  w.g_tiles = w.d_tiles + up(sizeof(float) * entries);
  w.qdq = w.g_tiles + up(sizeof(bf16_t) * entries);
  w.kdk = w.qdq + up(sizeof(float) * tokens * d->n_heads);
  w.dg_part = w.kdk + up(sizeof(float) * tokens * d->n_heads);
  w.total = w.dg_part + up(sizeof(float) * (size_t)d->n_seqs * d->n_heads);
  w.dq_full = w.dk_full = w.total;
  if (d->n_qk_heads > 0 && d->n_qk_heads != d->n_heads) {   // one dq, dk row per value head, summed per group at the end
    const size_t full = up(tokens * d->n_heads * d->dk * (d->dtype == PAL_DTYPE_BF16 ? 2 : 4));
    w.dk_full = w.dq_full + full;
    w.total = w.dk_full + full;
  }
  return w;
}

}  // namespace pal

extern "C" size_t pal_gla_chunk_bwd_workspace_bytes(const PalDims* d) {
  if (pal_validate_dims(d) != PAL_OK || d->total_chunks <= 0) return 0;
  return pal::gla_bwd_layout(d).total;
}

extern "C" int pal_gla_chunk_bwd(const PalDims* d, const PalFwdTensors* t, const PalBwdTensors* gr, void* workspace,
                                 size_t workspace_bytes, void* stream) {
  using namespace pal;
  if (int rc = check_gla(d, t)) return rc;
  if (!gr) return PAL_E_NULL;
  if (!gr->d_o || !gr->dq || !gr->dk || !gr->dv || !gr->dgt || !gr->dg) return PAL_E_NULL;
  if (gr->d_init_mu && !(d->flags & PAL_FLAG_HAS_INIT)) return PAL_E_STATE;
  const void* ptrs[] = {gr->d_o, gr->dq, gr->dk, gr->dv, gr->d_init_mu, workspace};
  for (const void* p : ptrs)
    if (p && !is_aligned16(p)) return PAL_E_ALIGN;
  const GlaBwdWorkspace w = gla_bwd_layout(d);
  if (!workspace || workspace_bytes < w.total) return PAL_E_WORKSPACE;
  char* ws = (char*)workspace;
  float* d_tiles = (float*)(ws + w.d_tiles);
  bf16_t* g_tiles = (bf16_t*)(ws + w.g_tiles);
  float* qdq = (float*)(ws + w.qdq);
  float* kdk = (float*)(ws + w.kdk);
  float* dg_part = (float*)(ws + w.dg_part);
  hipStream_t s = (hipStream_t)stream;

  ChunkArgs a;
  fill_gla_args(a, d, t);
  a.final_mu = nullptr;
  // shared q/k heads: the kernels leave one dq, dk row per value head in the workspace; they are summed over each
  // group in a fixed order at the end (the gate terms q.dq, k.dk are per value head anyway)
  const bool grouped = a.Hq != a.H;
  void* dq_out = grouped ? (void*)(ws + w.dq_full) : gr->dq;
  void* dk_out = grouped ? (void*)(ws + w.dk_full) : gr->dk;
  // D_c = sum_t F_t dO_t q_t^T per tile, then the reverse scan over the tiles of each sequence
  {
    ChunkArgs b = a;
    b.k = t->q; b.v = gr->d_o; b.chunk_mu = d_tiles; b.flags |= kFlagDecayFromStart;
    if (state_pass_applies(b, d->dtype, false)) {
      if (int rc = launch_state_pass(b, false, g_tiles, nullptr, nullptr, nullptr, gr->d_init_mu, nullptr, true, a.scale,
                                     kKernGlaBwdStates, s))
        return rc;
    } else {
    if (int rc = launch_tile_delta(b, d->dtype, false, s)) return rc;
    const int64_t blocks = (int64_t)d->n_seqs * d->n_heads * (((int64_t)d->dv * d->dk + 1023) / 1024);
    if (blocks > 0x7fffffff) return PAL_E_DIM;
    PAL_TIMED_LAUNCH(kKernGlaBwdScan, s, gla_bwd_scan_kernel, dim3((unsigned)blocks), dim3(256), 0, s, a, d_tiles,
                     g_tiles, gr->d_init_mu);
    PAL_HIP_LAUNCH_CHECK();
    }
  }
  if (gla_bwd_tile_applies(d)) {
    GlaBwdTileArgs F{};
    F.c = a;
    F.q = t->q; F.k = t->k; F.v = t->v; F.d_o = gr->d_o;
    F.S = (const bf16_t*)t->chunk_I; F.G = g_tiles;
    F.dq = dq_out; F.dk = dk_out; F.dv = gr->dv; F.qdq = qdq; F.kdk = kdk;
    F.n_tokens = (int64_t)d->batch * d->seq_len;
    if (int rc = launch_gla_bwd_tile(F, s)) return rc;
  } else {
  GlaTileArgs A{};
  A.c = a;
  A.n_tokens = (int64_t)d->batch * d->seq_len;
  // dq: X = dO, Y = v, Z = k, tile-start states read transposed; q . dq on the side
  A.X = gr->d_o; A.Y = t->v; A.Z = t->k; A.St = (const bf16_t*)t->chunk_I; A.out = dq_out; A.W = t->q; A.dot = qdq;
  A.dc = d->dv; A.de = d->dk;
  A.hX = a.H; A.hY = a.H; A.hZ = a.Hq; A.hW = a.Hq;
  if (int rc = launch_gla_tile_dt(A, d->dtype, kGlaDq, s)) return rc;
  // dv: X = k, Y = q, Z = dO, tile-end state gradients
  A.X = t->k; A.Y = t->q; A.Z = gr->d_o; A.St = g_tiles; A.out = gr->dv; A.W = nullptr; A.dot = nullptr;
  A.dc = d->dk; A.de = d->dv;
  A.hX = a.Hq; A.hY = a.Hq; A.hZ = a.H; A.hW = a.H;
  if (int rc = launch_gla_tile_dt(A, d->dtype, kGlaDv, s)) return rc;
  // dk: X = v, Y = dO, Z = q, tile-end state gradients read transposed; k . dk on the side
  A.X = t->v; A.Y = gr->d_o; A.Z = t->q; A.St = g_tiles; A.out = dk_out; A.W = t->k; A.dot = kdk;
  A.dc = d->dv; A.de = d->dk;
  A.hX = a.H; A.hY = a.H; A.hZ = a.Hq; A.hW = a.Hq;
  if (int rc = launch_gla_tile_dt(A, d->dtype, kGlaDk, s)) return rc;
  }
  {
    const int64_t blocks = (int64_t)d->n_seqs * d->n_heads;
    PAL_TIMED_LAUNCH(kKernGlaBwdGate, s, gla_bwd_gate_kernel, dim3((unsigned)blocks), dim3(256), 0, s, a, qdq, kdk, gr->dgt,
                     dg_part, (int64_t)d->batch * d->seq_len);
    PAL_HIP_LAUNCH_CHECK();
    hipLaunchKernelGGL(gla_bwd_head_reduce_kernel, dim3((d->n_heads + 63) / 64), dim3(64), 0, s, dg_part, gr->dg,
                       d->n_seqs, d->n_heads);
    PAL_HIP_LAUNCH_CHECK();
  }
  if (grouped) {
    if (int rc = launch_group_sum(dq_out, dk_out, gr->dq, gr->dk, (int64_t)d->batch * d->seq_len, a.Hq, a.H / a.Hq, d->dk,
                                  d->dtype, s))
      return rc;
  }
  return PAL_OK;
}

extern "C" int pal_gla_chunk_fwd(const PalDims* d, const PalFwdTensors* t, void* stream) {
  using namespace pal;
  if (int rc = check_gla(d, t)) return rc;
  ChunkArgs a;
  fill_gla_args(a, d, t);
  // the fp32 scratch is only used by the two-kernel form of the tile-start states
  if (!t->chunk_mu && !state_pass_applies(a, d->dtype, false)) return PAL_E_NULL;
  hipStream_t s = (hipStream_t)stream;
  if (int rc = launch_tile_states(a, d->dtype, false, s)) return rc;
  GlaTileArgs A{};
  A.c = a;
  A.X = t->q; A.Y = t->k; A.Z = t->v; A.St = (const bf16_t*)t->chunk_I; A.out = t->o;
  A.dc = d->dk; A.de = d->dv;
  A.hX = a.Hq; A.hY = a.Hq; A.hZ = a.H; A.hW = a.H;
  return launch_gla_tile_dt(A, d->dtype, kGlaOut, s);
}
