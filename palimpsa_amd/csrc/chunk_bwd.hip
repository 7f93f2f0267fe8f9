// Chunked Palimpsa backward.
//
// Replaces chunk_palimpsa_bwd_kernel and the host-side reductions of
// ChunkPalimpsa.backward (chunk_palimpsa_forgetting_scalar.py:239-434, :519-620).
//
// With G_t = scale do_t q_t^T, the per-token local gradients are
//   dMloc_t = G_t / I_t,  dJloc_t = -G_t M_t / I_t^2 (- scale dovar_t (q_t*q_t)^T / I_t^2)
// and the state gradients obey the reverse recurrence dM_s = dMloc_s + f_{s+1} dM_{s+1}
// (:360-384).  All tiles of 64 tokens are processed in parallel; what crosses a
// tile boundary is handled by two small extra passes (scan, apply); the gate gradient is finished in the second:
//
//  local   per (tile, head): recompute M_t, I_t from the tile-start state (as the
//          forward does), form dMloc/dJloc, dq; feed them straight from the MFMA
//          accumulators into the reverse contraction dM^loc = L^T dMloc (k index =
//          token, so accumulator registers are already in operand layout); from it
//          the tile-local parts of dv, db, dk and the carry the tile hands to its
//          predecessor, R_loc = f_first * dM^loc_first.
//  scan    per state entry: R_{c-1} = R_loc,c + F_C,c R_c backwards over the tiles
//          of a sequence (the role of curr_dM/curr_dI, :429-430); also yields the
//          gradients of the initial state.
//  apply   per (tile, head): adds the carry terms a_s R k_s etc. to dv, db, dk
//          with four small MFMA products.
//  gate    d log f_s = <dM_s, f_s M_{s-1}> + <dJ_s, f_s J_{s-1}>, evaluated without any
//          cancellation (the reference un-shifts the state by dividing by f, :409-412):
//            local part   gamma_s = <dM^loc_s, S_s> + <dJ^loc_s, S^J_s>, S_s = f_s M_{s-1} from a
//                         strictly-lower-triangular MFMA product in the layout of dM^loc;
//            carry part   sum_{r<s, r in tile} beta_r + F_C (<R_M, M_0> + <R_J, J_0>), with
//                         beta_r = <v_r, dv^carry_r> + <b_r, db^carry_r> from the apply pass and
//                         (M_0, J_0) the state at the start of the tile.
//          dgt = -g dlogf, dg = -sum gt dlogf, dIp = sum dJloc (- sum dJ_0 with an initial state).
//          Every term belongs to the token's own tile: the apply kernel writes dgt and the tile's share of dg,
//          a last small kernel sums the shares per head.
#include <type_traits>

#include "chunk_common.h"
#include "pal_host.h"
#include "pal_profile.h"

namespace pal {

void fill_chunk_args(ChunkArgs& a, const PalDims* d, const PalFwdTensors* t);

struct BwdArgs {
  ChunkArgs c;
  const void *d_o, *d_o_var;
  void *dq, *dk, *dv, *db;
  float *dgt, *dg, *dIp, *d_init_mu, *d_init_I;
  void *wDM, *wDJ;        // [total_chunks,H,dv,dk] local carries, then incoming carries, in the dtype of the rows
  float* wFtot;           // [total_chunks,H] log2 of the total decay of a tile
  float* wSig;            // [total_chunks,H] sum over the tile of dJloc
  float* wE;              // [H, tokens]  local part of d log f
  float* wInitPart;       // [n_seqs,H,dv*dk/256] partial sums of dJ_0
  float* wDgTile;         // [total_chunks,H] the tiles' shares of dg
  int32_t tokens;
  int32_t apply_alias;     // carry apply: db^carry shares LDS with the bf16 carries (large head dims)
};

constexpr int kVS2 = 68;
// local pass: rows the consumers run behind the first producer (the second producer runs one row behind it)
constexpr int kLagC = 2;
// value rows staged at a time: 8 with two column blocks per workgroup, so that two such workgroups fit a compute unit's LDS
__host__ __device__ constexpr int local_dg(int NB, bool prec) { return (!prec && NB == 2) ? 8 : 16; }


// ------------------------------------------------- local pass, four wave roles
// One workgroup per (tile, head).  For every value row d the tile recomputes M_t, I_t for its 64 tokens
// (orientation [t, n]), forms dMloc/dJloc and dq, contracts them backwards in time (dM^loc[n, s]) and
// runs the dv/db/dk/gate epilogue on the result.
// Organised for four waves per SIMD: one wave issues a VALU instruction every 5-9 cycles at best while
// the SIMD can start one every 2-3, so the work on a block of 16 key columns is cut into four roles
// small enough for 128 registers each.  A workgroup has 4*NB waves; wave = role*NB + (column block).
//   roles 0/1 ("producers", tokens 0..31 / 32..63): recompute the states of one value row for 16 key
//     columns, form dMloc/dJloc and dq, and leave packed bf16 operands P^M, P^J (local gradients) and X^M, X^J
//     (rank-one updates) of their half of the tile in an LDS slot;
//   roles 2/3 ("consumers", column tokens s in 0..31 / 32..63): pick their half's slot up two iterations after the
//     first producer wrote its own and do the reverse contraction, the strictly-lower product and the
//     dv/db/dk/gate epilogue.
// Every role has its own loop (its own register allocation) with the same sequence of barriers.
// The tile is worked as two halves of 32 tokens coupled through LDS (see the producers).
// NB <= 4 column blocks are in flight at a time (16 waves); a wider head dim takes several passes over
// the tile, the later ones adding their dv/db/gate contributions to those of the earlier ones.
// PREC (fp32 rows): every operand is carried as two bf16 halves and every product takes three matrix instructions
// (split_bf16 / mfma16_split); the LDS slots hold twice the operands and a wave may use 256 registers
// (two waves per SIMD), so at most 2 column blocks are in flight.
// Three column blocks (dk = 48) are 12 waves, three per SIMD and one workgroup per compute unit (its LDS): that
// instance may use 168 registers.
template <typename TIn, int NB, bool HAS_VAR, bool MULTI, bool PREC>
__global__ __launch_bounds__(4 * NB * 64) __attribute__((amdgpu_waves_per_eu(PREC ? 2 : (NB == 3 ? 3 : 4))))
void chunk_bwd_local_roles_kernel(BwdArgs A) {
  const ChunkArgs& a = A.c;
  extern __shared__ float smem[];
  constexpr int NST = HAS_VAR ? 4 : 3;  // staged tensors: v, b, do, (dovar)
  constexpr int DG = local_dg(NB, PREC);   // value rows per staging group
  constexpr int STG = DG * kVS2;
  float* sC = smem;                      // [64] running log2 decay
  float* sF = sC + kC;                   // [64] decay from before the half of the tile: 2^c_t (t < 32), 2^(c_t - c_31)
  float* sSt = sF + kC;                  // [2][NST][DG][kVS2]
  float* sPv = sSt + 2 * NST * STG;      // [NB][DG][64] per-wave partial dv
  float* sPb = sPv + NB * DG * kC;       // [NB][DG][64] per-wave partial db
  // The second producer runs one value row behind the first (it takes the state after token 31 from it), the
  // consumers follow two rows behind.  The first producer's half of a slot is then alive for three rows, the second
  // one's for two:
  //   sX  [NB][3 x {P^M_0, P^J_0, X^M_0, X^J_0} | 2 x {P^M_1, P^J_1, X^M_1, X^J_1}][64 lanes]
  //       (PREC: each group of four is followed by its four lo halves),
  //   sMJ [NB][3 slots][M_0, J_0, M_31, J_31, what flows back over token 31 (M, J)][16]   (see the producers).
  float* sMJ = sPb + NB * DG * kC;
  constexpr int XS = PREC ? 2 : 1;
  bf16x8* sX = (bf16x8*)(sMJ + NB * 288);
  // [NB][DG rows][4][M 0..3, J 0..3] first column of dM^loc, dJ^loc of a group of value rows (the carry to the previous tile)
  float* sCar = (float*)(sX + NB * 20 * XS * 64);
  // [NB][64] d log f partials of the consumer waves, then [2 NB] sums of dJloc: written after the last row of a pass,
  // when the operand slots are dead, so they share their memory
  float* sRed = (float*)sX;
  const int tid = threadIdx.x;
  int lane = tid & 63, i = lane & 15, g = lane >> 4;   // re-derived per pass from an opaque copy, see below
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // wave-uniform: role branches are scalar
  const int role = wave / NB, nbl = wave - role * NB;   // nbl: column block inside the current group
  const int H = a.H, dk = a.dk, dv = a.dv;
  // NB blocks of 16 key columns are handled at a time; wider heads take several passes over the tile
  const int nb_total = dk >> 4, n_pass = MULTI ? (nb_total + NB - 1) / NB : 1;   // MULTI = false: dk == 16*NB
  const int cidx = blockIdx.x / H, h = blockIdx.x % H;
  int seq, t0, clen, cis;
  chunk_lookup(a, cidx, seq, t0, clen, cis);
  const float Ip = a.Ip[h];
  const float gh = a.g[h] * kLog2e;
  const float scale = a.scale;
  const bool fold = !PREC && a.init_mu == nullptr;

  if (wave == 0) {
    const float gt = (lane < clen) ? load_gate(a.gt, (int64_t)(t0 + lane) * H + h, a.gate_bf16) : 0.f;
    const float c = wave_inclusive_scan(-gt * gh, lane);
    sC[lane] = c;
    const float c31 = __shfl(c, 31);   // every lane takes part: not inside the conditional
    sF[lane] = fast_exp2(lane >= 32 ? c - c31 : c);
    if (lane == 63) A.wFtot[(int64_t)cidx * H + h] = c;
  }
  // Global addresses are kept as a wave-uniform base plus a 32-bit lane offset, so that the
  // loop-invariant parts live in scalar registers.
  // Staging of DG value rows x 64 tokens (v, b, do, dovar) and the dv/db flush: threads 0..16 DG - 1,
  // thread = (token s, quad of rows q4).
  const int64_t row0 = ((int64_t)t0 * H + h) * dv;
  const TIn* vp = (const TIn*)a.v + row0;
  const TIn* bp = (const TIn*)a.b + row0;
  const TIn* dop = (const TIn*)A.d_o + row0;
  const int st_s = tid / (DG / 4), st_q = tid % (DG / 4);
  const bool st_on = tid < kC * DG / 4;
  const unsigned st_off = (unsigned)(st_s * H * dv + 4 * st_q);
  auto stage = [&](int dg) {
    if (!st_on) return;
    float st[NST][4];
    // the lane offset is made opaque here so that no per-lane 64-bit address is kept across the loop
    unsigned off = st_off;
    asm volatile("" : "+v"(off));
    if (st_s < clen) {
      load_vec<4>(vp + dg * DG + off, st[0]);
      load_vec<4>(bp + dg * DG + off, st[1]);
      load_vec<4>(dop + dg * DG + off, st[2]);
#pragma unroll
      for (int e = 0; e < 4; ++e) st[2][e] *= scale;
      if (HAS_VAR) {
#pragma unroll
        for (int e = 0; e < 4; ++e) st[NST - 1][e] = scale * load_rt(A.d_o_var, row0 + dg * DG + off + e, a.var_bf16);
      }
    } else {
#pragma unroll
      for (int x = 0; x < NST; ++x)
#pragma unroll
        for (int e = 0; e < 4; ++e) st[x][e] = 0.f;
    }
    const int buf = dg & 1;
#pragma unroll
    for (int x = 0; x < NST; ++x)
#pragma unroll
      for (int e = 0; e < 4; ++e) sSt[((buf * NST + x) * DG + 4 * st_q + e) * kVS2 + st_s] = st[x][e];
  };
  const int64_t rs = qk_stride(a);      // token stride of q, k
  const int64_t rso = (int64_t)H * dk;  // token stride of dq, dk (one row per value head)
  const int64_t tile_off = (((int64_t)cidx * H + h) * dv) * dk;
  const int n_groups = dv / DG;
  int pass = 0, nb = nbl, n_act = NB;   // set per pass: global column block of this wave, active blocks

  // end of one iteration, identical for every role: stage the next group of DG value rows mid-group
  // into the other buffer, synchronise, and flush dv/db once the consumers have finished a group
  auto iter_tail = [&](int it) {
    if ((it & (DG - 1)) == DG / 2 && it / DG + 1 < n_groups) stage(it / DG + 1);
    __syncthreads();
    if (it >= kLagC && ((it - kLagC) & (DG - 1)) == DG - 1) {
      const int dg = (it - kLagC) / DG;
      if (st_on && st_s < clen) {
        unsigned off = st_off;
        asm volatile("" : "+v"(off));
        TIn* dvo = (TIn*)A.dv + row0 + dg * DG + off;
        TIn* dbo = (TIn*)A.db + row0 + dg * DG + off;
        float sv[4] = {0.f, 0.f, 0.f, 0.f}, sb_[4] = {0.f, 0.f, 0.f, 0.f};
        if (MULTI && pass > 0) {   // later passes add to what the earlier column groups left
          load_vec<4>(dvo, sv);
          load_vec<4>(dbo, sb_);
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) {
#pragma unroll
          for (int w = 0; w < NB; ++w) {
            if (!MULTI || w < n_act) {
              sv[e] += sPv[(w * DG + 4 * st_q + e) * kC + st_s];
              sb_[e] += sPb[(w * DG + 4 * st_q + e) * kC + st_s];
            }
          }
        }
        store_vec<4>(dvo, sv);
        store_vec<4>(dbo, sb_);
      }
      // carry handed to the previous tile, f_first * dM^loc at the first token: thread = (column block, row, quad of columns)
      if (tid < n_act * DG * 4) {
        const int w = tid / (DG * 4), row = (tid >> 2) & (DG - 1), q4 = tid & 3;
        const float f_first = fast_exp2(sC[0]);
        const f32x4 cm = *(const f32x4*)&sCar[tid * 8], cj = *(const f32x4*)&sCar[tid * 8 + 4];
        const float rm[4] = {f_first * cm[0], f_first * cm[1], f_first * cm[2], f_first * cm[3]};
        const float rj[4] = {f_first * cj[0], f_first * cj[1], f_first * cj[2], f_first * cj[3]};
        const int64_t co = tile_off + (int64_t)(dg * DG + row) * dk + 16 * (pass * NB + w) + 4 * q4;
        store_vec<4>((TIn*)A.wDM + co, rm);
        store_vec<4>((TIn*)A.wDJ + co, rj);
      }
      __syncthreads();
    }
  };

  // ------------------------------------------------------------------ the tile as two halves of 32 tokens
  // A causal product over 64 tokens costs 6 matrix instructions per 16 columns (token blocks of 16 against
  // K = 16, 32, 48, 64, padded to multiples of 32), over two halves of 32 tokens 4: the second half starts from the
  // state after token 31, which the first producer has in its accumulators and leaves in sMJ for the second one, a
  // row behind.  The reverse contraction of the first half needs what flows back over the border,
  // f_32 dM^loc_32 = sum_{t >= 32} 2^(c_t - c_31) dMloc_t: the second producer sums it from its local gradients and
  // the first consumer adds it to the local gradient of token 31 in its operand.  The two producers are then the
  // same code on tokens 0..31 and 32..63 and each consumer reads only its own half's operands: 24 matrix
  // instructions (PREC: 72) and 16 KB of LDS traffic per value row and column block.
  //   sMJ slot of a row (d mod 3): [M_0, J_0, M_31, J_31, f_32 dM^loc_32, f_32 dJ^loc_32][16 key columns]
  // How the state before a half (M_p, J_p) enters its products:
  //   FOLD (bf16 operands, no initial state): it rides in the operand of the half's first token,
  //     X'_first = X_first + f_first (M_p, J_p), since the decay from before the half to token t is L[t,first] f_first;
  //     the strictly-lower product gets it for the first token itself as a virtual token in its last contraction slot
  //     (token 31 / 63, which is never below a column token of the half).  The state is rounded to bf16 there like
  //     every other operand; a J_0 below zero (an initial state with I_0 < Ip) would cancel against Ip, so launches
  //     with an initial state take the next form;
  //   else in fp32: M_t = Fh_t M_p + (product), with Fh_t = sF[t] the decay from before the half; the strictly-lower
  //     product of bf16 operands takes Fh_s M_p through the virtual token (on every column), that of split
  //     operands (PREC) adds it in fp32.
  auto producer = [&](auto hfc, auto foldc) {
    constexpr int HF = decltype(hfc)::value;   // tokens 32HF .. 32HF+31
    constexpr bool FOLD = decltype(foldc)::value;
    bf16x8 Lop[2];            // L[t,s] inside the half: t = 32HF+16tl+i, s = 32HF+8g+j <= t
    bf16x8 Lol[PREC ? 2 : 1]; // PREC: its lo halves
    float kk[8], kk2[8];      // k and its square in operand layout (n = i, s = 32HF+8g+j)
    float qq[8];              // q in result layout (t = 32HF+16tl+4g+r, n = i)
    float dq[8];
    // second half: 2^(c_t - c_31), the weight of token t in what flows back to token 31 (bf16 pairs / PREC: fp32)
    bf16x2 wD[(HF && !PREC) ? 4 : 1];
    float wDf[(HF && PREC) ? 8 : 1];
    float sigacc = 0.f;
    {
      const TIn* kp = (const TIn*)a.k + qk_row(a, t0, h) + 16 * nb;
      const TIn* qp = (const TIn*)a.q + qk_row(a, t0, h) + 16 * nb;
      float ct[2], cs[8];
#pragma unroll
      for (int tl = 0; tl < 2; ++tl) ct[tl] = sC[32 * HF + 16 * tl + i];
      *(f32x4*)&cs[0] = *(const f32x4*)&sC[32 * HF + 8 * g];
      *(f32x4*)&cs[4] = *(const f32x4*)&sC[32 * HF + 8 * g + 4];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int s = 32 * HF + 8 * g + j;
        const bool ok = s < clen;
        const float kv = to_f32((kp + (int64_t)(ok ? s : 0) * rs)[i]);
        kk[j] = ok ? kv : 0.f;
        kk2[j] = kk[j] * kk[j];
#pragma unroll
        for (int tl = 0; tl < 2; ++tl) {
          const int t = 32 * HF + 16 * tl + i;
          const float lv = (s <= t) ? fast_exp2(ct[tl] - cs[j]) : 0.f;
          const bf16_t lh = (bf16_t)lv;
          Lop[tl][j] = lh;
          if constexpr (PREC) Lol[tl][j] = (bf16_t)(lv - (float)lh);
        }
      }
#pragma unroll
      for (int tl = 0; tl < 2; ++tl)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int t = 32 * HF + 16 * tl + 4 * g + r;
          const bool ok = t < clen;
          const float qv = to_f32((qp + (int64_t)(ok ? t : 0) * rs)[i]);
          qq[tl * 4 + r] = ok ? qv : 0.f;
          dq[tl * 4 + r] = 0.f;
        }
      if (HF) {
#pragma unroll
        for (int tl = 0; tl < 2; ++tl) {
          const f32x4 w4 = *(const f32x4*)&sF[32 + 16 * tl + 4 * g];
          if constexpr (PREC) {
#pragma unroll
            for (int r = 0; r < 4; ++r) wDf[tl * 4 + r] = w4[r];
          } else {
            wD[tl * 2] = pack2(w4[0], w4[1]);
            wD[tl * 2 + 1] = pack2(w4[2], w4[3]);
          }
        }
      }
    }
    // first half: tile-start state of the next value row (entry of the own key column n = i), fetched one row ahead
    const float* cmu = a.chunk_mu + tile_off + 16 * nb;
    const float* cI = a.chunk_I + tile_off + 16 * nb;
    float mu_n = 0.f, I_n = 0.f;
    if (!HF) { mu_n = cmu[i]; I_n = cI[i]; }
    // FOLD: decay of the incoming state into the first token of the half, on the lanes that hold that token's operand
    const float f0m = (FOLD && g == 0) ? sF[32 * HF] : 0.f;
    int b3 = 0;                                 // d mod 3: the row's slot of sMJ and of the first producer's operands
    for (int it = 0; it < dv + kLagC; ++it) {
      if (it >= HF && it - HF < dv) {
        const int d = it - HF, dd = d & (DG - 1), buf = (d / DG) & 1;
        const float* sV = sSt + (buf * NST + 0) * STG + dd * kVS2;
        const float* sB = sSt + (buf * NST + 1) * STG + dd * kVS2;
        const float* sDo = sSt + (buf * NST + 2) * STG + dd * kVS2;
        const float* sDov = sSt + (buf * NST + NST - 1) * STG + dd * kVS2;
        float* mj = sMJ + (nbl * 3 + b3) * 96;
        float Mp, Jp;   // state before the first token of the half
        if (!HF) {
          const float mu0 = mu_n, I0 = I_n;
          const int64_t dn = (int64_t)min(d + 1, dv - 1) * dk;
          mu_n = (cmu + dn)[i];
          I_n = (cI + dn)[i];
          Mp = mu0 * I0;
          Jp = I0 - Ip;
          if (g == 0) { mj[i] = Mp; mj[16 + i] = Jp; }
        } else {
          Mp = mj[32 + i];
          Jp = mj[48 + i];
        }
        bf16x8 XM, XJ;
        bf16x8 XMl, XJl;   // PREC: the lo halves
        {
          const f32x4 v0 = *(const f32x4*)&sV[32 * HF + 8 * g], v1 = *(const f32x4*)&sV[32 * HF + 8 * g + 4];
          const f32x4 b0 = *(const f32x4*)&sB[32 * HF + 8 * g], b1 = *(const f32x4*)&sB[32 * HF + 8 * g + 4];
          if constexpr (PREC) {
            float xm[8], xj[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) {
              xm[j] = kk[j] * (j < 4 ? v0[j & 3] : v1[j & 3]);
              xj[j] = kk2[j] * (j < 4 ? b0[j & 3] : b1[j & 3]);
            }
            split_bf16(xm, XM, XMl);
            split_bf16(xj, XJ, XJl);
          } else {
            const float fM = f0m * Mp, fJ = f0m * Jp;
#pragma unroll
            for (int j = 0; j < 8; j += 2) {
              const float va = j < 4 ? v0[j & 3] : v1[j & 3], vb = j < 4 ? v0[(j & 3) + 1] : v1[(j & 3) + 1];
              const float ba = j < 4 ? b0[j & 3] : b1[j & 3], bb = j < 4 ? b0[(j & 3) + 1] : b1[(j & 3) + 1];
              const bool tok0 = FOLD && j == 0;
              const bf16x2 pm = pack2(tok0 ? fmaf(kk[j], va, fM) : kk[j] * va, kk[j + 1] * vb);
              const bf16x2 pj = pack2(tok0 ? fmaf(kk2[j], ba, fJ) : kk2[j] * ba, kk2[j + 1] * bb);
              XM[j] = pm[0]; XM[j + 1] = pm[1];
              XJ[j] = pj[0]; XJ[j + 1] = pj[1];
            }
          }
        }
        bf16x8 PM, PJ;
        float pmf[PREC ? 8 : 1], pjf[PREC ? 8 : 1];   // PREC: the local gradients in fp32 until they are split
        float backM = 0.f, backJ = 0.f;
#pragma unroll
        for (int tl = 0; tl < 2; ++tl) {
          const int tb = 2 * HF + tl;
          f32x4 accM = {0.f, 0.f, 0.f, 0.f};
          f32x4 accI = {Ip, Ip, Ip, Ip};
          if constexpr (PREC) {
            accM = mfma16_split(Lop[tl], Lol[tl], XM, XMl, accM);
            accI = mfma16_split(Lop[tl], Lol[tl], XJ, XJl, accI);
          } else {
            accM = mfma16(Lop[tl], XM, accM);
            accI = mfma16(Lop[tl], XJ, accI);
          }
          f32x4 Fv = {0.f, 0.f, 0.f, 0.f};
          if constexpr (!FOLD) Fv = *(const f32x4*)&sF[16 * tb + 4 * g];
          const f32x4 dov = *(const f32x4*)&sDo[16 * tb + 4 * g];
          f32x4 dvv = {0.f, 0.f, 0.f, 0.f};
          if (HAS_VAR) dvv = *(const f32x4*)&sDov[16 * tb + 4 * g];
          float dMl[4], dJl[4];
          float M3 = 0.f, I3 = 0.f;
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const float Mf = FOLD ? accM[r] : fmaf(Fv[r], Mp, accM[r]);
            const float If = FOLD ? accI[r] : fmaf(Fv[r], Jp, accI[r]);
            if (r == 3) { M3 = Mf; I3 = If; }
            const float rI = fast_rcp(If);
            const float mu = Mf * rI;
            const float q = qq[tl * 4 + r];
            dMl[r] = (dov[r] * q) * rI;
            dJl[r] = -(dMl[r] * mu);
            dq[tl * 4 + r] = fmaf(mu, dov[r], dq[tl * 4 + r]);
            if (HAS_VAR) {
              const float wq = dvv[r] * q;          // scale*dovar*q
              const float w = wq * q * rI;          // scale*dovar*q^2/I
              dJl[r] = fmaf(-w, rI, dJl[r]);
              dq[tl * 4 + r] = fmaf(2.f * wq, rI, dq[tl * 4 + r]);
            }
            if constexpr (PREC) sigacc += dJl[r];
          }
          if (!HF && tl == 1 && g == 3) {   // state after token 31 for the second half of the row
            mj[32 + i] = M3;
            mj[48 + i] = I3 - Ip;
          }
          const int o4 = tl * 4;
          if constexpr (PREC) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
              pmf[o4 + r] = dMl[r];
              pjf[o4 + r] = dJl[r];
              if (HF) {   // what flows back over the border
                backM = fmaf(wDf[o4 + r], dMl[r], backM);
                backJ = fmaf(wDf[o4 + r], dJl[r], backJ);
              }
            }
          } else {
            const bf16x2 m0 = pack2(dMl[0], dMl[1]), m1 = pack2(dMl[2], dMl[3]);
            const bf16x2 j0 = pack2(dJl[0], dJl[1]), j1 = pack2(dJl[2], dJl[3]);
            // the sum of dJloc (for dIp) from the packed pairs: one instruction per two entries
            const bf16x2 one2 = {(bf16_t)1.f, (bf16_t)1.f};
            sigacc = __builtin_amdgcn_fdot2_f32_bf16(j0, one2, sigacc, false);
            sigacc = __builtin_amdgcn_fdot2_f32_bf16(j1, one2, sigacc, false);
            if (HF) {   // what flows back over the border, from the packed pairs
              backM = __builtin_amdgcn_fdot2_f32_bf16(m0, wD[tl * 2], backM, false);
              backM = __builtin_amdgcn_fdot2_f32_bf16(m1, wD[tl * 2 + 1], backM, false);
              backJ = __builtin_amdgcn_fdot2_f32_bf16(j0, wD[tl * 2], backJ, false);
              backJ = __builtin_amdgcn_fdot2_f32_bf16(j1, wD[tl * 2 + 1], backJ, false);
            }
            PM[o4 + 0] = m0[0]; PM[o4 + 1] = m0[1]; PM[o4 + 2] = m1[0]; PM[o4 + 3] = m1[1];
            PJ[o4 + 0] = j0[0]; PJ[o4 + 1] = j0[1]; PJ[o4 + 2] = j1[0]; PJ[o4 + 3] = j1[1];
          }
        }
        if (HF) {   // sums over the four lane rows: row 0 gets the mean branch's total, row 1 the precision branch's
          const float tot = rows4_sum_x4(backM, backJ, 0.f, 0.f);
          if (g < 2) mj[64 + 16 * g + i] = tot;
        }
        bf16x8* mine = sX + ((nbl * 20 + (HF ? 12 + 4 * (d & 1) : 4 * b3)) * XS) * 64 + lane;
        if constexpr (PREC) {
          bf16x8 PMl, PJl;
          split_bf16(pmf, PM, PMl);
          split_bf16(pjf, PJ, PJl);
          mine[4 * 64] = PMl; mine[5 * 64] = PJl; mine[6 * 64] = XMl; mine[7 * 64] = XJl;
        }
        mine[0] = PM; mine[64] = PJ; mine[2 * 64] = XM; mine[3 * 64] = XJ;
        b3 = (b3 == 2) ? 0 : b3 + 1;
      }
      iter_tail(it);
    }
    TIn* dqp = (TIn*)A.dq + ((int64_t)t0 * H + h) * dk + 16 * nb;
#pragma unroll
    for (int tl = 0; tl < 2; ++tl)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int t = 32 * HF + 16 * tl + 4 * g + r;
        if (t < clen) (dqp + (int64_t)t * rso)[i] = from_f32<TIn>(dq[tl * 4 + r]);
      }
    const float x = wave_sum(sigacc);
    if (lane == 0) sRed[NB * kC + HF * NB + nbl] = x;
  };

  // ------------------------------------------------------------------ consumers
  auto consumer = [&](auto hfc, auto foldc) {
    constexpr int HF = decltype(hfc)::value;   // column tokens 32HF .. 32HF+31 (blocks sb = 2HF+sl)
    constexpr bool FOLD = decltype(foldc)::value;
    bf16x8 Lr[2];     // reverse operand inside the half: contraction (g,j) <-> token t = 32HF + 16(j/4) + 4g + j%4 >= s
    bf16x8 Ls[2];     // strictly-lower operand: contraction token s' = 32HF + 8g + j < column token s = 16sb+i
    bf16x8 Lrl[PREC ? 2 : 1], Lsl[PREC ? 2 : 1];   // PREC: their lo halves
    float kr[8], kr2[8];   // k and its square in result layout (s = 16sb+i, n = 4g+r)
    float dkM[8], dkJ[8];
    float gate[2], Fs[2];
    {
      const TIn* kp4 = (const TIn*)a.k + qk_row(a, t0, h) + 16 * nb;
      float ct[2], cs[8], ctt[8];
#pragma unroll
      for (int sl = 0; sl < 2; ++sl) ct[sl] = sC[16 * (2 * HF + sl) + i];
      *(f32x4*)&cs[0] = *(const f32x4*)&sC[32 * HF + 8 * g];
      *(f32x4*)&cs[4] = *(const f32x4*)&sC[32 * HF + 8 * g + 4];
      *(f32x4*)&ctt[0] = *(const f32x4*)&sC[32 * HF + 4 * g];
      *(f32x4*)&ctt[4] = *(const f32x4*)&sC[32 * HF + 16 + 4 * g];
#pragma unroll
      for (int sl = 0; sl < 2; ++sl) {
        const int s = 16 * (2 * HF + sl) + i;
        Fs[sl] = sF[s];   // decay from before the half to the column token
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const int sp = 32 * HF + 8 * g + j;
          float lv = (sp < s) ? fast_exp2(ct[sl] - cs[j]) : 0.f;
          // the virtual token (bf16 operands): the state before the half, for the half's first token only when the
          // operands carry it already (FOLD), else for every column token
          if (!PREC && g == 3 && j == 7) lv = (FOLD && s != 32 * HF) ? 0.f : Fs[sl];
          const bf16_t lh = (bf16_t)lv;
          Ls[sl][j] = lh;
          if constexpr (PREC) Lsl[sl][j] = (bf16_t)(lv - (float)lh);
          const int t = 32 * HF + 16 * (j >> 2) + 4 * g + (j & 3);
          const float rv = (t >= s) ? fast_exp2(ctt[j] - ct[sl]) : 0.f;
          const bf16_t rh = (bf16_t)rv;
          Lr[sl][j] = rh;
          if constexpr (PREC) Lrl[sl][j] = (bf16_t)(rv - (float)rh);
        }
#pragma unroll
        for (int r = 0; r < 4; ++r) { kr[sl * 4 + r] = 0.f; dkM[sl * 4 + r] = 0.f; dkJ[sl * 4 + r] = 0.f; }
        if (s < clen) load_vec<4>(kp4 + (int64_t)s * rs + 4 * g, &kr[sl * 4]);
#pragma unroll
        for (int r = 0; r < 4; ++r) kr2[sl * 4 + r] = kr[sl * 4 + r] * kr[sl * 4 + r];
        gate[sl] = 0.f;
      }
    }
    // the carries between tiles are kept in the dtype of the rows: bf16 rows feed them to the matrix cores in bf16
    // anyway (carry apply), and the scan that sums them over the tiles runs in fp32 registers.  The consumer of the
    // first column token parks them per group of value rows; the flush of the group scales and stores them.
    float* car = sCar + ((nbl * DG) * 4 + g) * 8;
    // after the 4-way transposing reduction, row g of the wave holds dv (g<2) or db (g>=2) of token block g&1
    float* pw = ((g < 2) ? sPv : sPb) + nbl * DG * kC + 16 * (2 * HF + (g & 1)) + i;
    int b3 = 0;   // d mod 3
    for (int it = 0; it < dv + kLagC; ++it) {
      if (it >= kLagC) {
        const int d = it - kLagC, dd = d & (DG - 1), buf = (d / DG) & 1;
        const float* sV = sSt + (buf * NST + 0) * STG + dd * kVS2;
        const float* sB = sSt + (buf * NST + 1) * STG + dd * kVS2;
        // the own half's operands
        const bf16x8* ph = sX + ((nbl * 20 + (HF ? 12 + 4 * (d & 1) : 4 * b3)) * XS) * 64 + lane;
        const float* mj = sMJ + (nbl * 3 + b3) * 96;
        b3 = (b3 == 2) ? 0 : b3 + 1;
        bf16x8 PM = ph[0], PJ = ph[64], XM = ph[2 * 64], XJ = ph[3 * 64];
        bf16x8 PMl, PJl, XMl, XJl;   // PREC: the lo halves
        f32x4 MpT = {0.f, 0.f, 0.f, 0.f}, JpT = {0.f, 0.f, 0.f, 0.f};   // PREC: state before the half, key columns n = 4g+r
        if constexpr (PREC) {
          PMl = ph[4 * 64]; PJl = ph[5 * 64]; XMl = ph[6 * 64]; XJl = ph[7 * 64];
          MpT = *(const f32x4*)&mj[32 * HF + 4 * g];
          JpT = *(const f32x4*)&mj[32 * HF + 16 + 4 * g];
        } else {
          // virtual token of the strictly-lower products: the state before the half's first token (key column n = i)
          const bf16x2 st2 = pack2(mj[32 * HF + i], mj[32 * HF + 16 + i]);
          if (g == 3) { XM[7] = st2[0]; XJ[7] = st2[1]; }
        }
        if (!HF) {
          // what flows back over the border joins the local gradient of token 31 (element 7 of the lanes g = 3)
          const float bm = mj[64 + i], bj = mj[80 + i];
          if (g == 3) {
            if constexpr (PREC) {
              const float xm = ((float)PM[7] + (float)PMl[7]) + bm, xj = ((float)PJ[7] + (float)PJl[7]) + bj;
              const bf16_t mh = (bf16_t)xm, jh = (bf16_t)xj;
              PM[7] = mh; PMl[7] = (bf16_t)(xm - (float)mh);
              PJ[7] = jh; PJl[7] = (bf16_t)(xj - (float)jh);
            } else {
              PM[7] = (bf16_t)((float)PM[7] + bm);
              PJ[7] = (bf16_t)((float)PJ[7] + bj);
            }
          }
        }
        float dvp[2], dbp[2];
        const f32x4 z4 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int sl = 0; sl < 2; ++sl) {
          const int sb = 2 * HF + sl;
          f32x4 aM, aJ, sM, sJ;
          if constexpr (PREC) {
            aM = mfma16_split(PM, PMl, Lr[sl], Lrl[sl], z4);
            aJ = mfma16_split(PJ, PJl, Lr[sl], Lrl[sl], z4);
            sM = mfma16_split(XM, XMl, Ls[sl], Lsl[sl], z4);
            sJ = mfma16_split(XJ, XJl, Ls[sl], Lsl[sl], z4);
          } else {
            aM = mfma16(PM, Lr[sl], z4);
            aJ = mfma16(PJ, Lr[sl], z4);
            // S[n, s] = f_s M_{s-1}: strictly-lower product in the same [n, s] layout
            sM = mfma16(XM, Ls[sl], z4);
            sJ = mfma16(XJ, Ls[sl], z4);
          }
          const float vS = sV[16 * sb + i];
          const float bS = sB[16 * sb + i];
          float dvs = 0.f, dbs = 0.f, gm = gate[sl];
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            dvs = fmaf(aM[r], kr[sl * 4 + r], dvs);
            dbs = fmaf(aJ[r], kr2[sl * 4 + r], dbs);
            dkM[sl * 4 + r] = fmaf(aM[r], vS, dkM[sl * 4 + r]);
            dkJ[sl * 4 + r] = fmaf(aJ[r], bS, dkJ[sl * 4 + r]);
            const float Ss = PREC ? fmaf(Fs[sl], MpT[r], sM[r]) : sM[r];
            const float SJ = PREC ? fmaf(Fs[sl], JpT[r], sJ[r]) : sJ[r];
            gm = fmaf(aM[r], Ss, gm);
            gm = fmaf(aJ[r], SJ, gm);
          }
          gate[sl] = gm;
          dvp[sl] = dvs;
          dbp[sl] = dbs;
          if (!HF && sl == 0 && i == 0) {
            *(f32x4*)&car[dd * 32] = aM;
            *(f32x4*)&car[dd * 32 + 4] = aJ;
          }
        }
        pw[dd * kC] = rows4_sum_x4(dvp[0], dvp[1], dbp[0], dbp[1]);
      }
      iter_tail(it);
    }
    TIn* dkp = (TIn*)A.dk + ((int64_t)t0 * H + h) * dk + 16 * nb;
#pragma unroll
    for (int sl = 0; sl < 2; ++sl) {
      const int s = 16 * (2 * HF + sl) + i;
      if (s < clen) {
#pragma unroll
        for (int r = 0; r < 4; ++r)
          (dkp + (int64_t)s * rso)[4 * g + r] = from_f32<TIn>(fmaf(2.f * kr[sl * 4 + r], dkJ[sl * 4 + r], dkM[sl * 4 + r]));
      }
      const float x = rows4_sum(gate[sl]);
      if (g == 0) sRed[nbl * kC + 16 * (2 * HF + sl) + i] = x;
    }
  };

  // every role runs dv+1 iterations with the same barriers; a wave whose column block lies beyond dk
  // (last pass of a head dim that is not a multiple of 16*NB) only keeps the barriers
  float gm_tot = 0.f, sg_tot = 0.f;   // threads 0..63: gate term of token tid; thread 0: sum of dJloc
  for (pass = 0; pass < n_pass; ++pass) {
    nb = pass * NB + nbl;
    n_act = MULTI ? min(NB, nb_total - pass * NB) : NB;
    // the per-role constants that do not depend on the column block (decay operands) must be computed
    // inside the role that uses them: hoisted above the role branches or out of this loop they would be
    // live for all four roles at once
    asm volatile("" : "+v"(lane));
    i = lane & 15;
    g = lane >> 4;
    stage(0);
    __syncthreads();
    if (MULTI && nbl >= n_act) {
      for (int it = 0; it < dv + kLagC; ++it) iter_tail(it);
    } else if (fold) {
      if constexpr (!PREC) {
        if (role == 0) producer(std::integral_constant<int, 0>{}, std::true_type{});
        else if (role == 1) producer(std::integral_constant<int, 1>{}, std::true_type{});
        else if (role == 2) consumer(std::integral_constant<int, 0>{}, std::true_type{});
        else consumer(std::integral_constant<int, 1>{}, std::true_type{});
      }
    } else if (role == 0) producer(std::integral_constant<int, 0>{}, std::false_type{});
    else if (role == 1) producer(std::integral_constant<int, 1>{}, std::false_type{});
    else if (role == 2) consumer(std::integral_constant<int, 0>{}, std::false_type{});
    else consumer(std::integral_constant<int, 1>{}, std::false_type{});
    __syncthreads();
    if (tid < kC) {
#pragma unroll
      for (int w = 0; w < NB; ++w)
        if (!MULTI || w < n_act) gm_tot += sRed[w * kC + tid];
      if (tid == 0) {
#pragma unroll
        for (int w = 0; w < NB; ++w)
          if (!MULTI || w < n_act) sg_tot += sRed[NB * kC + w] + sRed[NB * kC + NB + w];
      }
    }
    __syncthreads();
  }
  if (tid < clen) A.wE[(int64_t)h * A.tokens + t0 + tid] = gm_tot;
  if (tid == 0) A.wSig[(int64_t)cidx * H + h] = sg_tot;
}

// ----------------------------------------------------------------- carry scan
// R_{c-1} = R_loc,c + F_c R_c backwards over the tiles of a sequence: one thread per four consecutive state
// entries of a (sequence, head), 1024 entries per block; the running sums stay in fp32 registers, the slot of a
// tile is read (its local carry) and overwritten (the carry coming in from the later tiles) in the row dtype.
__host__ __device__ inline int carry_scan_blocks(int64_t E) { return (int)((E + 1023) / 1024); }

template <typename TC>
__global__ __launch_bounds__(256) void chunk_bwd_carry_scan_kernel(BwdArgs A) {
  const ChunkArgs& a = A.c;
  __shared__ float sW[4];
  const int64_t E = (int64_t)a.dv * a.dk;
  const int nblk = carry_scan_blocks(E);
  const int blk = blockIdx.x % nblk;
  const int nh = blockIdx.x / nblk;
  const int h = nh % a.H, n = nh / a.H;
  const int64_t e = ((int64_t)blk * 256 + threadIdx.x) * 4;
  const bool on = e < E;
  int bos, len, cbase;
  seq_lookup(a, n, bos, len, cbase);
  const int nchunks = (len + kC - 1) / kC;
  TC* wDM = (TC*)A.wDM;
  TC* wDJ = (TC*)A.wDJ;
  float RM[4] = {0.f, 0.f, 0.f, 0.f}, RJ[4] = {0.f, 0.f, 0.f, 0.f};
  if (on) {
    auto advance = [&](int64_t off, const float* DM, const float* DJ, float Ft) {
      store_vec<4>(wDM + off, RM);
      store_vec<4>(wDJ + off, RJ);
#pragma unroll
      for (int x = 0; x < 4; ++x) {
        RM[x] = fmaf(Ft, RM[x], DM[x]);
        RJ[x] = fmaf(Ft, RJ[x], DJ[x]);
      }
    };
    int c = nchunks - 1;
    for (; c >= 3; c -= 4) {   // four tiles' loads in flight at a time
      float DM[4][4], DJ[4][4], Ft[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int64_t off = ((int64_t)(cbase + c - u) * a.H + h) * E + e;
        load_vec<4>(wDM + off, DM[u]);
        load_vec<4>(wDJ + off, DJ[u]);
        Ft[u] = A.wFtot[(int64_t)(cbase + c - u) * a.H + h];
      }
#pragma unroll
      for (int u = 0; u < 4; ++u)
        advance(((int64_t)(cbase + c - u) * a.H + h) * E + e, DM[u], DJ[u], fast_exp2(Ft[u]));
    }
    for (; c >= 0; --c) {
      const int64_t off = ((int64_t)(cbase + c) * a.H + h) * E + e;
      float DM[4], DJ[4];
      load_vec<4>(wDM + off, DM);
      load_vec<4>(wDJ + off, DJ);
      advance(off, DM, DJ, fast_exp2(A.wFtot[(int64_t)(cbase + c) * a.H + h]));
    }
  }
  if (a.init_mu) {
    const int64_t so = (int64_t)nh * E + e;
    if (A.d_init_mu && on) {
      const f32x4 mu0 = *(const f32x4*)(a.init_mu + so), I0 = *(const f32x4*)(a.init_I + so);
      const f32x4 dmu = {RM[0] * I0[0], RM[1] * I0[1], RM[2] * I0[2], RM[3] * I0[3]};
      const f32x4 dI = {fmaf(RM[0], mu0[0], RJ[0]), fmaf(RM[1], mu0[1], RJ[1]), fmaf(RM[2], mu0[2], RJ[2]),
                        fmaf(RM[3], mu0[3], RJ[3])};
      *(f32x4*)(A.d_init_mu + so) = dmu;
      *(f32x4*)(A.d_init_I + so) = dI;
    }
    // J_0 = I_0 - Ip: the prior also receives -sum dJ_0
    float s = wave_sum((RJ[0] + RJ[1]) + (RJ[2] + RJ[3]));
    if ((threadIdx.x & 63) == 0) sW[threadIdx.x >> 6] = s;
    __syncthreads();
    if (threadIdx.x == 0) A.wInitPart[(int64_t)nh * nblk + blk] = sW[0] + sW[1] + sW[2] + sW[3];
  }
}

// ---------------------------------------------------------------- carry apply
// dv_s += a_s R_M k_s ; db_s += a_s R_J k_s^2 ; dk_s += a_s (R_M^T v_s + 2 k_s * R_J^T b_s)
// One workgroup of 4 waves per (tile, head); wave w owns tokens [16w, 16w+16).  The four products
// run on the matrix cores (bf16 operands, fp32 accumulate); their results are parked in LDS and then
// added to the tile-local gradients with 16-byte loads/stores that are contiguous along the head dim.
// KSMAX = operand registers per product (32 contraction indices each: head dims up to 32 KSMAX).  With
// SEQ the dv and db products take turns in one result buffer: less LDS, so that more workgroups share
// a compute unit (the kernel is a chain of dependent load, product and store phases, and it is the
// number of resident workgroups that hides them).
// PREC (fp32 rows): operands as two bf16 halves, three matrix instructions per product; the transposed copy of the
// carries then holds a second plane with the lo halves (never shared with a result buffer).
// (second launch bound: at most 256 registers per lane, so matrix results stay in ordinary vector registers)
// The kernel is a chain of phases, each of which starts with fetches from global memory (the carries, the operand
// rows, the gradients it adds to); taken in turn their latencies add up to most of the kernel's time.  So every fetch
// is issued as early as its address is known: the operand rows of all four products before the carries are staged,
// the gradients that a phase adds to before the matrix instructions of that phase.  Every wave scans the gates
// itself (the decay a_s of its own token rows), so the operands do not wait for another wave.
template <typename TIn, int KSMAX, bool SEQ, bool PREC>
__global__ __launch_bounds__(256, 2) void chunk_bwd_carry_apply_kernel(BwdArgs A) {
  const ChunkArgs& a = A.c;
  extern __shared__ float smem[];
  const int H = a.H, dk = a.dk, dv = a.dv;
  const int dmax = dk > dv ? dk : dv;
  float* sW4 = smem + kC;                  // [8]
  float* sBt = sW4 + 8;                    // [64][dv/8] beta of the carry terms, one slot per work item
  float* sO1 = sBt + kC * (dv >> 3);       // [64][OS] dk^carry, later dv^carry
  float* sO2 = SEQ ? sO1 : sO1 + kC * (dmax + 4);   // [64][OS] db^carry (SEQ: after dv^carry has been applied)
  // [2][dk][dv + 8] R_M^T, R_J^T in bf16, operand source of all four products.  When both do not fit the LDS
  // (large head dims) the bf16 copy shares its bytes with db^carry and the dv/db products read the fp32
  // carries from global memory instead.
  const bool alias = !SEQ && A.apply_alias != 0;
  bf16_t* sRT = (bf16_t*)(alias ? sO2 : sO2 + kC * (dmax + 4));
  const int RS = dv + 8;
  bf16_t* sRTl = sRT + 2 * dk * RS;        // PREC: [2][dk][dv + 8] lo halves
  const int OS = dmax + 4;
  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6, i = lane & 15, g = lane >> 4;
  const int cidx = blockIdx.x / H, h = blockIdx.x % H;
  int seq, t0, clen, cis;
  chunk_lookup(a, cidx, seq, t0, clen, cis);
  int bos, len, cbase;
  seq_lookup(a, seq, bos, len, cbase);
  const bool last = cis == (len + kC - 1) / kC - 1;
  // the gates of the tile's tokens (every wave), and for wave 0 the local part of d log f
  const bool tok_ok = lane < clen;
  const int64_t tokL = (int64_t)t0 + lane;
  const float gt_l = tok_ok ? load_gate(a.gt, tokL * H + h, a.gate_bf16) : 0.f;
  float e_l = 0.f;
  if (w == 0 && tok_ok) e_l = A.wE[(int64_t)h * A.tokens + tokL];
  // Gate gradient of the tile's tokens, by wave 0 once the carry terms are known:
  //   d log f_t = (local part, from the tile kernel) + (carry terms of the earlier tokens of the tile) + (boundary term),
  //   dgt_t = -g d log f_t, and the tile's share of dg = -sum_t gt_t d log f_t.
  auto gate_grad = [&](float bc, float bnd) {
    const float pre = wave_inclusive_scan(bc, lane) - bc;
    const float dlogf = tok_ok ? e_l + pre + bnd : 0.f;
    if (tok_ok) A.dgt[tokL * H + h] = -a.g[h] * dlogf;
    const float share = wave_sum(-gt_l * dlogf);
    if (lane == 0) A.wDgTile[(int64_t)cidx * H + h] = share;
  };
  if (last) {  // nothing flows in from beyond the end of the sequence (uniform for the block)
    if (w == 0) gate_grad(0.f, 0.f);
    return;
  }
  const float gh = a.g[h] * kLog2e;
  const int srow = 16 * w + i;            // operand row (token) of this lane
  const bool row_ok = srow < clen;
  float as, Ftot;                         // decay from token srow to the end of the tile, and over the whole tile
  {
    const float c = wave_inclusive_scan(-gt_l * gh, lane);
    const float tot = __shfl(c, 63);
    as = fast_exp2(tot - __shfl(c, srow));
    Ftot = fast_exp2(tot);
  }
  const int64_t tokA = ((int64_t)(t0 + (row_ok ? srow : 0)) * H + h);
  const int64_t tok0 = ((int64_t)t0 * H + h);

  // operands of the four products: rows a_s v_s, a_s b_s (contraction over the value rows) and a_s k_s, a_s k_s^2
  // (over the key columns) of this lane's token.  EARLY: built before anything else (the registers are there).
  constexpr bool EARLY = (PREC ? 2 : 1) * KSMAX <= 4;
  bf16x8 A3[KSMAX], A4[KSMAX], A1[KSMAX], A2[KSMAX];
  bf16x8 A3l[PREC ? KSMAX : 1], A4l[PREC ? KSMAX : 1], A1l[PREC ? KSMAX : 1], A2l[PREC ? KSMAX : 1];
  auto build_vb = [&]() {
    const int KS = (dv + 31) / 32;
    const TIn* vp = (const TIn*)a.v + tokA * dv;
    const TIn* bp = (const TIn*)a.b + tokA * dv;
#pragma unroll
    for (int ks = 0; ks < KSMAX; ++ks) {
      if (ks < KS) {
        const int d0 = 8 * g + 32 * ks;
        float vv[8], bb[8];
        if (row_ok && d0 < dv) {
          load_vec<4>(vp + d0, vv); load_vec<4>(vp + d0 + 4, vv + 4);
          load_vec<4>(bp + d0, bb); load_vec<4>(bp + d0 + 4, bb + 4);
        } else {
#pragma unroll
          for (int j = 0; j < 8; ++j) { vv[j] = 0.f; bb[j] = 0.f; }
        }
        if constexpr (PREC) {
#pragma unroll
          for (int j = 0; j < 8; ++j) { vv[j] *= as; bb[j] *= as; }
          split_bf16(vv, A3[ks], A3l[ks]);
          split_bf16(bb, A4[ks], A4l[ks]);
        } else {
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            A3[ks][j] = (bf16_t)(as * vv[j]);
            A4[ks][j] = (bf16_t)(as * bb[j]);
          }
        }
      }
    }
  };
  auto build_k = [&]() {
    const int KS = (dk + 31) / 32;
    const TIn* kp = (const TIn*)a.k + qk_row(a, t0 + (row_ok ? srow : 0), h);
#pragma unroll
    for (int ks = 0; ks < KSMAX; ++ks) {
      if (ks < KS) {
        const int n0 = 8 * g + 32 * ks;
        float kv[8];
        if (row_ok && n0 < dk) {
          load_vec<4>(kp + n0, kv);
          load_vec<4>(kp + n0 + 4, kv + 4);
        } else {
#pragma unroll
          for (int j = 0; j < 8; ++j) kv[j] = 0.f;
        }
        if constexpr (PREC) {
          float k1[8], k2[8];
#pragma unroll
          for (int j = 0; j < 8; ++j) { k1[j] = as * kv[j]; k2[j] = k1[j] * kv[j]; }
          split_bf16(k1, A1[ks], A1l[ks]);
          split_bf16(k2, A2[ks], A2l[ks]);
        } else {
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            A1[ks][j] = (bf16_t)(as * kv[j]);
            A2[ks][j] = (bf16_t)(as * kv[j] * kv[j]);
          }
        }
      }
    }
  };
  build_vb();
  if constexpr (EARLY) build_k();

  const int64_t E = (int64_t)dv * dk;
  const TIn* RM = (const TIn*)A.wDM + ((int64_t)cidx * H + h) * E;
  const TIn* RJ = (const TIn*)A.wDJ + ((int64_t)cidx * H + h) * E;
  {
    // F_C (<R_M, M_0> + <R_J, J_0>) with (M_0, J_0) the state at the start of this tile; the same
    // pass leaves R^T in LDS for the products that contract over the value rows
    const float* smu = a.chunk_mu + ((int64_t)cidx * H + h) * E;
    const float* sI = a.chunk_I + ((int64_t)cidx * H + h) * E;
    const float Ipb = a.Ip[h];
    float acc = 0.f;
    // a wave instruction covers 16 value rows x 64 bytes, and a wave walks along the rows before it
    // moves to other rows, so that both halves of a 128-byte line are used while it is still in L1;
    // four blocks are fetched before the first is used
    const int nc = dk >> 4, nblk = (dv >> 4) * nc, per = (nblk + 3) >> 2;
    for (int j0 = 0; j0 < per; j0 += 4) {
      float rm[4][4], rj[4][4];
      f32x4 mu[4], I[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int blk = w * per + j0 + u;
        if (j0 + u < per && blk < nblk) {
          const int64_t e = (int64_t)(16 * (blk / nc) + i) * dk + 4 * (4 * (blk % nc) + g);
          load_vec<4>(RM + e, rm[u]);
          load_vec<4>(RJ + e, rj[u]);
          mu[u] = *(const f32x4*)(smu + e);
          I[u] = *(const f32x4*)(sI + e);
        }
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int blk = w * per + j0 + u;
        if (j0 + u < per && blk < nblk) {
          const int d = 16 * (blk / nc) + i, c4 = 4 * (blk % nc) + g;
#pragma unroll
          for (int x = 0; x < 4; ++x) {
            acc = fmaf(rm[u][x], mu[u][x] * I[u][x], acc);
            acc = fmaf(rj[u][x], I[u][x] - Ipb, acc);
            const bf16_t mh = (bf16_t)rm[u][x], jh = (bf16_t)rj[u][x];
            sRT[(4 * c4 + x) * RS + d] = mh;
            sRT[(dk + 4 * c4 + x) * RS + d] = jh;
            if constexpr (PREC) {
              sRTl[(4 * c4 + x) * RS + d] = (bf16_t)(rm[u][x] - (float)mh);
              sRTl[(dk + 4 * c4 + x) * RS + d] = (bf16_t)(rj[u][x] - (float)jh);
            }
          }
        }
      }
    }
    acc = wave_sum(acc);
    if (lane == 0) sW4[w] = acc;
  }
  // gradients this kernel adds to, as fetched: item m of a thread is (token s, eight consecutive entries c8) with
  // s * groups + c8 = tid + 256 m; a row has at most 4 KSMAX groups of eight, so a thread has at most KSMAX items
  // PRE: fetched a phase ahead, where the registers are there for it (else right before they are used)
  constexpr bool PRE = KSMAX <= 2 || (KSMAX == 4 && SEQ && !PREC && sizeof(TIn) == 2);
  Raw8<TIn> old1[KSMAX], old2[KSMAX], in1[KSMAX], in2[KSMAX];
  auto fetch_items = [&](const TIn* p, int groups, int row_len, Raw8<TIn>* dst) {
#pragma unroll
    for (int m = 0; m < KSMAX; ++m) {
      const int idx = tid + 256 * m, c8 = idx % groups, s = idx / groups;
      if (idx < kC * groups && s < clen) dst[m].load(p + (int64_t)s * H * row_len + 8 * c8);
    }
  };
  TIn* dko = (TIn*)A.dk + tok0 * dk;
  if constexpr (PRE) fetch_items(dko, dk >> 3, dk, old1);
  __syncthreads();
  const float bnd = Ftot * (sW4[0] + sW4[1] + sW4[2] + sW4[3]);   // every thread; the slots are not written again

  // ---- dk: out[s, n] = sum_d (a_s v_s[d]) R_M[d, n] + 2 k_s[n] sum_d (a_s b_s[d]) R_J[d, n]
  {
    const int KS = (dv + 31) / 32;
    const TIn* kin = (const TIn*)a.k + qk_row(a, t0, h);
    // k of the result entries (row s = 16w + 4g + r, column n = 16nbk + i), fetched one step ahead
    auto load_k4 = [&](int nbk, float* kv) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int s = 16 * w + 4 * g + r;
        kv[r] = (s < clen) ? to_f32(kin[(int64_t)s * qk_stride(a) + 16 * nbk + i]) : 0.f;
      }
    };
    float kcur[4], knext[4] = {0.f, 0.f, 0.f, 0.f};
    load_k4(0, kcur);
    const int NBK = dk / 16;
    for (int nbk = 0; nbk < NBK; ++nbk) {
      if (nbk + 1 < NBK) load_k4(nbk + 1, knext);
      f32x4 accM = {0.f, 0.f, 0.f, 0.f}, accJ = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < KSMAX; ++ks) {
        if (ks < KS) {
          const int d0 = 8 * g + 32 * ks;
          bf16x8 B3, B4;
          if (d0 < dv) {
            B3 = *(const bf16x8*)&sRT[(16 * nbk + i) * RS + d0];
            B4 = *(const bf16x8*)&sRT[(dk + 16 * nbk + i) * RS + d0];
          } else {
#pragma unroll
            for (int j = 0; j < 8; ++j) { B3[j] = (bf16_t)0.f; B4[j] = (bf16_t)0.f; }
          }
          if constexpr (PREC) {
            bf16x8 B3l = B3, B4l = B4;   // zero beyond dv
            if (d0 < dv) {
              B3l = *(const bf16x8*)&sRTl[(16 * nbk + i) * RS + d0];
              B4l = *(const bf16x8*)&sRTl[(dk + 16 * nbk + i) * RS + d0];
            }
            accM = mfma16_split(A3[ks], A3l[ks], B3, B3l, accM);
            accJ = mfma16_split(A4[ks], A4l[ks], B4, B4l, accJ);
          } else {
            accM = mfma16(A3[ks], B3, accM);
            accJ = mfma16(A4[ks], B4, accJ);
          }
        }
      }
      // rows s = 16w + 4g + r, column n = 16nbk + i
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int s = 16 * w + 4 * g + r;
        sO1[s * OS + 16 * nbk + i] = fmaf(2.f * kcur[r], accJ[r], accM[r]);
        kcur[r] = knext[r];
      }
    }
  }
  if constexpr (!EARLY) build_k();
  const int vgroups = dv >> 3;   // work item = (token, 8 value rows); the items of a token sit in adjacent lanes
  const TIn* vin = (const TIn*)a.v + tok0 * dv;
  const TIn* bin = (const TIn*)a.b + tok0 * dv;
  TIn* dvo = (TIn*)A.dv + tok0 * dv;
  TIn* dbo = (TIn*)A.db + tok0 * dv;
  // dv and its v rows for the next phase (SEQ: db and b before the second pass)
  if constexpr (PRE) {
    fetch_items(vin, vgroups, dv, in1);
    fetch_items(dvo, vgroups, dv, old2);
  }
  __syncthreads();
  {
    const int groups = dk >> 3;
    auto item = [&](int m) {
      const int idx = tid + 256 * m, c8 = idx % groups, s = idx / groups;
      if (idx < kC * groups && s < clen) {
        TIn* o = dko + (int64_t)s * H * dk + 8 * c8;
        Raw8<TIn> now;
        if constexpr (!PRE) now.load(o);
        const Raw8<TIn>& was = PRE ? old1[m] : now;
        float gk[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) gk[e] = was.get(e) + sO1[s * OS + 8 * c8 + e];
        store_vec<4>(o, gk); store_vec<4>(o + 4, gk + 4);
      }
    };
    if constexpr (PRE) {
#pragma unroll
      for (int m = 0; m < KSMAX; ++m) item(m);
    } else {
#pragma unroll 1
      for (int m = 0; m < KSMAX; ++m) item(m);
    }
  }
  if constexpr (PRE && !SEQ) {
    fetch_items(bin, vgroups, dv, in2);
    fetch_items(dbo, vgroups, dv, old1);
  }
  __syncthreads();   // sO1 is free again

  // ---- dv, db: out[s, d] = sum_n (a_s k_s[n]) R_M[d, n]
  {
    const int KS = (dk + 31) / 32;
    const int groups = vgroups;
    constexpr int NPASS = SEQ ? 2 : 1;
#pragma unroll
    for (int pass = 0; pass < NPASS; ++pass) {
      const bool doV = !SEQ || pass == 0, doB = !SEQ || pass == 1;
      for (int db_ = 0; db_ < dv / 16; ++db_) {
        f32x4 accV = {0.f, 0.f, 0.f, 0.f}, accB = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < KSMAX; ++ks) {
          if (ks < KS) {
            const int n0 = 8 * g + 32 * ks;
            bf16x8 B1, B2;
#pragma unroll
            for (int j = 0; j < 8; ++j) { B1[j] = (bf16_t)0.f; B2[j] = (bf16_t)0.f; }
            bf16x8 B1l = B1, B2l = B2;
            if constexpr (PREC) {
              if (n0 < dk) {
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                  if (doV) { B1[j] = sRT[(n0 + j) * RS + 16 * db_ + i]; B1l[j] = sRTl[(n0 + j) * RS + 16 * db_ + i]; }
                  if (doB) { B2[j] = sRT[(dk + n0 + j) * RS + 16 * db_ + i]; B2l[j] = sRTl[(dk + n0 + j) * RS + 16 * db_ + i]; }
                }
              }
              if (doV) accV = mfma16_split(A1[ks], A1l[ks], B1, B1l, accV);
              if (doB) accB = mfma16_split(A2[ks], A2l[ks], B2, B2l, accB);
              continue;
            }
            if (n0 < dk && !alias) {
              // 8 consecutive key columns of value row d = 16db_ + i: a column walk through the transposed
              // bf16 copy in LDS (the fp32 carries in global memory would miss L2 on this second read)
#pragma unroll
              for (int j = 0; j < 8; ++j) {
                if (doV) B1[j] = sRT[(n0 + j) * RS + 16 * db_ + i];
                if (doB) B2[j] = sRT[(dk + n0 + j) * RS + 16 * db_ + i];
              }
            } else if (n0 < dk) {
              const TIn* r1 = RM + (int64_t)(16 * db_ + i) * dk + n0;
              const TIn* r2 = RJ + (int64_t)(16 * db_ + i) * dk + n0;
              float x[8], y[8];
              load_vec<4>(r1, x); load_vec<4>(r1 + 4, x + 4);
              load_vec<4>(r2, y); load_vec<4>(r2 + 4, y + 4);
#pragma unroll
              for (int j = 0; j < 8; ++j) {
                B1[j] = (bf16_t)x[j];
                B2[j] = (bf16_t)y[j];
              }
            }
            if (doV) accV = mfma16(A1[ks], B1, accV);
            if (doB) accB = mfma16(A2[ks], B2, accB);
          }
        }
        // accumulator layout: rows s = 16w + 4g + r, column d = 16db_ + i
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          if (doV) sO1[(16 * w + 4 * g + r) * OS + 16 * db_ + i] = accV[r];
          if (doB) sO2[(16 * w + 4 * g + r) * OS + 16 * db_ + i] = accB[r];
        }
      }
      __syncthreads();
      // add to the tile-local dv, db; beta_s = <v_s, dv^carry_s> + <b_s, db^carry_s>
      // (SEQ: the rows of the pass are in in1/old2; else v, dv in in1/old2 and b, db in in2/old1)
      auto item = [&](int m) {
        const int idx = tid + 256 * m, c8 = idx % groups, s = idx / groups;
        if (idx < kC * groups) {
          float beta = 0.f;
          if (s < clen) {
            const int64_t off = (int64_t)s * H * dv + 8 * c8;
            if (doV) {
              Raw8<TIn> x_now, g_now;
              if constexpr (!PRE) { x_now.load(vin + off); g_now.load(dvo + off); }
              const Raw8<TIn>& xv = PRE ? in1[m] : x_now;
              const Raw8<TIn>& gvo = PRE ? old2[m] : g_now;
              float gv[8];
#pragma unroll
              for (int e = 0; e < 8; ++e) {
                const float cv = sO1[s * OS + 8 * c8 + e];
                beta = fmaf(xv.get(e), cv, beta);
                gv[e] = gvo.get(e) + cv;
              }
              store_vec<4>(dvo + off, gv); store_vec<4>(dvo + off + 4, gv + 4);
            }
            if (doB) {
              Raw8<TIn> x_now, g_now;
              if constexpr (!PRE) { x_now.load(bin + off); g_now.load(dbo + off); }
              const Raw8<TIn>& xb = PRE ? (SEQ ? in1[m] : in2[m]) : x_now;
              const Raw8<TIn>& gbo = PRE ? (SEQ ? old2[m] : old1[m]) : g_now;
              float gb[8];
#pragma unroll
              for (int e = 0; e < 8; ++e) {
                const float cb = sO2[s * OS + 8 * c8 + e];
                beta = fmaf(xb.get(e), cb, beta);
                gb[e] = gbo.get(e) + cb;
              }
              store_vec<4>(dbo + off, gb); store_vec<4>(dbo + off + 4, gb + 4);
            }
          }
          // the second pass of SEQ adds to the share the same thread left in the first
          sBt[idx] = (SEQ && pass == 1) ? sBt[idx] + beta : beta;
        }
      };
      if constexpr (PRE) {
#pragma unroll
        for (int m = 0; m < KSMAX; ++m) item(m);
      } else {
#pragma unroll 1
        for (int m = 0; m < KSMAX; ++m) item(m);
      }
      if (PRE && SEQ && pass == 0) {
        fetch_items(bin, groups, dv, in1);
        fetch_items(dbo, groups, dv, old2);
      }
      __syncthreads();   // SEQ: the result buffer is free for the next pass; last pass: sBt is complete
    }
    if (w == 0) {
      float bsum = 0.f;
      if (tok_ok)
        for (int c8 = 0; c8 < groups; ++c8) bsum += sBt[lane * groups + c8];   // fixed order
      gate_grad(bsum, bnd);
    }
  }
}

// ----------------------------------------------------------------- head sums
// dg[h] = sum over the tiles of their shares; dIp[h] = sum over the tiles of the local terms and, with an initial
// state, - sum dJ_0 (J_0 = I_0 - Ip).  One wave per head, lane-strided then over the lanes (fixed order), in double.
__global__ __launch_bounds__(64) void chunk_bwd_head_reduce_kernel(BwdArgs A) {
  const ChunkArgs& a = A.c;
  const int h = blockIdx.x, lane = threadIdx.x;
  double sg = 0.0, si = 0.0;
  for (int c = lane; c < a.total_chunks; c += 64) {
    sg += (double)A.wDgTile[(int64_t)c * a.H + h];
    si += (double)A.wSig[(int64_t)c * a.H + h];
  }
  if (a.init_mu) {
    const int nblk = carry_scan_blocks((int64_t)a.dv * a.dk);
    for (int j = lane; j < a.n_seqs * nblk; j += 64) {
      const int n = j / nblk, b2 = j - n * nblk;
      si -= (double)A.wInitPart[((int64_t)n * a.H + h) * nblk + b2];
    }
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    sg += __shfl_xor(sg, off);
    si += __shfl_xor(si, off);
  }
  if (lane == 0) {
    A.dg[h] = (float)sg;
    A.dIp[h] = (float)si;
  }
}

struct BwdLayout {
  size_t oDM, oDJ, oFtot, oSig, oE, oInit, oDgTile, oDqFull, oDkFull, total;
};

// dq, dk of a q/k head shared by `rep` value heads: the kernels leave one row per value head ([tokens, H, dk]) in the
// workspace, this adds the rows of a group in a fixed order (fp32) into the caller's [tokens, Hq, dk].
template <typename T>
__global__ __launch_bounds__(256) void group_sum_kernel(const T* src_q, const T* src_k, T* dst_q, T* dst_k, int64_t n4,
                                                        int Hq, int rep, int dk) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;   // four consecutive columns of one (token, q/k head) row
  if (idx >= n4) return;
  const int per = dk >> 2;
  const int c4 = (int)(idx % per);
  const int64_t row = idx / per;                                 // token * Hq + hq
  const int64_t tok = row / Hq;
  const int hq = (int)(row - tok * Hq);
  float aq[4] = {0.f, 0.f, 0.f, 0.f}, ak[4] = {0.f, 0.f, 0.f, 0.f};
  for (int r = 0; r < rep; ++r) {
    const int64_t so = ((tok * Hq + hq) * rep + r) * (int64_t)dk + 4 * c4;   // value head hq * rep + r
    float x[4], y[4];
    load_vec<4>(src_q + so, x);
    load_vec<4>(src_k + so, y);
#pragma unroll
    for (int e = 0; e < 4; ++e) { aq[e] += x[e]; ak[e] += y[e]; }
  }
  store_vec<4>(dst_q + row * dk + 4 * c4, aq);
  store_vec<4>(dst_k + row * dk + 4 * c4, ak);
}

// dq, dk of [tokens, Hq * rep, dk] summed over the rep value heads of each group into [tokens, Hq, dk]
int launch_group_sum(const void* src_q, const void* src_k, void* dst_q, void* dst_k, int64_t tokens, int Hq, int rep, int dk,
                     int dtype, hipStream_t s) {
  const int64_t n4 = tokens * Hq * (dk / 4);
  if ((n4 + 255) / 256 > 0x7fffffff) return PAL_E_DIM;
  const unsigned gblocks = (unsigned)((n4 + 255) / 256);
  if (dtype == PAL_DTYPE_BF16)
    hipLaunchKernelGGL(group_sum_kernel<bf16_t>, dim3(gblocks), dim3(256), 0, s, (const bf16_t*)src_q, (const bf16_t*)src_k,
                       (bf16_t*)dst_q, (bf16_t*)dst_k, n4, Hq, rep, dk);
  else
    hipLaunchKernelGGL(group_sum_kernel<float>, dim3(gblocks), dim3(256), 0, s, (const float*)src_q, (const float*)src_k,
                       (float*)dst_q, (float*)dst_k, n4, Hq, rep, dk);
  PAL_HIP_LAUNCH_CHECK();
  return PAL_OK;
}

static size_t align256(size_t x) { return (x + 255) & ~(size_t)255; }

static BwdLayout bwd_layout(const PalDims* d) {
  BwdLayout L;
  const size_t E = (size_t)d->dv * d->dk;
  const size_t tiles = (size_t)d->total_chunks * d->n_heads;
  const size_t tokens = (size_t)d->batch * d->seq_len;
  size_t o = 0;
  L.oDM = o; o = align256(o + tiles * E * 4);
  L.oDJ = o; o = align256(o + tiles * E * 4);
  L.oFtot = o; o = align256(o + tiles * 4);
  L.oSig = o; o = align256(o + tiles * 4);
  L.oE = o; o = align256(o + tokens * d->n_heads * 4);
  L.oInit = o; o = align256(o + (size_t)d->n_seqs * d->n_heads * (E / 256) * 4);
  L.oDgTile = o; o = align256(o + tiles * 4);
  L.oDqFull = L.oDkFull = o;
  if (d->n_qk_heads > 0 && d->n_qk_heads != d->n_heads) {
    const size_t full = tokens * d->n_heads * d->dk * (d->dtype == PAL_DTYPE_BF16 ? 2 : 4);
    L.oDqFull = o; o = align256(o + full);
    L.oDkFull = o; o = align256(o + full);
  }
  L.total = o;
  return L;
}

// Launch shapes that depend on the head dims only; worked out before the first launch so that a head-dim pair the
// backward cannot serve is refused while nothing has been enqueued.
struct BwdPlan {
  int nb_local;        // column blocks per pass of the tile kernel
  size_t lds_local;
  size_t lds_apply;
  int apply_alias, apply_seq, apply_ksmax;
};

static size_t local_lds_bytes(int NB, bool var, bool prec) {
  const int DG = local_dg(NB, prec);
  return sizeof(float) * (2 * kC + 2 * (var ? 4 : 3) * DG * kVS2 + 2 * NB * DG * kC + NB * 288 + NB * DG * 32) +
         (size_t)NB * 20 * (prec ? 2 : 1) * 64 * 16;
}

// prec: the fp32-accurate variants (fp32 rows without PAL_FLAG_FP32_FAST)
static int bwd_plan(int dk, int dv, bool var, bool prec, BwdPlan& P) {
  const int nb_total = dk / 16;
  if (nb_total < 1 || nb_total > 16) return PAL_E_HEADDIM;
  // At most 4 column blocks (16 waves, 128 registers each: one workgroup per compute unit) in flight; wider heads
  // take several passes.  Passes of 4 blocks when they divide the head dim, else passes of 2: two workgroups of
  // 8 waves then share a compute unit and fill each other's barrier waits, which measured 14-17 % faster than
  // passes of 3 (12 waves, one workgroup per unit) at dk = 80 and 96 and the same as 4 + 3 at dk = 112.
  P.nb_local = nb_total <= 4 ? nb_total : (nb_total % 4 == 0 ? 4 : 2);
  if (prec && P.nb_local > 2) P.nb_local = 2;   // 16-operand slots: at most two column blocks fit the LDS
  P.lds_local = local_lds_bytes(P.nb_local, var, prec);
  if (P.lds_local > kMaxLds) return PAL_E_HEADDIM;
  const int dmax = dk > dv ? dk : dv;
  const size_t rt_bytes = (prec ? 2 : 1) * 2 * (size_t)2 * dk * (dv + 8), o_bytes = sizeof(float) * kC * (dmax + 4);
  if (prec && dmax > 128) return PAL_E_HEADDIM;
  const size_t lds_fixed = sizeof(float) * (kC + 8 + kC * (dv >> 3)) + o_bytes;
  size_t lds = lds_fixed + o_bytes + rt_bytes;
  P.apply_alias = 0;
  if (lds > kMaxLds && !prec) {
    P.apply_alias = 1;
    lds = lds_fixed + (rt_bytes > o_bytes ? rt_bytes : o_bytes);
  }
  // one result buffer used twice when that lets more workgroups share a compute unit
  const size_t lds_seq = lds_fixed + rt_bytes;
  P.apply_seq = lds_seq <= kMaxLds && kMaxLds / lds_seq > (lds > kMaxLds ? 0 : kMaxLds / lds);
  if (P.apply_seq) { lds = lds_seq; P.apply_alias = 0; }
  if (lds > kMaxLds) return PAL_E_HEADDIM;
  P.lds_apply = lds;
  P.apply_ksmax = dmax <= 64 ? 2 : dmax <= 128 ? 4 : 8;
  return PAL_OK;
}

template <typename TIn, int NB, bool PREC>
static int launch_local_nb(const BwdArgs& A, hipStream_t s) {
  const bool var = A.c.flags & PAL_FLAG_HAS_VAR;
  const int64_t blocks = (int64_t)A.c.total_chunks * A.c.H;
  if (blocks > 0x7fffffff) return PAL_E_DIM;
  // four wave roles per block of 16 key columns, NB such blocks at a time (see chunk_bwd_local_roles_kernel)
  const int NT = 4 * NB * 64;
  const size_t lds = local_lds_bytes(NB, var, PREC);
  if (lds > kMaxLds) return PAL_E_HEADDIM;
  const bool multi = A.c.dk != 16 * NB;
  auto go = [&](auto kern) -> int {
    if (int rc = allow_lds((const void*)kern, lds)) return rc;
    PAL_TIMED_LAUNCH(kKernBwdLocal, s, kern, dim3((unsigned)blocks), dim3(NT), lds, s, A);
    return 0;
  };
  int rc;
  if constexpr (NB == 2 || NB == 4) {   // the only block counts that run several passes (see bwd_plan)
    if (multi) rc = var ? go(&chunk_bwd_local_roles_kernel<TIn, NB, true, true, PREC>) : go(&chunk_bwd_local_roles_kernel<TIn, NB, false, true, PREC>);
    else rc = var ? go(&chunk_bwd_local_roles_kernel<TIn, NB, true, false, PREC>) : go(&chunk_bwd_local_roles_kernel<TIn, NB, false, false, PREC>);
  } else {
    rc = var ? go(&chunk_bwd_local_roles_kernel<TIn, NB, true, false, PREC>) : go(&chunk_bwd_local_roles_kernel<TIn, NB, false, false, PREC>);
  }
  if (rc) return rc;
  PAL_HIP_LAUNCH_CHECK();
  return PAL_OK;
}

template <typename TIn, bool PREC>
static int launch_local(const BwdArgs& A, const BwdPlan& P, hipStream_t s) {
  switch (P.nb_local) {
    case 1: return launch_local_nb<TIn, 1, PREC>(A, s);
    case 2: return launch_local_nb<TIn, 2, PREC>(A, s);
    case 3: if constexpr (!PREC) return launch_local_nb<TIn, 3, false>(A, s); else return PAL_E_HEADDIM;
    case 4: if constexpr (!PREC) return launch_local_nb<TIn, 4, false>(A, s); else return PAL_E_HEADDIM;
    default: return PAL_E_HEADDIM;
  }
}

template <typename TIn, int KSMAX, bool SEQ, bool PREC>
static int launch_carry_apply_t(const BwdArgs& A, unsigned blocks, size_t lds, hipStream_t s) {
  if (int rc = allow_lds((const void*)&chunk_bwd_carry_apply_kernel<TIn, KSMAX, SEQ, PREC>, lds)) return rc;
  PAL_TIMED_LAUNCH(kKernBwdCarryApply, s, (chunk_bwd_carry_apply_kernel<TIn, KSMAX, SEQ, PREC>), dim3(blocks), dim3(256), lds, s, A);
  PAL_HIP_LAUNCH_CHECK();
  return PAL_OK;
}
template <typename TIn, bool PREC>
static int launch_carry_apply(const BwdArgs& A, int ksmax, bool seq, unsigned blocks, size_t lds, hipStream_t s) {
  if (ksmax == 2) return seq ? launch_carry_apply_t<TIn, 2, true, PREC>(A, blocks, lds, s) : launch_carry_apply_t<TIn, 2, false, PREC>(A, blocks, lds, s);
  if (ksmax == 4) return seq ? launch_carry_apply_t<TIn, 4, true, PREC>(A, blocks, lds, s) : launch_carry_apply_t<TIn, 4, false, PREC>(A, blocks, lds, s);
  if constexpr (PREC) return PAL_E_HEADDIM;   // the split operands of 256-wide heads do not fit the registers
  else return seq ? launch_carry_apply_t<TIn, 8, true, false>(A, blocks, lds, s) : launch_carry_apply_t<TIn, 8, false, false>(A, blocks, lds, s);
}

}  // namespace pal

extern "C" size_t pal_chunk_bwd_workspace_bytes(const PalDims* d) {
  if (pal_validate_dims(d) != PAL_OK || d->total_chunks <= 0) return 0;
  pal::BwdPlan P;
  const bool prec = d->dtype == PAL_DTYPE_F32 && !(d->flags & PAL_FLAG_FP32_FAST);
  if (pal::bwd_plan(d->dk, d->dv, (d->flags & PAL_FLAG_HAS_VAR) != 0, prec, P) != PAL_OK) return 0;
  return pal::bwd_layout(d).total;
}

extern "C" int pal_chunk_bwd_supported(int32_t dk, int32_t dv, int32_t dtype, uint32_t flags) {
  if (dk < 16 || dk > 256 || (dk & 15) || dv < 16 || dv > 256 || (dv & 15)) return PAL_E_HEADDIM;
  if (dtype != PAL_DTYPE_F32 && dtype != PAL_DTYPE_BF16) return PAL_E_DTYPE;
  pal::BwdPlan P;
  return pal::bwd_plan(dk, dv, true, dtype == PAL_DTYPE_F32 && !(flags & PAL_FLAG_FP32_FAST), P);
}

extern "C" int pal_chunk_bwd(const PalDims* d, const PalFwdTensors* t, const PalBwdTensors* gr, void* workspace,
                             size_t workspace_bytes, void* stream) {
  using namespace pal;
  if (!d || !t) return PAL_E_NULL;
  // the forward-side struct is reused with o pointing at any valid buffer; final states are not needed
  PalDims dd = *d;
  dd.flags &= ~PAL_FLAG_STORE_FINAL;
  PalFwdTensors tt = *t;
  tt.final_mu = tt.final_I = nullptr;
  if (!tt.o) tt.o = gr ? (void*)gr->d_o : nullptr;
  if ((dd.flags & PAL_FLAG_HAS_VAR) && !tt.o_var) tt.o_var = gr ? (void*)gr->d_o_var : nullptr;
  int rc = check_chunk_common(&dd, &tt);
  if (rc) return rc;
  rc = check_bwd_common(&dd, gr);
  if (rc) return rc;
  BwdPlan P;
  const bool prec = dd.dtype == PAL_DTYPE_F32 && !(dd.flags & PAL_FLAG_FP32_FAST);
  rc = bwd_plan(dd.dk, dd.dv, (dd.flags & PAL_FLAG_HAS_VAR) != 0, prec, P);
  if (rc) return rc;
  if ((int64_t)dd.total_chunks * dd.n_heads > 0x7fffffff ||
      (int64_t)dd.n_seqs * dd.n_heads * carry_scan_blocks((int64_t)dd.dv * dd.dk) > 0x7fffffff)
    return PAL_E_DIM;
  const BwdLayout L = bwd_layout(&dd);
  if (!workspace || workspace_bytes < L.total || !is_aligned16(workspace)) return PAL_E_WORKSPACE;
  BwdArgs A;
  fill_chunk_args(A.c, &dd, &tt);
  A.d_o = gr->d_o;
  A.d_o_var = (dd.flags & PAL_FLAG_HAS_VAR) ? gr->d_o_var : nullptr;
  A.dq = gr->dq; A.dk = gr->dk; A.dv = gr->dv; A.db = gr->db;
  const bool grouped = A.c.Hq != A.c.H;
  if (grouped) {   // one row per value head first, summed over each group at the end
    A.dq = (char*)workspace + L.oDqFull;
    A.dk = (char*)workspace + L.oDkFull;
  }
  A.dgt = gr->dgt; A.dg = gr->dg; A.dIp = gr->dIp;
  A.d_init_mu = gr->d_init_mu; A.d_init_I = gr->d_init_I;
  char* ws = (char*)workspace;
  A.wDM = ws + L.oDM; A.wDJ = ws + L.oDJ;
  A.wFtot = (float*)(ws + L.oFtot); A.wSig = (float*)(ws + L.oSig);
  A.wE = (float*)(ws + L.oE); A.wInitPart = (float*)(ws + L.oInit);
  A.wDgTile = (float*)(ws + L.oDgTile);
  A.tokens = dd.batch * dd.seq_len;
  hipStream_t s = (hipStream_t)stream;
  const bool bf = dd.dtype == PAL_DTYPE_BF16;
  rc = bf ? launch_local<bf16_t, false>(A, P, s) : prec ? launch_local<float, true>(A, P, s) : launch_local<float, false>(A, P, s);
  if (rc) return rc;
  {
    const int64_t blocks = (int64_t)dd.n_seqs * dd.n_heads * carry_scan_blocks((int64_t)dd.dv * dd.dk);
    if (blocks > 0x7fffffff) return PAL_E_DIM;
    if (bf) PAL_TIMED_LAUNCH(kKernBwdCarryScan, s, chunk_bwd_carry_scan_kernel<bf16_t>, dim3((unsigned)blocks), dim3(256), 0, s, A);
    else PAL_TIMED_LAUNCH(kKernBwdCarryScan, s, chunk_bwd_carry_scan_kernel<float>, dim3((unsigned)blocks), dim3(256), 0, s, A);
    PAL_HIP_LAUNCH_CHECK();
  }
  {
    const unsigned blocks = (unsigned)((int64_t)dd.total_chunks * dd.n_heads);
    A.apply_alias = P.apply_alias;
    rc = bf     ? launch_carry_apply<bf16_t, false>(A, P.apply_ksmax, P.apply_seq != 0, blocks, P.lds_apply, s)
         : prec ? launch_carry_apply<float, true>(A, P.apply_ksmax, P.apply_seq != 0, blocks, P.lds_apply, s)
                : launch_carry_apply<float, false>(A, P.apply_ksmax, P.apply_seq != 0, blocks, P.lds_apply, s);
    if (rc) return rc;
    PAL_HIP_LAUNCH_CHECK();
  }
  PAL_TIMED_LAUNCH(kKernBwdHeadReduce, s, chunk_bwd_head_reduce_kernel, dim3((unsigned)dd.n_heads), dim3(64), 0, s, A);
  PAL_HIP_LAUNCH_CHECK();
  if (grouped) {
    if (int rc2 = launch_group_sum(A.dq, A.dk, gr->dq, gr->dk, A.tokens, A.c.Hq, A.c.H / A.c.Hq, dd.dk, dd.dtype, s)) return rc2;
  }
  return PAL_OK;
}
