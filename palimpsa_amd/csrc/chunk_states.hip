// Tile-start states of the chunked algorithm in one pass (bf16 rows):
//     S_c = F_c S_{c-1} + Delta_c ,  Delta_c = sum_s a_s v_s k_s^T  (and sum_s a_s b_s (k_s*k_s)^T for the
//     precision state)
// computed by a workgroup that walks the tiles of one sequence in order with the running state in the
// accumulators of the matrix cores, so that the per-tile contributions Delta_c never go to memory (the
// two-kernel form, chunk_delta_kernel + a scan kernel, writes them in fp32 and reads them back: three times
// the bytes of the states themselves).  What the reference keeps as intermediate_*_state
// (chunk_palimpsa_forgetting_scalar.py:187-188) is written at the start of every tile, the state after
// the last tile at the end (:214-218).
//
// One workgroup of 12 waves per (sequence, head, slice of ds value rows): four hold the state (the slice times
// dk is at most 6144 entries = 24 blocks of 16x16, up to six per wave), two groups of four stage the rows for them.  The rows of a tile are staged transposed in LDS
// (token index fastest, two tokens per 32-bit word) as in chunk_delta_kernel.  The serial chain over the tiles
// is hidden by fetching ahead: rows are fetched into registers three steps before they go to LDS, two LDS
// buffers hold the current and the next tile, one barrier per tile.
// The same kernel walks a sequence backwards for the gradient of the scalar-gated path (weights from the
// start of the tile, G_{c-1} = F_c G_c + D_c, the value left after the first tile is the gradient of the
// initial state).
#include <type_traits>

#include "chunk_common.h"
#include "pal_host.h"
#include "pal_profile.h"

namespace pal {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int kStTS = 72;          // tokens (bf16) per staged row: 64 + 8 keeps 16-byte reads conflict-free
constexpr int kStMaxBlocks = 6;    // 16x16 state blocks per wave

struct StatePassArgs {
  ChunkArgs c;
  void* tiles_a;          // scalar-gated: bf16 tile states; Palimpsa: fp32 mu at the start of every tile
  float* tiles_b;         // Palimpsa: fp32 I at the start of every tile
  const float *init_a, *init_b;
  float *fin_a, *fin_b;
  int32_t ds, nsplit, reverse, per_xcd, total;
  int32_t dks, ksplit;    // key columns per workgroup and slices of the key columns (dk = dks * ksplit)
  int32_t by_length;      // packed sequences are handed out longest first (see the kernel)
  float fin_scale;
};

template <int NIK>
struct StageRegs {
  u32x4 k[NIK][2];
  u32x4 v[2], b[2];
  uint32_t gt;   // gate of token `lane` as loaded: fp32 bits or a bf16 in the low half (last wave)
};

template <bool HAS_J, int NIK>
__global__ __launch_bounds__(768) void chunk_states_kernel(StatePassArgs A) {
  const ChunkArgs& a = A.c;
  extern __shared__ float smem[];
  const int tid = threadIdx.x, lane = tid & 63, i = lane & 15, g = lane >> 4;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int H = a.H, dk = a.dk, dv = a.dv, ds = A.ds, dks = A.dks;
  // consecutive workgroup ids go to different XCDs: give the slices of one (sequence, head) to the same one,
  // they read the same key rows.  A workgroup owns the state entries (value rows [d0, d0 + ds)) x (key columns
  // [k0, k0 + dks)) of a (sequence, head).
  const int n_sl = A.nsplit * A.ksplit;
  const int xcd = (int)blockIdx.x & 7, pos = (int)blockIdx.x >> 3;
  int m, n;
  if (A.by_length) {
    // Packed sequences of unequal length (at most 64): the walk over a sequence's tiles is serial, so a long sequence
    // that starts late ends the kernel late.  The sequence of rank r in descending length goes to XCD r mod 8, in
    // rank order there; every wave finds the sequence of its rank with one lane per sequence.
    const int rank = (pos / (H * n_sl)) * 8 + xcd;
    if (rank >= a.n_seqs) return;
    int b_l = 0, len_l = -1;
    if (lane < a.n_seqs) packed_seq_bounds(a.cu_seqlens, lane, a.T, b_l, len_l);
    int before = 0;   // sequences ahead of lane's own in the order (longer, or as long with a smaller index)
    for (int j = 0; j < a.n_seqs; ++j) {
      const int len_j = __builtin_amdgcn_readlane(len_l, j);
      before += (len_j > len_l || (len_j == len_l && j < lane)) ? 1 : 0;
    }
    const uint64_t hit = __ballot(lane < a.n_seqs && before == rank);
    n = hit ? (int)__builtin_ctzll(hit) : 0;
    m = n * H * n_sl + pos % (H * n_sl);
  } else {
    m = xcd * A.per_xcd + pos;
    if (m >= A.total) return;
    n = (m / n_sl) / H;
  }
  const int sl = m % n_sl;
  const int d0 = (sl / A.ksplit) * ds, k0 = (sl % A.ksplit) * dks;
  const int h = (m / n_sl) % H;
  const int nh = n * H + h;
  int bos, len, cbase;
  seq_lookup(a, n, bos, len, cbase);
  const int nchunks = (len + kC - 1) / kC;

  float* sA = smem;                                   // [3][64] weight of token s in its tile (ring over tiles)
  float* sF = sA + 3 * kC;                            // [3] decay over the whole tile (+1 pad)
  uint32_t* sKT = (uint32_t*)(sF + 4);                // [2][dks][36] words = [dks][72] bf16
  uint32_t* sVT = sKT + 2 * dks * (kStTS / 2);        // [2][ds][36]
  uint32_t* sBT = sVT + 2 * ds * (kStTS / 2);         // [2][ds][36] (HAS_J)
  const int kbuf = dks * (kStTS / 2), vbuf = ds * (kStTS / 2);


  // Waves 0-3 own the state (a 16x16 block per wave and slot), waves 4-11 feed them: a single wave issues an
  // instruction every five to eight cycles, so the kinds of work sit on different waves of each SIMD instead
  // of following one another.  The feeding waves form two groups of four, one for the even tiles (LDS buffer
  // 0) and one for the odd tiles (buffer 1): a group works out the weights of a tile and fetches ahead in one
  // step, and puts the tile's rows into its buffer in the next, while the other group does the opposite.
  // All roles pass the same barriers, one per step; steps -2 and -1 fill the pipeline.
  if (w >= 4) {
    // ---------------------------------------------------------------- staging role
    // Items of a thread: (token pair, 8 columns).  The key and the value items start at thread 0 of the group,
    // the items of b follow those of v (wrapping around), and the last wave turns the gates of a tile into its
    // weights (in the step in which the group stages nothing).  Byte offsets of the two tokens from the first row of a tile and word offsets in the
    // staging tiles do not change from tile to tile.
    const int grp = (w - 4) >> 2;           // parity of the tiles this group stages
    const int wg = (w - 4) & 3;             // wave in the group
    const int st = tid - 256 - 256 * grp;
    const int gk = dks >> 3, gv = ds >> 3;
    int ksp[NIK];
    uint32_t koff[NIK][2], kdst[NIK];
    bool kval[NIK];
#pragma unroll
    for (int j = 0; j < NIK; ++j) {
      const int idx = st + 256 * j;
      kval[j] = idx < 32 * gk;
      ksp[j] = idx / gk;
      const int c8 = idx - ksp[j] * gk;
      koff[j][0] = kval[j] ? (uint32_t)(((2 * ksp[j]) * a.Hq * dk + k0 + 8 * c8) * 2) : 0x80000000u;
      koff[j][1] = kval[j] ? (uint32_t)(((2 * ksp[j] + 1) * a.Hq * dk + k0 + 8 * c8) * 2) : 0x80000000u;
      kdst[j] = (uint32_t)(8 * c8 * (kStTS / 2) + ksp[j]);
    }
    const int vtid = st, btid = (st + 256 - 32 * gv) & 255;
    const bool vval = vtid < 32 * gv, bval = HAS_J && btid < 32 * gv;
    const int vsp = vtid / gv, vc8 = vtid - vsp * gv, bsp = btid / gv, bc8 = btid - bsp * gv;
    uint32_t voff[2], boff[2];
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      voff[u] = vval ? (uint32_t)(((2 * vsp + u) * H * dv + 8 * vc8) * 2) : 0x80000000u;
      boff[u] = bval ? (uint32_t)(((2 * bsp + u) * H * dv + 8 * bc8) * 2) : 0x80000000u;
    }
    const uint32_t vdst = (uint32_t)(8 * vc8 * (kStTS / 2) + vsp), bdst = (uint32_t)(8 * bc8 * (kStTS / 2) + bsp);
    // Rows are fetched through buffer descriptors that end with the last row of the sequence: the byte offset
    // of a row piece is a per-thread constant plus the offset of the tile, rows beyond the end of the sequence
    // (the tail of its last tile, tiles past its end) are out of range and read as zero, so no fetch needs a
    // branch or a select.  Nothing touches a fetched value before it goes to LDS: any use here would make the
    // wave wait for everything it has in flight, which is what fetching ahead is meant to avoid.
    const bf16_t* kbase = (const bf16_t*)a.k + qk_row(a, bos, h);
    const bf16_t* vbase = (const bf16_t*)a.v + ((int64_t)bos * H + h) * dv + d0;
    const int esz = a.gate_bf16 ? 2 : 4;
    const uint32_t kbytes = len > 0 ? (uint32_t)(((len - 1) * a.Hq * dk + dk) * 2) : 0u;
    const uint32_t vbytes = len > 0 ? (uint32_t)(((len - 1) * H * dv + ds) * 2) : 0u;
    const uint32_t gbytes = len > 0 ? (uint32_t)(((len - 1) * H + 1) * esz) : 0u;
    const __amdgpu_buffer_rsrc_t krs = __builtin_amdgcn_make_buffer_rsrc((void*)kbase, 0, kbytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t vrs = __builtin_amdgcn_make_buffer_rsrc((void*)vbase, 0, vbytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t brs = __builtin_amdgcn_make_buffer_rsrc(
        HAS_J ? (void*)((const bf16_t*)a.b + ((int64_t)bos * H + h) * dv + d0) : (void*)vbase, 0, vbytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t grs = __builtin_amdgcn_make_buffer_rsrc(
        (void*)((const char*)a.gt + ((int64_t)bos * H + h) * esz), 0, gbytes, 0x00020000);
    const uint32_t goff = (uint32_t)(lane * H * esz);
    const float gh = a.g[h] * kLog2e;
    const bool from_start = (a.flags & kFlagDecayFromStart) != 0;

    auto load_stage = [&](StageRegs<NIK>& R, int p) {
      const int c = A.reverse ? nchunks - 1 - p : p;
      const bool live = p < nchunks;
      // a tile past the end: every offset out of range
      const uint32_t tk = live ? (uint32_t)(c * kC * a.Hq * dk * 2) : 0x80000000u;
      const uint32_t tv = live ? (uint32_t)(c * kC * H * dv * 2) : 0x80000000u;
#pragma unroll
      for (int j = 0; j < NIK; ++j) {
        R.k[j][0] = __builtin_amdgcn_raw_buffer_load_b128(krs, koff[j][0] + tk, 0, 0);
        R.k[j][1] = __builtin_amdgcn_raw_buffer_load_b128(krs, koff[j][1] + tk, 0, 0);
      }
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        R.v[u] = __builtin_amdgcn_raw_buffer_load_b128(vrs, voff[u] + tv, 0, 0);
        if (HAS_J) R.b[u] = __builtin_amdgcn_raw_buffer_load_b128(brs, boff[u] + tv, 0, 0);
      }
      if (wg == 3) {
        const uint32_t tg = live ? (uint32_t)(c * kC * H * esz) : 0x80000000u;
        R.gt = a.gate_bf16 ? (uint32_t)__builtin_amdgcn_raw_buffer_load_b16(grs, goff + tg, 0, 0)
                           : __builtin_amdgcn_raw_buffer_load_b32(grs, goff + tg, 0, 0);   // raw; widened below
      }
    };
    // eight columns of two tokens -> one word (token pair) per column
    auto put = [&](uint32_t* dst, const u32x4& x0, const u32x4& x1) {
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const uint32_t sel = (e & 1) ? 0x07060302u : 0x05040100u;
        dst[e * (kStTS / 2)] = __builtin_amdgcn_perm(x1[e >> 1], x0[e >> 1], sel);
      }
    };
    // the same for rows of v and b, which are staged times the weight of their token (the operand the matrix
    // cores take is a_s v_s, rounded to bf16 once)
    auto put_weighted = [&](uint32_t* dst, const u32x4& x0, const u32x4& x1, int sp, const float* wts) {
      const f32x2 a2 = *(const f32x2*)&wts[2 * sp];
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const uint32_t w0 = x0[e >> 1], w1 = x1[e >> 1];
        const float f0 = __builtin_bit_cast(float, (e & 1) ? (w0 & 0xffff0000u) : (w0 << 16));
        const float f1 = __builtin_bit_cast(float, (e & 1) ? (w1 & 0xffff0000u) : (w1 << 16));
        *(bf16x2*)&dst[e * (kStTS / 2)] = pack2(f0 * a2[0], f1 * a2[1]);
      }
    };
    auto store_stage = [&](const StageRegs<NIK>& R, int buf, int p) {
#pragma unroll
      for (int j = 0; j < NIK; ++j)
        if (kval[j]) put(sKT + buf * kbuf + kdst[j], R.k[j][0], R.k[j][1]);
      const float* wts = sA + (p % 3) * kC;
      if (vval) put_weighted(sVT + buf * vbuf + vdst, R.v[0], R.v[1], vsp, wts);
      if (HAS_J && bval) put_weighted(sBT + buf * vbuf + bdst, R.b[0], R.b[1], bsp, wts);
    };
    // weights of the tokens of tile p and the decay over the whole tile, one step before its rows are staged
    auto scan_stage = [&](const StageRegs<NIK>& R, int p) {
      if (wg == 3) {
        const float gt = __builtin_bit_cast(float, a.gate_bf16 ? R.gt << 16 : R.gt);   // zero beyond the sequence
        const float cs = wave_inclusive_scan(-gt * gh, lane);
        const float tot = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, cs), 63));
        sA[(p % 3) * kC + lane] = fast_exp2(from_start ? cs : tot - cs);
        if (lane == 0) sF[p % 3] = fast_exp2(tot);
      }
    };

    // Two register sets per group: the tile being staged and the group's next one (two tiles later), which is
    // fetched three steps before its rows go to LDS.  In step p the group of parity (p + 1) & 1 stages tile p + 1,
    // the other one handles tile p + 2: weights from its gates (set (p + 2) / 2 % 2), then the fetch of tile p + 4
    // into the set that was staged a step ago.
    // (One copy of the loop per group: with the group a compile-time constant the order of fetches and uses is
    // static, and the compiler can count how many younger fetches may still be in flight when a set is used;
    // with a run-time test it has to wait for all of them, which throws the fetching ahead away.)
    auto run = [&](auto parity) {
      constexpr int G = decltype(parity)::value;
      StageRegs<NIK> R[2];
      load_stage(R[0], G);
      for (int p0 = -2; p0 < nchunks; p0 += 4) {
#pragma unroll
        for (int ph = 0; ph < 4; ++ph) {
          const int p = p0 + ph;           // p + 2 = ph (mod 4)
          if ((ph & 1) == G) {   // folds once the loop is unrolled
            scan_stage(R[(ph >> 1) & 1], p + 2);
            load_stage(R[1 - ((ph >> 1) & 1)], p + 4);
          } else {
            if (p + 1 >= 0) store_stage(R[(((ph + 3) & 3) >> 1) & 1], G, p + 1);
          }
          __syncthreads();
        }
      }
    };
    if (grp == 0) run(std::integral_constant<int, 0>{});
    else run(std::integral_constant<int, 1>{});
    return;
  }

  // ------------------------------------------------------------------ state role
  // state blocks of this wave: block sb = w + 4 jj -> (value rows 16 db.., key columns 16 nb..)
  const int NB = dks >> 4, NSB = (ds >> 4) * NB;
  int ldk[kStMaxBlocks], ldv[kStMaxBlocks], goff[kStMaxBlocks];   // operand rows in the staging tiles, entry in a state
  bool sval[kStMaxBlocks];
  f32x4 accM[kStMaxBlocks], accJ[kStMaxBlocks];
  const int64_t E = (int64_t)dv * dk;
  const float Ip = HAS_J ? a.Ip[h] : 0.f;
#pragma unroll
  for (int jj = 0; jj < kStMaxBlocks; ++jj) {
    const int sb = w + 4 * jj;
    sval[jj] = sb < NSB;
    const int db = sb / NB, nb = sb - db * NB;
    // rows n = 16 nb + 4 g + r (four consecutive key columns), column d = d0 + 16 db + i
    ldk[jj] = (16 * nb + i) * kStTS + 8 * g;
    ldv[jj] = (16 * db + i) * kStTS + 8 * g;
    goff[jj] = (d0 + 16 * db + i) * dk + k0 + 16 * nb + 4 * g;
    accM[jj] = f32x4{0.f, 0.f, 0.f, 0.f};
    accJ[jj] = f32x4{0.f, 0.f, 0.f, 0.f};
    if (sval[jj] && A.init_a) {
      const int64_t off = (int64_t)nh * E + goff[jj];
      const f32x4 x = *(const f32x4*)(A.init_a + off);
      if (HAS_J) {
        const f32x4 I = *(const f32x4*)(A.init_b + off);
#pragma unroll
        for (int r = 0; r < 4; ++r) { accM[jj][r] = x[r] * I[r]; accJ[jj][r] = I[r] - Ip; }
      } else {
        accM[jj] = x;
      }
    }
  }
  __syncthreads();   // steps -2 and -1 of the feeding waves
  __syncthreads();
  for (int p = 0; p < nchunks; ++p) {
    const int buf = p & 1;
    const int c = A.reverse ? nchunks - 1 - p : p;
    const int64_t slot = ((int64_t)(cbase + c) * H + h) * E;
    const float F = sF[p % 3];
    const bf16_t* kt = (const bf16_t*)(sKT + buf * kbuf);
    const bf16_t* vt = (const bf16_t*)(sVT + buf * vbuf);
    const bf16_t* bt = (const bf16_t*)(sBT + buf * vbuf);
#pragma unroll
    for (int jj = 0; jj < kStMaxBlocks; ++jj) {
      if (!sval[jj]) continue;
      const int64_t off = slot + goff[jj];
      if (HAS_J) {
        f32x4 mu, I;
#pragma unroll
        for (int r = 0; r < 4; ++r) { I[r] = accJ[jj][r] + Ip; mu[r] = accM[jj][r] * fast_rcp(I[r]); }
        *(f32x4*)((float*)A.tiles_a + off) = mu;
        *(f32x4*)(A.tiles_b + off) = I;
      } else {
        store_vec<4>((bf16_t*)A.tiles_a + off, (const float*)&accM[jj]);
      }
      f32x4 M = accM[jj] * F, J = accJ[jj] * F;
#pragma unroll
      for (int ks = 0; ks < 2; ++ks) {
        const bf16x8 BK = *(const bf16x8*)&kt[ldk[jj] + 32 * ks];
        const bf16x8 AM = *(const bf16x8*)&vt[ldv[jj] + 32 * ks];
        M = mfma16(BK, AM, M);
        if (HAS_J) {
          const bf16x8 AJ = *(const bf16x8*)&bt[ldv[jj] + 32 * ks];
          bf16x8 BKK;
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            const float kf = (float)BK[j];
            BKK[j] = (bf16_t)(kf * kf);
          }
          J = mfma16(BKK, AJ, J);
        }
      }
      accM[jj] = M;
      accJ[jj] = J;
    }
    __syncthreads();
  }
  // the feeding waves take their steps in groups of four, starting at -2
  for (int p = nchunks; ((p + 2) & 3) != 0; ++p) __syncthreads();

  if (A.fin_a) {
#pragma unroll
    for (int jj = 0; jj < kStMaxBlocks; ++jj) {
      if (!sval[jj]) continue;
      const int64_t off = (int64_t)nh * E + goff[jj];
      if (HAS_J) {
        f32x4 mu, I;
#pragma unroll
        for (int r = 0; r < 4; ++r) { I[r] = accJ[jj][r] + Ip; mu[r] = accM[jj][r] * fast_rcp(I[r]); }
        *(f32x4*)(A.fin_a + off) = mu;
        *(f32x4*)(A.fin_b + off) = I;
      } else {
        *(f32x4*)(A.fin_a + off) = accM[jj] * A.fin_scale;
      }
    }
  }
}

template <bool HAS_J, int NIK>
static int launch_state_pass_t(const StatePassArgs& A, int kern_id, unsigned grid, size_t lds, hipStream_t s) {
  if (int rc = allow_lds((const void*)&chunk_states_kernel<HAS_J, NIK>, lds)) return rc;
  PAL_TIMED_LAUNCH(kern_id, s, (chunk_states_kernel<HAS_J, NIK>), dim3(grid), dim3(768), lds, s, A);
  PAL_HIP_LAUNCH_CHECK();
  return PAL_OK;
}

template <bool HAS_J>
static int launch_state_pass_j(const StatePassArgs& A, int kern_id, unsigned grid, size_t lds, hipStream_t s) {
  switch ((A.dks + 63) / 64) {
    case 1: return launch_state_pass_t<HAS_J, 1>(A, kern_id, grid, lds, s);
    case 2: return launch_state_pass_t<HAS_J, 2>(A, kern_id, grid, lds, s);
    case 3: return launch_state_pass_t<HAS_J, 3>(A, kern_id, grid, lds, s);
    case 4: return launch_state_pass_t<HAS_J, 4>(A, kern_id, grid, lds, s);
    default: return PAL_E_HEADDIM;
  }
}

// key columns per workgroup of the one-pass form, see launch_state_pass
static int state_pass_key_slice(const ChunkArgs& a, int ds) {
  if (ds == 16 && a.dk % 128 == 0 && (int64_t)a.n_seqs * a.H * (a.dv / 16) < 192) return 64;
  return a.dk;
}

// Whether the one-pass form serves this call: bf16 rows, and enough (sequence, head, slice) workgroups that
// the serial walk over the tiles does not leave most of the GPU idle.
bool state_pass_applies(const ChunkArgs& a, int dtype, bool has_j) {
  if (dtype != PAL_DTYPE_BF16 || (a.flags & PAL_FLAG_STATES_TWO_KERNELS)) return false;
  if (a.dk < 16 || a.dk > 256 || a.dk % 16 || a.dv % 16) return false;
  // rows are addressed with 32-bit byte offsets from the first row of a sequence
  if ((int64_t)a.T * a.H * (a.dk > a.dv ? a.dk : a.dv) * 2 >= 0x7fffffffLL) return false;
  if (a.flags & PAL_FLAG_STATES_ONE_PASS) return true;
  // The walk over the tiles is serial per workgroup (0.4-0.7 us per tile): with fewer workgroups than this the
  // two-kernel form, which spreads the tiles over the whole GPU, is faster.
  return (int64_t)a.n_seqs * a.H * (a.dv / 16) * (a.dk / state_pass_key_slice(a, 16)) >= 192;
}

// tiles_a / tiles_b, init_*, fin_*: see StatePassArgs.  reverse walks every sequence from its last tile.
int launch_state_pass(const ChunkArgs& a, bool has_j, void* tiles_a, float* tiles_b, const float* init_a,
                      const float* init_b, float* fin_a, float* fin_b, bool reverse, float fin_scale, int kern_id,
                      hipStream_t s) {
  StatePassArgs A;
  A.c = a;
  A.tiles_a = tiles_a; A.tiles_b = tiles_b;
  A.init_a = init_a; A.init_b = init_b; A.fin_a = fin_a; A.fin_b = fin_b;
  A.reverse = reverse ? 1 : 0;
  A.fin_scale = fin_scale;
  // value rows per workgroup: the largest slice that still gives three quarters of the compute units a
  // workgroup (measured: wider slices stage the key rows for more state at the same cost per tile; with
  // fewer workgroups than that the idle units cost more)
  int ds = 16;
  const int cand[3] = {64, 48, 32};
  for (int c : cand) {
    if (a.dv % c || c * a.dk > 256 * 4 * kStMaxBlocks) continue;
    if ((int64_t)a.n_seqs * a.H * (a.dv / c) >= 192) { ds = c; break; }
  }
  // key columns per workgroup: all of them, unless even slices of 16 value rows leave the GPU short of workgroups and
  // the key columns can be halved into slices of 64 (measured at one sequence of 16 heads, 128x128: 128 workgroups
  // 102 us per 64 tiles, 256 workgroups of 16 x 64 entries 72 us, the two-kernel form 96 us; slices of 32 columns or
  // 32 x 32 entries are slower again, and with enough workgroups splitting the columns gains nothing)
  const int dks = state_pass_key_slice(a, ds);
  if (ds * dks > 256 * 4 * kStMaxBlocks) return PAL_E_HEADDIM;
  A.ds = ds;
  A.nsplit = a.dv / ds;
  A.dks = dks;
  A.ksplit = a.dk / dks;
  const int n_sl = A.nsplit * A.ksplit;
  const int64_t total = (int64_t)a.n_seqs * a.H * n_sl;
  if (total <= 0) return PAL_OK;
  int64_t per_xcd = (total + 7) / 8;
  per_xcd = (per_xcd + n_sl - 1) / n_sl * n_sl;
  A.by_length = (a.cu_seqlens && a.n_seqs > 1 && a.n_seqs <= 64) ? 1 : 0;
  if (A.by_length) per_xcd = (int64_t)((a.n_seqs + 7) / 8) * a.H * n_sl;   // whole sequences per XCD
  if (per_xcd * 8 > 0x7fffffff) return PAL_E_DIM;
  A.total = (int32_t)total;
  A.per_xcd = (int32_t)per_xcd;
  const size_t lds = sizeof(float) * (3 * kC + 4) + (size_t)2 * 2 * kStTS * (dks + ds * (has_j ? 2 : 1));
  if (lds > kMaxLds) return PAL_E_HEADDIM;
  const unsigned grid = (unsigned)(per_xcd * 8);
  return has_j ? launch_state_pass_j<true>(A, kern_id, grid, lds, s) : launch_state_pass_j<false>(A, kern_id, grid, lds, s);
}

}  // namespace pal

extern "C" int pal_state_pass_applies(const PalDims* d, int has_precision_state) {
  if (pal_validate_dims(d) != PAL_OK) return 0;
  pal::ChunkArgs a = {};
  a.T = d->seq_len; a.H = d->n_heads; a.dk = d->dk; a.dv = d->dv; a.n_seqs = d->n_seqs;
  a.Hq = d->n_qk_heads > 0 ? d->n_qk_heads : d->n_heads;
  a.flags = d->flags;
  return pal::state_pass_applies(a, d->dtype, has_precision_state != 0) ? 1 : 0;
}
