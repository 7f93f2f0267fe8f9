// Element-wise work of the reference layer either side of the operator, one kernel per direction:
//   prologue (palimpsa/layers/palimpsa.py:266-279): L2-normalised q, k (heads repeated), v = x * bs,
//     b = sigmoid(b_raw) * softplus(b_scale) * bs, gt = softplus(dt_raw + dt_bias);
//   epilogue (:337-343): y = rmsnorm(o + x * D) * weight * swish(gate).
// and of the reference's other caller of the operator (palimpsa/layers/meta_mamba2.py):
//   prologue (:283-299): dt = clamp(softplus(dt_raw + dt_bias)), v = x * dt, b = sigmoid(b_raw) * softplus(b_scale) * dt
//     (q = C and k = B go to the operator as they are, shared heads through its n_qk_heads);
//   epilogue (:355-363): y = rmsnorm over all heads of a token of ((o + x * D) * swish(gate)) * weight.
// All of it is bound by HBM: every row is read once and written once.  A row of d elements is handled
// by a group of GL lanes (the power of two >= d/8), eight consecutive elements per lane (16-byte
// accesses for bf16 rows); a workgroup of 256 threads owns one head and a range of tokens, so that the
// per-head sums of the backward are accumulated in a fixed order (no atomics).
#include <type_traits>

#include "pal_common.h"
#include "pal_host.h"
#include "pal_profile.h"

namespace pal {

constexpr int kGlueIter = 8;   // rows per row slot of a workgroup
// rows of a slot that are fetched before the first of them is used: a thread has one or two 16-byte fetches per row and
// tensor, and taken one row at a time each fetch waits for the stores of the row before it (the kernels ran at
// 3.3-3.7 TB/s that way).  Four rows in the forward kernels; two in the backward ones, which hold twice the tensors
// per row (with four they need 200 registers and lose more to the occupancy than they gain).
constexpr int kGlueBatch = 4;
constexpr int kGlueBatchBwd = 2;

template <typename T>
__device__ __forceinline__ void load8(const T* p, float* x) {
  load_vec<4>(p, x);
  load_vec<4>(p + 4, x + 4);
}
template <typename T>
__device__ __forceinline__ void store8(T* p, const float* x) {
  store_vec<4>(p, x);
  store_vec<4>(p + 4, x + 4);
}
// eight fp32 elements as two 16-byte accesses (rows are 16-byte aligned)
struct F32x8 {
  f32x4 lo, hi;
  __device__ __forceinline__ float operator[](int e) const { return e < 4 ? lo[e & 3] : hi[e & 3]; }
};
template <int CTRL>
__device__ __forceinline__ float dpp_move(float x) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xf, 0xf, false));
}
// sum over the GL lanes of a row group (GL a power of two <= 32, the same for the whole wave, groups
// aligned to multiples of GL); every lane of the group gets it.  Lane exchanges inside a row of 16
// lanes are data-parallel moves: neighbours in a quad, quads, then the mirrored half rows and rows
// (by then every lane of the smaller group holds the same partial sum, so a mirror pairs as an xor does).
__device__ __forceinline__ float group_sum(float x, int GL) {
  if (GL > 1) x += dpp_move<0xB1>(x);    // quad_perm [1,0,3,2]
  if (GL > 2) x += dpp_move<0x4E>(x);    // quad_perm [2,3,0,1]
  if (GL > 4) x += dpp_move<0x141>(x);   // row_half_mirror
  if (GL > 8) x += dpp_move<0x140>(x);   // row_mirror
  if (GL > 16) {
    float a = x, b = x;
    swap_rows(a, b);
    x = a + b;
  }
  return x;
}
// reciprocal to 1 ulp (one instruction; an IEEE division is ten)
__device__ __forceinline__ float rcpf_(float x) { return __builtin_amdgcn_rcpf(x); }
__device__ __forceinline__ float sigmoidf_(float x) { return rcpf_(1.f + __expf(-x)); }
// softplus as torch computes it (threshold 20)
__device__ __forceinline__ float softplusf_(float x) { return x > 20.f ? x : log1pf(__expf(x)); }
template <typename T>
__device__ __forceinline__ float round_to(float x) { return to_f32(from_f32<T>(x)); }

struct GlueGeom {
  int GLk, GLv;     // lanes per q/k row and per v row
  int tok_per_block;
};
static GlueGeom glue_geom(const PalGlueDims* d) {
  auto pow2 = [](int n) { int p = 1; while (p < n) p <<= 1; return p; };
  GlueGeom g;
  g.GLk = pow2(d->dk / 8);
  g.GLv = pow2(d->dv / 8);
  const int GLmax = g.GLk > g.GLv ? g.GLk : g.GLv;
  g.tok_per_block = (256 / GLmax) * kGlueIter;
  return g;
}

// ------------------------------------------------------------------ prologue
struct PrologueArgs {
  PalPrologueTensors t;
  PalPrologueGrads g;
  float* part;          // backward: [H][n_token_blocks][2] partial sums (ddt_bias, db_scale)
  int tokens, H, Hqk, dk, dv, GLk, GLv, tok_per_block;
  float eps;
  int mamba;            // the multiplier of x and b is gt itself, clamped to [dt_min, dt_max] (no bs_raw)
  int task0;            // first task of the grid's z axis (2 when there are no q, k rows)
  float dt_min, dt_max;
};

// grid (token blocks, heads, 3): z = 0 rows of q, z = 1 rows of k (heads of q_raw / k_raw), z = 2 rows of v, b and gt
template <typename T>
__global__ __launch_bounds__(256) void prologue_fwd_kernel(PrologueArgs A) {
  const int tid = threadIdx.x, task = blockIdx.z + A.task0, h = blockIdx.y;
  const int tok0 = blockIdx.x * A.tok_per_block;
  const int tok1 = min(A.tokens, tok0 + A.tok_per_block);
  if (task < 2) {
    if (h >= A.Hqk) return;
    const int GL = A.GLk, d = A.dk, rep = A.H / A.Hqk;
    const int slot = tid / GL, l = tid % GL, rows = 256 / GL;
    const T* src = (const T*)(task ? A.t.k_raw : A.t.q_raw);
    T* dst = (T*)(task ? A.t.k : A.t.q);
    const bool on = 8 * l < d;
    for (int tb = tok0 + slot; tb < tok1; tb += kGlueBatch * rows) {
      float xb[kGlueBatch][8];
#pragma unroll
      for (int u = 0; u < kGlueBatch; ++u) {
        const int tok = tb + u * rows;
#pragma unroll
        for (int e = 0; e < 8; ++e) xb[u][e] = 0.f;
        if (on && tok < tok1) load8(src + ((int64_t)tok * A.Hqk + h) * d + 8 * l, xb[u]);
      }
#pragma unroll
      for (int u = 0; u < kGlueBatch; ++u) {
        const int tok = tb + u * rows;
        float* x = xb[u];
        float ss = 0.f;
#pragma unroll
        for (int e = 0; e < 8; ++e) ss = fmaf(x[e], x[e], ss);
        ss = group_sum(ss, GL);
        const float inv = rcpf_(fmaxf(__builtin_amdgcn_sqrtf(ss), A.eps));
#pragma unroll
        for (int e = 0; e < 8; ++e) x[e] *= inv;
        if (on && tok < tok1)
          for (int r = 0; r < rep; ++r) store8(dst + ((int64_t)tok * A.H + h * rep + r) * d + 8 * l, x);
      }
    }
  } else {
    const int GL = A.GLv, d = A.dv;
    const int slot = tid / GL, l = tid % GL, rows = 256 / GL;
    const bool on = 8 * l < d;
    const float sp = A.t.b_raw ? softplusf_(A.t.b_scale[h]) : 0.f;
    const float bias = A.t.dt_bias[h];
    const bool has_b = A.t.b_raw != nullptr;
    for (int tb = tok0 + slot; tb < tok1; tb += kGlueBatch * rows) {
      float xb[kGlueBatch][8], bb[kGlueBatch][8], dtr[kGlueBatch], bsr[kGlueBatch];
#pragma unroll
      for (int u = 0; u < kGlueBatch; ++u) {
        const int tok = tb + u * rows;
        dtr[u] = bsr[u] = 0.f;
        if (tok < tok1) {
          const int64_t th = (int64_t)tok * A.H + h;
          dtr[u] = to_f32(((const T*)A.t.dt_raw)[th]);
          if (!A.mamba) bsr[u] = to_f32(((const T*)A.t.bs_raw)[th]);
          if (on) {
            load8((const T*)A.t.x + th * d + 8 * l, xb[u]);
            if (has_b) load8((const T*)A.t.b_raw + th * d + 8 * l, bb[u]);
          }
        }
      }
#pragma unroll
      for (int u = 0; u < kGlueBatch; ++u) {
        const int tok = tb + u * rows;
        if (tok >= tok1) break;
        const int64_t th = (int64_t)tok * A.H + h;
        float gtv = softplusf_(dtr[u] + bias), bs;
        if (A.mamba) {
          gtv = fminf(fmaxf(gtv, A.dt_min), A.dt_max);
          bs = gtv;
        } else {
          bs = round_to<T>(sigmoidf_(bsr[u]));
        }
        if (l == 0) A.t.gt[th] = gtv;
        if (!on) continue;
        float* x = xb[u];
#pragma unroll
        for (int e = 0; e < 8; ++e) x[e] *= bs;
        store8((T*)A.t.v + th * d + 8 * l, x);
        if (has_b) {
          float* br = bb[u];
#pragma unroll
          for (int e = 0; e < 8; ++e) br[e] = sigmoidf_(br[e]) * sp * bs;
          store8((T*)A.t.b + th * d + 8 * l, br);
        }
      }
    }
  }
}

template <typename T>
__global__ __launch_bounds__(256) void prologue_bwd_kernel(PrologueArgs A) {
  __shared__ float sRed[4][2];
  const int tid = threadIdx.x, task = blockIdx.z + A.task0, h = blockIdx.y;
  const int tok0 = blockIdx.x * A.tok_per_block;
  const int tok1 = min(A.tokens, tok0 + A.tok_per_block);
  if (task < 2) {
    if (h >= A.Hqk) return;
    // y = x / n, n = max(|x|, eps):  dx = (s - y (y . s)) / n with s the sum of the gradients of the repeated heads
    // (for |x| < eps the norm is the constant eps and dx = s / eps)
    const int GL = A.GLk, d = A.dk, rep = A.H / A.Hqk;
    const int slot = tid / GL, l = tid % GL, rows = 256 / GL;
    const T* src = (const T*)(task ? A.t.k_raw : A.t.q_raw);
    const T* gsrc = (const T*)(task ? A.g.dk : A.g.dq);
    T* dst = (T*)(task ? A.g.dk_raw : A.g.dq_raw);
    const bool on = 8 * l < d;
    for (int tb = tok0 + slot; tb < tok1; tb += kGlueBatchBwd * rows) {
      float xb[kGlueBatchBwd][8], sb[kGlueBatchBwd][8];
#pragma unroll
      for (int u = 0; u < kGlueBatchBwd; ++u) {
        const int tok = tb + u * rows;
#pragma unroll
        for (int e = 0; e < 8; ++e) xb[u][e] = sb[u][e] = 0.f;
        if (on && tok < tok1) {
          load8(src + ((int64_t)tok * A.Hqk + h) * d + 8 * l, xb[u]);
          for (int r = 0; r < rep; ++r) {
            float gy[8];
            load8(gsrc + ((int64_t)tok * A.H + h * rep + r) * d + 8 * l, gy);
#pragma unroll
            for (int e = 0; e < 8; ++e) sb[u][e] += gy[e];
          }
        }
      }
#pragma unroll
      for (int u = 0; u < kGlueBatchBwd; ++u) {
        const int tok = tb + u * rows;
        const float *x = xb[u], *s = sb[u];
        float ss = 0.f, xs = 0.f;
#pragma unroll
        for (int e = 0; e < 8; ++e) { ss = fmaf(x[e], x[e], ss); xs = fmaf(x[e], s[e], xs); }
        ss = group_sum(ss, GL);
        xs = group_sum(xs, GL);
        const float nrm = __builtin_amdgcn_sqrtf(ss);
        const bool clamped = nrm < A.eps;
        const float inv = rcpf_(fmaxf(nrm, A.eps));
        const float c = clamped ? 0.f : xs * inv * inv * inv;   // dx = s/n - x (x.s)/n^3
        float out[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) out[e] = s[e] * inv - x[e] * c;
        if (on && tok < tok1) store8(dst + ((int64_t)tok * A.Hqk + h) * d + 8 * l, out);
      }
    }
  } else {
    const int GL = A.GLv, d = A.dv;
    const int slot = tid / GL, l = tid % GL, rows = 256 / GL;
    const bool on = 8 * l < d;
    const bool has_b = A.t.b_raw != nullptr;
    const float sp = has_b ? softplusf_(A.t.b_scale[h]) : 0.f;
    const float bias = A.t.dt_bias[h];
    float acc_dt = 0.f, acc_bs = 0.f;   // this thread's share of ddt_bias[h] and of sum db * sigmoid(b_raw) * bs
    for (int tb = tok0 + slot; tb < tok1; tb += kGlueBatchBwd * rows) {
      float xb[kGlueBatchBwd][8], gvb[kGlueBatchBwd][8], brb[kGlueBatchBwd][8], gbb[kGlueBatchBwd][8];
      float dtr[kGlueBatchBwd], bsr[kGlueBatchBwd], dgr[kGlueBatchBwd];
#pragma unroll
      for (int u = 0; u < kGlueBatchBwd; ++u) {
        const int tok = tb + u * rows;
        dtr[u] = bsr[u] = dgr[u] = 0.f;
        if (tok < tok1) {
          const int64_t th = (int64_t)tok * A.H + h;
          dtr[u] = to_f32(((const T*)A.t.dt_raw)[th]);
          if (!A.mamba) bsr[u] = to_f32(((const T*)A.t.bs_raw)[th]);
          if (l == 0) dgr[u] = A.g.dgt[th];
          if (on) {
            load8((const T*)A.t.x + th * d + 8 * l, xb[u]);
            load8((const T*)A.g.dv + th * d + 8 * l, gvb[u]);
            if (has_b) {
              load8((const T*)A.t.b_raw + th * d + 8 * l, brb[u]);
              load8((const T*)A.g.db + th * d + 8 * l, gbb[u]);
            }
          }
        }
      }
#pragma unroll
      for (int u = 0; u < kGlueBatchBwd; ++u) {
        const int tok = tb + u * rows;
        if (tok >= tok1) break;   // the lanes of a row leave together
        const int64_t th = (int64_t)tok * A.H + h;
        const float pre = dtr[u] + bias;
        float sg = 0.f, bs;
        bool pass = true;     // mamba: the clamp lets the gradient through (bounds included, as torch.clamp)
        if (A.mamba) {
          const float spd = softplusf_(pre);
          pass = spd >= A.dt_min && spd <= A.dt_max;
          bs = fminf(fmaxf(spd, A.dt_min), A.dt_max);
        } else {
          sg = sigmoidf_(bsr[u]);
          bs = round_to<T>(sg);
        }
        float dbs = 0.f, dsp = 0.f;
        if (on) {
          const float *x = xb[u], *gv = gvb[u];
          float dx[8];
#pragma unroll
          for (int e = 0; e < 8; ++e) { dx[e] = gv[e] * bs; dbs = fmaf(gv[e], x[e], dbs); }
          store8((T*)A.g.dx + th * d + 8 * l, dx);
          if (has_b) {
            const float *br = brb[u], *gb = gbb[u];
            float out[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) {
              const float s = sigmoidf_(br[e]);
              out[e] = gb[e] * sp * bs * s * (1.f - s);
              dsp = fmaf(gb[e], s, dsp);
            }
            store8((T*)A.g.db_raw + th * d + 8 * l, out);
          }
        }
        dbs = group_sum(fmaf(dsp, sp, dbs), GL);   // d/d bs of v = x bs and b = s sp bs
        if (l == 0) {
          float ddt;
          if (A.mamba) {
            // gt is an output and the multiplier of x and b
            ddt = pass ? (dgr[u] + dbs) * sigmoidf_(pre) : 0.f;
          } else {
            ((T*)A.g.dbs_raw)[th] = from_f32<T>(dbs * sg * (1.f - sg));
            ddt = dgr[u] * sigmoidf_(pre);
          }
          ((T*)A.g.ddt_raw)[th] = from_f32<T>(ddt);
          acc_dt += ddt;
        }
        acc_bs = fmaf(dsp, bs, acc_bs);
      }
    }
    // workgroup totals in a fixed order: lanes, then waves
    acc_dt = wave_sum(acc_dt);
    acc_bs = wave_sum(acc_bs);
    if ((tid & 63) == 0) { sRed[tid >> 6][0] = acc_dt; sRed[tid >> 6][1] = acc_bs; }
    __syncthreads();
    if (tid == 0) {
      float* p = A.part + ((int64_t)h * gridDim.x + blockIdx.x) * 2;
      p[0] = sRed[0][0] + sRed[1][0] + sRed[2][0] + sRed[3][0];
      p[1] = sRed[0][1] + sRed[1][1] + sRed[2][1] + sRed[3][1];
    }
  }
}

// ddt_bias[h], db_scale[h] from the per-workgroup partial sums; db_scale picks up softplus'(b_scale) = sigmoid(b_scale)
__global__ void prologue_bwd_reduce_kernel(PrologueArgs A, int n_blocks) {
  const int h = blockIdx.x, lane = threadIdx.x;
  float a = 0.f, b = 0.f;
  for (int j = lane; j < n_blocks; j += 64) {
    a += A.part[((int64_t)h * n_blocks + j) * 2];
    b += A.part[((int64_t)h * n_blocks + j) * 2 + 1];
  }
  a = wave_sum(a);
  b = wave_sum(b);
  if (lane == 0) {
    A.g.ddt_bias[h] = a;
    if (A.g.db_scale) A.g.db_scale[h] = A.t.b_raw ? b * sigmoidf_(A.t.b_scale[h]) : 0.f;
  }
}

// ------------------------------------------------------------------ epilogue
struct EpilogueArgs {
  PalEpilogueTensors t;
  PalEpilogueGrads g;
  float* part_w;        // backward: [H][n_token_blocks][dv] partial sums of dweight
  float* part_D;        // backward: [H][n_token_blocks]
  int tokens, H, dv, GL, tok_per_block;
  float eps;
};

template <typename T>
__global__ __launch_bounds__(256) void epilogue_fwd_kernel(EpilogueArgs A) {
  const int tid = threadIdx.x, h = blockIdx.y;
  const int tok0 = blockIdx.x * A.tok_per_block;
  const int tok1 = min(A.tokens, tok0 + A.tok_per_block);
  const int GL = A.GL, d = A.dv;
  const int slot = tid / GL, l = tid % GL, rows = 256 / GL;
  const bool on = 8 * l < d;
  const float Dh = A.t.x ? A.t.D[h] : 0.f;
  float w[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  if (on) load8(A.t.weight + 8 * l, w);
  const float inv_d = 1.f / (float)d;
  const bool has_x = A.t.x != nullptr, has_gate = A.t.gate != nullptr;
  for (int tb = tok0 + slot; tb < tok1; tb += kGlueBatch * rows) {
    float rb[kGlueBatch][8], xb[kGlueBatch][8], gb[kGlueBatch][8];
#pragma unroll
    for (int u = 0; u < kGlueBatch; ++u) {
      const int tok = tb + u * rows;
      const int64_t th = (int64_t)tok * A.H + h;
#pragma unroll
      for (int e = 0; e < 8; ++e) rb[u][e] = xb[u][e] = gb[u][e] = 0.f;
      if (on && tok < tok1) {
        load8((const T*)A.t.o + th * d + 8 * l, rb[u]);
        if (has_x) load8((const T*)A.t.x + th * d + 8 * l, xb[u]);
        if (has_gate) load8((const T*)A.t.gate + th * d + 8 * l, gb[u]);
      }
    }
#pragma unroll
    for (int u = 0; u < kGlueBatch; ++u) {
      const int tok = tb + u * rows;
      if (tok >= tok1) break;   // the lanes of a row leave together
      const int64_t th = (int64_t)tok * A.H + h;
      float* r = rb[u];
#pragma unroll
      for (int e = 0; e < 8; ++e) r[e] = fmaf(xb[u][e], Dh, r[e]);
      float ss = 0.f;
#pragma unroll
      for (int e = 0; e < 8; ++e) ss = fmaf(r[e], r[e], ss);
      ss = group_sum(ss, GL);
      const float rstd = rsqrtf(ss * inv_d + A.eps);
      if (l == 0) A.t.rstd[th] = rstd;
      if (!on) continue;
      float y[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) y[e] = r[e] * rstd * w[e];
      if (has_gate) {
#pragma unroll
        for (int e = 0; e < 8; ++e) y[e] *= gb[u][e] * sigmoidf_(gb[u][e]);
      }
      store8((T*)A.t.y + th * d + 8 * l, y);
    }
  }
}

template <typename T>
__global__ __launch_bounds__(256) void epilogue_bwd_kernel(EpilogueArgs A) {
  extern __shared__ float sW[];   // [rows][dv padded to 8 GL] dweight shares of the row slots
  __shared__ float sRed[4];
  const int tid = threadIdx.x, h = blockIdx.y;
  const int tok0 = blockIdx.x * A.tok_per_block;
  const int tok1 = min(A.tokens, tok0 + A.tok_per_block);
  const int GL = A.GL, d = A.dv;
  const int slot = tid / GL, l = tid % GL, rows = 256 / GL;
  const bool on = 8 * l < d;
  const float Dh = A.t.x ? A.t.D[h] : 0.f;
  float w[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  if (on) load8(A.t.weight + 8 * l, w);
  const float inv_d = 1.f / (float)d;
  float dw[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  float accD = 0.f;
  const bool has_x = A.t.x != nullptr, has_gate = A.t.gate != nullptr;
  for (int tb = tok0 + slot; tb < tok1; tb += kGlueBatchBwd * rows) {
    float rb[kGlueBatchBwd][8], xb[kGlueBatchBwd][8], gyb[kGlueBatchBwd][8], gtb[kGlueBatchBwd][8], rsb[kGlueBatchBwd];
#pragma unroll
    for (int u = 0; u < kGlueBatchBwd; ++u) {
      const int tok = tb + u * rows;
      const int64_t th = (int64_t)tok * A.H + h;
#pragma unroll
      for (int e = 0; e < 8; ++e) rb[u][e] = xb[u][e] = gyb[u][e] = gtb[u][e] = 0.f;
      rsb[u] = 0.f;
      if (tok < tok1) {
        rsb[u] = A.t.rstd[th];
        if (on) {
          load8((const T*)A.t.o + th * d + 8 * l, rb[u]);
          load8((const T*)A.g.dy + th * d + 8 * l, gyb[u]);
          if (has_x) load8((const T*)A.t.x + th * d + 8 * l, xb[u]);
          if (has_gate) load8((const T*)A.t.gate + th * d + 8 * l, gtb[u]);
        }
      }
    }
#pragma unroll
    for (int u = 0; u < kGlueBatchBwd; ++u) {
      const int tok = tb + u * rows;
      if (tok >= tok1) break;   // the lanes of a row leave together
      const int64_t th = (int64_t)tok * A.H + h;
      float* r = rb[u];
      const float *x = xb[u], *gy = gyb[u];
      float sw[8], dsw[8];   // swish(gate) and its derivative
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        r[e] = fmaf(x[e], Dh, r[e]);
        sw[e] = 1.f;
        dsw[e] = 0.f;
        if (has_gate) {
          const float z = gtb[u][e], s = sigmoidf_(z);
          sw[e] = z * s;
          dsw[e] = s * (1.f + z * (1.f - s));
        }
      }
      const float rstd = rsb[u];
      // n = r rstd;  y = n w sw;  dn = dy w sw;  dr = rstd (dn - n mean(dn n))
      float n[8], dn[8], dot = 0.f;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        n[e] = r[e] * rstd;
        dn[e] = gy[e] * w[e] * sw[e];
        dot = fmaf(dn[e], n[e], dot);
        dw[e] = fmaf(gy[e] * n[e], sw[e], dw[e]);
      }
      dot = group_sum(dot, GL) * inv_d;
      if (!on) continue;
      float dr[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) dr[e] = rstd * (dn[e] - n[e] * dot);
      store8((T*)A.g.d_o + th * d + 8 * l, dr);
      if (has_x) {
        float dx[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) { dx[e] = dr[e] * Dh; accD = fmaf(dr[e], x[e], accD); }
        store8((T*)A.g.dx + th * d + 8 * l, dx);
      }
      if (has_gate) {
        float dg[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) dg[e] = gy[e] * n[e] * w[e] * dsw[e];
        store8((T*)A.g.dgate + th * d + 8 * l, dg);
      }
    }
  }
  // dweight: the row slots' shares are added in slot order
  const int dpad = 8 * GL;
#pragma unroll
  for (int e = 0; e < 8; ++e) sW[slot * dpad + 8 * l + e] = dw[e];
  accD = wave_sum(accD);
  if ((tid & 63) == 0) sRed[tid >> 6] = accD;
  __syncthreads();
  const int64_t blk = (int64_t)h * gridDim.x + blockIdx.x;
  for (int c = tid; c < d; c += 256) {
    float s = 0.f;
    for (int r = 0; r < rows; ++r) s += sW[r * dpad + c];
    A.part_w[blk * d + c] = s;
  }
  if (tid == 0 && A.t.x) A.part_D[blk] = sRed[0] + sRed[1] + sRed[2] + sRed[3];
}

// dweight[c] = sum over heads and token blocks; dD[h] = sum over token blocks (fixed order)
__global__ void epilogue_bwd_reduce_kernel(EpilogueArgs A, int n_blocks) {
  const int lane = threadIdx.x;
  if ((int)blockIdx.x < A.dv) {
    const int c = blockIdx.x;
    float s = 0.f;
    for (int64_t j = lane; j < (int64_t)A.H * n_blocks; j += 64) s += A.part_w[j * A.dv + c];
    s = wave_sum(s);
    if (lane == 0) A.g.dweight[c] = s;
  } else if (A.t.x) {
    const int h = blockIdx.x - A.dv;
    float s = 0.f;
    for (int j = lane; j < n_blocks; j += 64) s += A.part_D[(int64_t)h * n_blocks + j];
    s = wave_sum(s);
    if (lane == 0) A.g.dD[h] = s;
  }
}

// ------------------------------------------------------------------ epilogue over all heads of a token
// y = rmsnorm_{H dv}((o + x D) swish(gate)) weight  (palimpsa/layers/meta_mamba2.py:355-363: the gate is applied before
// a norm that runs over the whole token).  One wave per token, 512 elements per pass (eight per lane, inside one head
// since dv is a multiple of 8); a wave takes kHeadsIter tokens in turn and the four waves of a workgroup add their sums
// over tokens (dweight, dD of the backward) in LDS, so that a workgroup leaves one partial row per 16 tokens.
constexpr int kHeadsIter = 4;      // tokens per wave (a workgroup of four waves takes 16)
constexpr int kHeadsMaxCh = 8;     // passes of 512 elements: H dv <= 4096

template <typename T>
__global__ __launch_bounds__(256) void epilogue_heads_fwd_kernel(EpilogueArgs A) {
  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  const int dv = A.dv, HD = A.H * dv, nch = (HD + 511) >> 9;
  const float inv_n = 1.f / (float)HD;
  for (int it = 0; it < kHeadsIter; ++it) {
    const int tok = ((int)blockIdx.x * 4 + w) * kHeadsIter + it;
    if (tok >= A.tokens) break;
    const int64_t row = (int64_t)tok * HD;
    float r[kHeadsMaxCh][8];
    float ss = 0.f;
#pragma unroll
    for (int c = 0; c < kHeadsMaxCh; ++c) {
      const int e0 = 512 * c + 8 * lane;
#pragma unroll
      for (int e = 0; e < 8; ++e) r[c][e] = 0.f;
      if (c < nch && e0 < HD) {
        load8((const T*)A.t.o + row + e0, r[c]);
        if (A.t.x) {
          float x[8];
          load8((const T*)A.t.x + row + e0, x);
          const float Dh = A.t.D[e0 / dv];
#pragma unroll
          for (int e = 0; e < 8; ++e) r[c][e] = fmaf(x[e], Dh, r[c][e]);
        }
        if (A.t.gate) {
          float z[8];
          load8((const T*)A.t.gate + row + e0, z);
#pragma unroll
          for (int e = 0; e < 8; ++e) r[c][e] *= z[e] * sigmoidf_(z[e]);
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) ss = fmaf(r[c][e], r[c][e], ss);
      }
    }
    ss = wave_sum(ss);
    const float rstd = rsqrtf(ss * inv_n + A.eps);
    if (lane == 0) A.t.rstd[tok] = rstd;
#pragma unroll
    for (int c = 0; c < kHeadsMaxCh; ++c) {
      const int e0 = 512 * c + 8 * lane;
      if (c < nch && e0 < HD) {
        float wv[8], y[8];
        load8(A.t.weight + e0, wv);
#pragma unroll
        for (int e = 0; e < 8; ++e) y[e] = r[c][e] * rstd * wv[e];
        store8((T*)A.t.y + row + e0, y);
      }
    }
  }
}

// r = u s, u = o + x D, s = swish(gate);  n = r rstd;  y = n w;  g = dy w;  dr = rstd (g - n mean(g n));
// du = dr s (= d_o), dx = du D, dgate = dr u s', dD[h] += du . x, dweight += dy n.
// Two passes over the token's rows: the mean first, then the gradients.  NCH = passes of 512 elements, a template
// parameter: bf16 rows of up to 2048 elements stay in registers as loaded between the passes, longer or fp32 rows are
// fetched again (they come from the cache).  The sums over tokens (dweight, dD) are kept in the wave's own part of
// the LDS, not in registers: with 8 accumulators per pass in registers the kernel ran at two waves per SIMD and
// 2.8 TB/s.
// part_w: [workgroups][H dv] partial dweight, part_D: [workgroups][H dv / 8] partial dD (one slot per eight elements).
template <typename T, int NCH /* 0: any number of passes, rows fetched twice */>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(NCH <= 1 ? 4 : (NCH == 4 ? 2 : 3))))
void epilogue_heads_bwd_kernel(EpilogueArgs A) {
  extern __shared__ float sPartial[];   // [4 waves][H dv + H dv / 8]
  constexpr bool KEEP = NCH > 0;
  static_assert(!KEEP || (sizeof(T) == 2 && NCH <= 4), "rows kept in registers: bf16, at most 2048 elements");
  const int nch = KEEP ? NCH : (A.H * A.dv + 511) >> 9;
  using Raw = typename std::conditional<sizeof(T) == 2, bf16x8, F32x8>::type;
  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  const int dv = A.dv, HD = A.H * dv;
  const float inv_n = 1.f / (float)HD;
  const int64_t wave_id = (int64_t)blockIdx.x * 4 + w;
  const bool has_x = A.t.x != nullptr, has_gate = A.t.gate != nullptr;
  const int per_wave = HD + (HD >> 3);
  float* mine = sPartial + w * per_wave;   // this wave's sums: touched by no other wave before the barrier below
  for (int e = lane; e < per_wave; e += 64) mine[e] = 0.f;
  struct Rows { Raw o, x, z, gy; };
  auto fetch = [&](int64_t off, Rows& R) {
    R.o = *(const Raw*)((const T*)A.t.o + off);
    R.gy = *(const Raw*)((const T*)A.g.dy + off);
    if (has_x) R.x = *(const Raw*)((const T*)A.t.x + off);
    if (has_gate) R.z = *(const Raw*)((const T*)A.t.gate + off);
  };
  for (int it = 0; it < kHeadsIter; ++it) {
    const int tok = (int)wave_id * kHeadsIter + it;
    if (tok >= A.tokens) break;
    const int64_t row = (int64_t)tok * HD;
    const float rstd = A.t.rstd[tok];
    Rows keep[KEEP ? NCH : 1];
    float dot = 0.f;
    if constexpr (KEEP) {   // every fetch of the token in flight before the first use
#pragma unroll
      for (int c = 0; c < NCH; ++c) {
        const int e0 = 512 * c + 8 * lane;
        if (e0 < HD) fetch(row + e0, keep[c]);
      }
    }
    auto pass1 = [&](int c) {
      const int e0 = 512 * c + 8 * lane;
      if (e0 < HD) {
        Rows tmp;
        if constexpr (!KEEP) fetch(row + e0, tmp);
        const Rows& R = KEEP ? keep[c] : tmp;
        const float Dh = has_x ? A.t.D[e0 / dv] : 0.f;
        float wv[8];
        load8(A.t.weight + e0, wv);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          float r = (float)R.o[e];
          if (has_x) r = fmaf((float)R.x[e], Dh, r);
          if (has_gate) {
            const float z = (float)R.z[e];
            r *= z * sigmoidf_(z);
          }
          dot = fmaf((float)R.gy[e] * wv[e], r, dot);
        }
      }
      __builtin_amdgcn_sched_barrier(0);   // one pass of 512 elements at a time: the registers of a pass are reused
    };
    if constexpr (KEEP) {
#pragma unroll
      for (int c = 0; c < NCH; ++c) pass1(c);
    } else {
#pragma unroll 1
      for (int c = 0; c < nch; ++c) pass1(c);
    }
    dot = wave_sum(dot) * (rstd * inv_n);
    auto pass2 = [&](int c) {
      const int e0 = 512 * c + 8 * lane;
      if (e0 < HD) {
        Rows tmp;
        if constexpr (!KEEP) fetch(row + e0, tmp);
        const Rows& R = KEEP ? keep[c] : tmp;
        const float Dh = has_x ? A.t.D[e0 / dv] : 0.f;
        float wv[8], du[8], dz[8], dx[8], gn[8];
        load8(A.t.weight + e0, wv);
        float aD = 0.f;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float x = has_x ? (float)R.x[e] : 0.f, gy = (float)R.gy[e];
          const float u = fmaf(x, Dh, (float)R.o[e]);
          float sw = 1.f, dsw = 0.f;
          if (has_gate) {
            const float z = (float)R.z[e], sg = sigmoidf_(z);
            sw = z * sg;
            dsw = sg * (1.f + z * (1.f - sg));
          }
          const float n = u * sw * rstd;
          const float dr = rstd * (gy * wv[e] - n * dot);
          du[e] = dr * sw;
          dz[e] = dr * u * dsw;
          dx[e] = du[e] * Dh;
          aD = fmaf(du[e], x, aD);
          gn[e] = gy * n;
        }
        store8((T*)A.g.d_o + row + e0, du);
        if (has_x) store8((T*)A.g.dx + row + e0, dx);
        if (has_gate) store8((T*)A.g.dgate + row + e0, dz);
        f32x4 s0 = *(const f32x4*)(mine + e0), s1 = *(const f32x4*)(mine + e0 + 4);
        s0 += f32x4{gn[0], gn[1], gn[2], gn[3]};
        s1 += f32x4{gn[4], gn[5], gn[6], gn[7]};
        *(f32x4*)(mine + e0) = s0;
        *(f32x4*)(mine + e0 + 4) = s1;
        mine[HD + (e0 >> 3)] += aD;
      }
      __builtin_amdgcn_sched_barrier(0);
    };
    if constexpr (KEEP) {
#pragma unroll
      for (int c = 0; c < NCH; ++c) pass2(c);
    } else {
#pragma unroll 1
      for (int c = 0; c < nch; ++c) pass2(c);
    }
  }
  __syncthreads();
  // the four waves' rows in wave order (a wave without tokens holds zeros)
  for (int e = tid; e < per_wave; e += 256) {
    const float tot = (sPartial[e] + sPartial[per_wave + e]) + (sPartial[2 * per_wave + e] + sPartial[3 * per_wave + e]);
    if (e < HD) A.part_w[(int64_t)blockIdx.x * HD + e] = tot;
    else A.part_D[(int64_t)blockIdx.x * (HD >> 3) + (e - HD)] = tot;
  }
}

template <typename T, int NCH>
static int launch_heads_bwd(const EpilogueArgs& A, int nblk, size_t lds, hipStream_t hs) {
  if (int rc = allow_lds((const void*)&epilogue_heads_bwd_kernel<T, NCH>, lds)) return rc;
  PAL_TIMED_LAUNCH(kKernEpilogueBwd, hs, (epilogue_heads_bwd_kernel<T, NCH>), dim3(nblk), dim3(256), lds, hs, A);
  return PAL_OK;
}
template <typename T>
static int launch_heads_bwd_nch(int nch, const EpilogueArgs& A, int nblk, size_t lds, hipStream_t hs) {
  switch (nch) {
    case 1: return launch_heads_bwd<T, 1>(A, nblk, lds, hs);
    case 2: return launch_heads_bwd<T, 2>(A, nblk, lds, hs);
    case 3: return launch_heads_bwd<T, 3>(A, nblk, lds, hs);
    case 4: return launch_heads_bwd<T, 4>(A, nblk, lds, hs);
    default: return launch_heads_bwd<T, 0>(A, nblk, lds, hs);
  }
}

// dweight[e] (blocks 0 .. H dv / 64 - 1: 64 columns per block) and dD[h] (one block per head) from the partial rows of
// the backward kernel.  16 waves per block: wave w adds the rows j = w (mod 16) in order, four loads in flight, and
// the waves' sums are added in order, so the result does not depend on timing (one wave per block walked the rows
// alone before: 0.24 ms at 1024 partial rows).
constexpr int kRedWaves = 16;
__global__ __launch_bounds__(64 * kRedWaves) void epilogue_heads_reduce_kernel(EpilogueArgs A, int n_waves /* partial rows */) {
  __shared__ float sPart[kRedWaves][64];
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int dv = A.dv, HD = A.H * dv, n_wblocks = (HD + 63) / 64;
  float s = 0.f;
  if ((int)blockIdx.x < n_wblocks) {
    const int e = blockIdx.x * 64 + lane;
    if (e < HD) {
      float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
      int j = w;
      for (; j + 3 * kRedWaves < n_waves; j += 4 * kRedWaves) {
        s0 += A.part_w[(int64_t)j * HD + e];
        s1 += A.part_w[(int64_t)(j + kRedWaves) * HD + e];
        s2 += A.part_w[(int64_t)(j + 2 * kRedWaves) * HD + e];
        s3 += A.part_w[(int64_t)(j + 3 * kRedWaves) * HD + e];
      }
      for (; j < n_waves; j += kRedWaves) s0 += A.part_w[(int64_t)j * HD + e];
      s = (s0 + s1) + (s2 + s3);
    }
    sPart[w][lane] = s;
    __syncthreads();
    if (w == 0 && e < HD) {
      float t = 0.f;
#pragma unroll
      for (int x = 0; x < kRedWaves; ++x) t += sPart[x][lane];
      A.g.dweight[e] = t;
    }
  } else if (A.t.x) {
    const int h = blockIdx.x - n_wblocks, per = dv >> 3;
    for (int64_t j = threadIdx.x; j < (int64_t)n_waves * per; j += 64 * kRedWaves) {
      const int64_t wv = j / per, slot = j - wv * per;
      s += A.part_D[wv * (HD >> 3) + (int64_t)h * per + slot];
    }
    s = wave_sum(s);
    if (lane == 0) sPart[w][0] = s;
    __syncthreads();
    if (threadIdx.x == 0) {
      float t = 0.f;
#pragma unroll
      for (int x = 0; x < kRedWaves; ++x) t += sPart[x][0];
      A.g.dD[h] = t;
    }
  }
}

static int heads_waves(const PalGlueDims* d) { return (d->tokens + kHeadsIter - 1) / kHeadsIter; }

static int check_glue_dims(const PalGlueDims* d) {
  if (!d) return PAL_E_NULL;
  if (d->tokens <= 0 || d->n_heads <= 0 || d->n_qk_heads <= 0 || d->n_heads % d->n_qk_heads != 0) return PAL_E_DIM;
  if (d->n_heads > 65535) return PAL_E_DIM;
  if (d->dk < 8 || d->dk > 256 || d->dk % 8 || d->dv < 8 || d->dv > 256 || d->dv % 8) return PAL_E_HEADDIM;
  if (d->dtype != PAL_DTYPE_BF16 && d->dtype != PAL_DTYPE_F32) return PAL_E_DTYPE;
  if (!(d->eps >= 0.f)) return PAL_E_DIM;
  if (d->norm_over_heads && (int64_t)d->n_heads * d->dv > 512 * kHeadsMaxCh) return PAL_E_DIM;
  if (!(d->dt_min <= d->dt_max)) return PAL_E_DIM;   // also refuses NaN bounds
  return PAL_OK;
}

static int check_prologue(const PalGlueDims* d, const PalPrologueTensors* t) {
  if (int rc = check_glue_dims(d)) return rc;
  if (!t) return PAL_E_NULL;
  if (!t->x || !t->dt_raw || !t->dt_bias || !t->v || !t->gt) return PAL_E_NULL;
  // q, k rows: all four tensors or none (the MetaMamba2 form hands its B, C rows to the operator as they are)
  const int n_qk = (t->q_raw != nullptr) + (t->k_raw != nullptr) + (t->q != nullptr) + (t->k != nullptr);
  if (n_qk != 0 && n_qk != 4) return PAL_E_NULL;
  if (t->bs_raw && n_qk == 0) return PAL_E_NULL;     // the Palimpsa layer's form always has them
  if ((t->b_raw != nullptr) != (t->b != nullptr)) return PAL_E_STATE;
  if (t->b_raw && !t->b_scale) return PAL_E_NULL;
  const void* ptrs[] = {t->q_raw, t->k_raw, t->x, t->b_raw, t->q, t->k, t->v, t->b};
  for (const void* p : ptrs)
    if (p && !is_aligned16(p)) return PAL_E_ALIGN;
  return PAL_OK;
}

static void fill_prologue(PrologueArgs& A, const PalGlueDims* d, const PalPrologueTensors* t) {
  const GlueGeom g = glue_geom(d);
  A.t = *t;
  A.tokens = d->tokens; A.H = d->n_heads; A.Hqk = d->n_qk_heads; A.dk = d->dk; A.dv = d->dv;
  A.GLk = g.GLk; A.GLv = g.GLv; A.tok_per_block = g.tok_per_block;
  A.eps = d->eps;
  A.part = nullptr;
  A.mamba = t->bs_raw == nullptr;
  A.task0 = t->q_raw ? 0 : 2;
  A.dt_min = d->dt_min; A.dt_max = d->dt_max;
}

static int check_epilogue(const PalGlueDims* d, const PalEpilogueTensors* t) {
  if (int rc = check_glue_dims(d)) return rc;
  if (!t) return PAL_E_NULL;
  if (!t->o || !t->weight || !t->y || !t->rstd) return PAL_E_NULL;
  if (t->x && !t->D) return PAL_E_NULL;
  const void* ptrs[] = {t->o, t->x, t->gate, t->weight, t->y};
  for (const void* p : ptrs)
    if (p && !is_aligned16(p)) return PAL_E_ALIGN;
  return PAL_OK;
}

static void fill_epilogue(EpilogueArgs& A, const PalGlueDims* d, const PalEpilogueTensors* t) {
  const GlueGeom g = glue_geom(d);
  A.t = *t;
  A.tokens = d->tokens; A.H = d->n_heads; A.dv = d->dv;
  A.GL = g.GLv; A.tok_per_block = (256 / g.GLv) * kGlueIter;
  A.eps = d->eps;
  A.part_w = nullptr; A.part_D = nullptr;
}

static size_t up256(size_t x) { return (x + 255) & ~(size_t)255; }

}  // namespace pal

extern "C" int pal_prologue_fwd(const PalGlueDims* d, const PalPrologueTensors* t, void* stream) {
  using namespace pal;
  if (int rc = check_prologue(d, t)) return rc;
  PrologueArgs A{};
  fill_prologue(A, d, t);
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid((d->tokens + A.tok_per_block - 1) / A.tok_per_block, d->n_heads, 3 - A.task0);
  if (d->dtype == PAL_DTYPE_BF16) PAL_TIMED_LAUNCH(kKernPrologueFwd, s, prologue_fwd_kernel<bf16_t>, grid, dim3(256), 0, s, A);
  else PAL_TIMED_LAUNCH(kKernPrologueFwd, s, prologue_fwd_kernel<float>, grid, dim3(256), 0, s, A);
  PAL_HIP_LAUNCH_CHECK();
  return PAL_OK;
}

extern "C" size_t pal_prologue_bwd_workspace_bytes(const PalGlueDims* d) {
  using namespace pal;
  if (check_glue_dims(d) != PAL_OK) return 0;
  const GlueGeom g = glue_geom(d);
  const size_t nb = (d->tokens + g.tok_per_block - 1) / g.tok_per_block;
  return up256(sizeof(float) * 2 * nb * d->n_heads);
}

extern "C" int pal_prologue_bwd(const PalGlueDims* d, const PalPrologueTensors* t, const PalPrologueGrads* gr,
                                void* workspace, size_t workspace_bytes, void* stream) {
  using namespace pal;
  if (int rc = check_prologue(d, t)) return rc;
  if (!gr) return PAL_E_NULL;
  if (!gr->dv || !gr->dgt || !gr->dx || !gr->ddt_raw || !gr->ddt_bias) return PAL_E_NULL;
  if (t->q_raw && (!gr->dq || !gr->dk || !gr->dq_raw || !gr->dk_raw)) return PAL_E_NULL;
  if (t->bs_raw && !gr->dbs_raw) return PAL_E_NULL;
  if (t->b_raw && (!gr->db || !gr->db_raw || !gr->db_scale)) return PAL_E_NULL;
  const void* ptrs[] = {gr->dq, gr->dk, gr->dv, gr->db, gr->dq_raw, gr->dk_raw, gr->dx, gr->db_raw, workspace};
  for (const void* p : ptrs)
    if (p && !is_aligned16(p)) return PAL_E_ALIGN;
  if (!workspace || workspace_bytes < pal_prologue_bwd_workspace_bytes(d)) return PAL_E_WORKSPACE;
  PrologueArgs A{};
  fill_prologue(A, d, t);
  A.g = *gr;
  A.part = (float*)workspace;
  hipStream_t s = (hipStream_t)stream;
  const int nb = (d->tokens + A.tok_per_block - 1) / A.tok_per_block;
  const dim3 grid(nb, d->n_heads, 3 - A.task0);
  if (d->dtype == PAL_DTYPE_BF16) PAL_TIMED_LAUNCH(kKernPrologueBwd, s, prologue_bwd_kernel<bf16_t>, grid, dim3(256), 0, s, A);
  else PAL_TIMED_LAUNCH(kKernPrologueBwd, s, prologue_bwd_kernel<float>, grid, dim3(256), 0, s, A);
  PAL_HIP_LAUNCH_CHECK();
  hipLaunchKernelGGL(prologue_bwd_reduce_kernel, dim3(d->n_heads), dim3(64), 0, s, A, nb);
  PAL_HIP_LAUNCH_CHECK();
  return PAL_OK;
}

extern "C" int pal_epilogue_fwd(const PalGlueDims* d, const PalEpilogueTensors* t, void* stream) {
  using namespace pal;
  if (int rc = check_epilogue(d, t)) return rc;
  EpilogueArgs A{};
  fill_epilogue(A, d, t);
  hipStream_t s = (hipStream_t)stream;
  if (d->norm_over_heads) {
    const dim3 hgrid((heads_waves(d) + 3) / 4);
    if (d->dtype == PAL_DTYPE_BF16) PAL_TIMED_LAUNCH(kKernEpilogueFwd, s, epilogue_heads_fwd_kernel<bf16_t>, hgrid, dim3(256), 0, s, A);
    else PAL_TIMED_LAUNCH(kKernEpilogueFwd, s, epilogue_heads_fwd_kernel<float>, hgrid, dim3(256), 0, s, A);
    PAL_HIP_LAUNCH_CHECK();
    return PAL_OK;
  }
  const dim3 grid((d->tokens + A.tok_per_block - 1) / A.tok_per_block, d->n_heads);
  if (d->dtype == PAL_DTYPE_BF16) PAL_TIMED_LAUNCH(kKernEpilogueFwd, s, epilogue_fwd_kernel<bf16_t>, grid, dim3(256), 0, s, A);
  else PAL_TIMED_LAUNCH(kKernEpilogueFwd, s, epilogue_fwd_kernel<float>, grid, dim3(256), 0, s, A);
  PAL_HIP_LAUNCH_CHECK();
  return PAL_OK;
}

extern "C" size_t pal_epilogue_bwd_workspace_bytes(const PalGlueDims* d) {
  using namespace pal;
  if (check_glue_dims(d) != PAL_OK) return 0;
  if (d->norm_over_heads) {
    const size_t HD = (size_t)d->n_heads * d->dv, nblk = (size_t)((heads_waves(d) + 3) / 4);
    return up256(sizeof(float) * nblk * HD) + up256(sizeof(float) * nblk * (HD / 8));
  }
  const GlueGeom g = glue_geom(d);
  const int tpb = (256 / g.GLv) * kGlueIter;
  const size_t nb = (d->tokens + tpb - 1) / tpb;
  return up256(sizeof(float) * nb * d->n_heads * d->dv) + up256(sizeof(float) * nb * d->n_heads);
}

extern "C" int pal_epilogue_bwd(const PalGlueDims* d, const PalEpilogueTensors* t, const PalEpilogueGrads* gr,
                                void* workspace, size_t workspace_bytes, void* stream) {
  using namespace pal;
  if (int rc = check_epilogue(d, t)) return rc;
  if (!gr) return PAL_E_NULL;
  if (!gr->dy || !gr->d_o || !gr->dweight) return PAL_E_NULL;
  if (t->x && (!gr->dx || !gr->dD)) return PAL_E_NULL;
  if (t->gate && !gr->dgate) return PAL_E_NULL;
  const void* ptrs[] = {gr->dy, gr->d_o, gr->dx, gr->dgate, workspace};
  for (const void* p : ptrs)
    if (p && !is_aligned16(p)) return PAL_E_ALIGN;
  if (!workspace || workspace_bytes < pal_epilogue_bwd_workspace_bytes(d)) return PAL_E_WORKSPACE;
  EpilogueArgs A{};
  fill_epilogue(A, d, t);
  A.g = *gr;
  if (d->norm_over_heads) {
    const int nblk = (heads_waves(d) + 3) / 4;
    const size_t HD = (size_t)d->n_heads * d->dv;
    A.part_w = (float*)workspace;
    A.part_D = (float*)((char*)workspace + up256(sizeof(float) * (size_t)nblk * HD));
    hipStream_t hs = (hipStream_t)stream;
    const size_t lds = sizeof(float) * 4 * (HD + HD / 8);
    const int nch = (int)((HD + 511) / 512);
    if (int rc = d->dtype == PAL_DTYPE_BF16 ? launch_heads_bwd_nch<bf16_t>(nch, A, nblk, lds, hs)
                                            : launch_heads_bwd<float, 0>(A, nblk, lds, hs))
      return rc;
    PAL_HIP_LAUNCH_CHECK();
    hipLaunchKernelGGL(epilogue_heads_reduce_kernel, dim3((unsigned)((HD + 63) / 64 + d->n_heads)), dim3(64 * kRedWaves), 0, hs, A, nblk);
    PAL_HIP_LAUNCH_CHECK();
    return PAL_OK;
  }
  const int nb = (d->tokens + A.tok_per_block - 1) / A.tok_per_block;
  A.part_w = (float*)workspace;
  A.part_D = (float*)((char*)workspace + up256(sizeof(float) * (size_t)nb * d->n_heads * d->dv));
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid(nb, d->n_heads);
  const size_t lds = sizeof(float) * (256 / A.GL) * 8 * A.GL;   // = 8 KB
  if (d->dtype == PAL_DTYPE_BF16) PAL_TIMED_LAUNCH(kKernEpilogueBwd, s, epilogue_bwd_kernel<bf16_t>, grid, dim3(256), lds, s, A);
  else PAL_TIMED_LAUNCH(kKernEpilogueBwd, s, epilogue_bwd_kernel<float>, grid, dim3(256), lds, s, A);
  PAL_HIP_LAUNCH_CHECK();
  hipLaunchKernelGGL(epilogue_bwd_reduce_kernel, dim3(d->dv + d->n_heads), dim3(64), 0, s, A, nb);
  PAL_HIP_LAUNCH_CHECK();
  return PAL_OK;
}
