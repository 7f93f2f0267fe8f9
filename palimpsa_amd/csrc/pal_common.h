// Shared device/host helpers for the Palimpsa HIP kernels (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/palimpsa_hip.h"

namespace pal {

typedef __bf16 bf16_t;
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16_t;
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));

constexpr float kLog2e = 1.4426950408889634f;

// ------------------------------------------------------------------ scalars
__device__ __forceinline__ float to_f32(float x) { return x; }
__device__ __forceinline__ float to_f32(bf16_t x) { return (float)x; }

template <typename T>
__device__ __forceinline__ T from_f32(float x);
template <>
__device__ __forceinline__ float from_f32<float>(float x) { return x; }
template <>
__device__ __forceinline__ bf16_t from_f32<bf16_t>(float x) { return (bf16_t)x; }

__device__ __forceinline__ float fast_rcp(float x) { return __builtin_amdgcn_rcpf(x); }
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// gate tensor element i, fp32 or bf16 storage chosen at run time
__device__ __forceinline__ float load_gate(const void* p, int64_t i, int is_bf16) {
  return is_bf16 ? (float)((const bf16_t*)p)[i] : ((const float*)p)[i];
}

// the same in two steps for loops that keep several requests in flight: now the aligned 32-bit word that holds the
// element (one request of the same kind for both storage types, so that no wait is forced where the two would
// meet), later the value from the word
__device__ __forceinline__ unsigned load_gate_word(const void* p, int64_t i, int is_bf16) {
  const int64_t byte = is_bf16 ? 2 * i : 4 * i;
  return *(const unsigned*)((const char*)p + (byte & ~(int64_t)3));
}
__device__ __forceinline__ float gate_value(unsigned word, int64_t i, int is_bf16) {
  const unsigned bits = is_bf16 ? ((i & 1) ? (word & 0xffff0000u) : (word << 16)) : word;
  return __builtin_bit_cast(float, bits);
}

// store to an output whose element type is chosen at run time
__device__ __forceinline__ void store_rt(void* p, int64_t i, float x, int is_bf16) {
  if (is_bf16) ((bf16_t*)p)[i] = (bf16_t)x;
  else ((float*)p)[i] = x;
}
__device__ __forceinline__ float load_rt(const void* p, int64_t i, int is_bf16) {
  return is_bf16 ? (float)((const bf16_t*)p)[i] : ((const float*)p)[i];
}

// First token and length of sequence n of a packed batch of `total` tokens.  Both ends are clamped to the token
// range (a length below zero becomes zero), so that a cu_seqlens array that is not what the interface asks for
// (ascending from 0 to the token count) cannot make a kernel address memory beyond the tensors.
__device__ __forceinline__ void packed_seq_bounds(const int32_t* cu, int n, int total, int& bos, int& len) {
  const int s = min(max(cu[n], 0), total);
  const int e = min(max(cu[n + 1], s), total);
  bos = s;
  len = e - s;
}

// ---------------------------------------------------------- vector loads
// VW consecutive elements starting at p (aligned to VW*sizeof(T)) -> fp32
template <int VW>
__device__ __forceinline__ void load_vec(const float* p, float* out) {
  if constexpr (VW == 4) {
    f32x4 x = *(const f32x4*)p;
    out[0] = x[0]; out[1] = x[1]; out[2] = x[2]; out[3] = x[3];
  } else if constexpr (VW == 2) {
    f32x2 x = *(const f32x2*)p;
    out[0] = x[0]; out[1] = x[1];
  } else {
    out[0] = *p;
  }
}
template <int VW>
__device__ __forceinline__ void load_vec(const bf16_t* p, float* out) {
  if constexpr (VW == 4) {
    bf16x4 x = *(const bf16x4*)p;
    out[0] = (float)x[0]; out[1] = (float)x[1]; out[2] = (float)x[2]; out[3] = (float)x[3];
  } else if constexpr (VW == 2) {
    bf16x2 x = *(const bf16x2*)p;
    out[0] = (float)x[0]; out[1] = (float)x[1];
  } else {
    out[0] = (float)*p;
  }
}
// eight consecutive elements of a row as fetched (two 8- or 16-byte accesses), converted when they are used
template <typename T>
struct Raw8;
template <>
struct Raw8<bf16_t> {
  bf16x4 lo, hi;
  __device__ __forceinline__ void load(const bf16_t* p) { lo = *(const bf16x4*)p; hi = *(const bf16x4*)(p + 4); }
  __device__ __forceinline__ float get(int e) const { return (float)(e < 4 ? lo[e & 3] : hi[e & 3]); }
};
template <>
struct Raw8<float> {
  f32x4 lo, hi;
  __device__ __forceinline__ void load(const float* p) { lo = *(const f32x4*)p; hi = *(const f32x4*)(p + 4); }
  __device__ __forceinline__ float get(int e) const { return e < 4 ? lo[e & 3] : hi[e & 3]; }
};
template <int VW>
__device__ __forceinline__ void store_vec(float* p, const float* in) {
  if constexpr (VW == 4) {
    f32x4 x = {in[0], in[1], in[2], in[3]};
    *(f32x4*)p = x;
  } else if constexpr (VW == 2) {
    f32x2 x = {in[0], in[1]};
    *(f32x2*)p = x;
  } else {
    *p = in[0];
  }
}

// streaming variants for data that is touched exactly once (decode state): no reuse, so hint the
// caches not to keep it
template <int VW>
__device__ __forceinline__ void load_vec_stream(const float* p, float* out) {
  if constexpr (VW == 4) {
    f32x4 x = __builtin_nontemporal_load((const f32x4*)p);
    out[0] = x[0]; out[1] = x[1]; out[2] = x[2]; out[3] = x[3];
  } else if constexpr (VW == 2) {
    f32x2 x = __builtin_nontemporal_load((const f32x2*)p);
    out[0] = x[0]; out[1] = x[1];
  } else {
    out[0] = __builtin_nontemporal_load(p);
  }
}
template <int VW>
__device__ __forceinline__ void store_vec_stream(float* p, const float* in) {
  if constexpr (VW == 4) {
    f32x4 x = {in[0], in[1], in[2], in[3]};
    __builtin_nontemporal_store(x, (f32x4*)p);
  } else if constexpr (VW == 2) {
    f32x2 x = {in[0], in[1]};
    __builtin_nontemporal_store(x, (f32x2*)p);
  } else {
    __builtin_nontemporal_store(in[0], p);
  }
}

// the same for a bf16 array (a state kept in bf16): widened to fp32 on load, rounded to nearest even on store
template <int VW>
__device__ __forceinline__ void load_vec_stream(const bf16_t* p, float* out) {
  if constexpr (VW == 4) {
    const bf16x4 x = __builtin_bit_cast(bf16x4, __builtin_nontemporal_load((const f32x2*)p));
    out[0] = (float)x[0]; out[1] = (float)x[1]; out[2] = (float)x[2]; out[3] = (float)x[3];
  } else if constexpr (VW == 2) {
    const bf16x2 x = __builtin_bit_cast(bf16x2, __builtin_nontemporal_load((const float*)p));
    out[0] = (float)x[0]; out[1] = (float)x[1];
  } else {
    out[0] = (float)__builtin_bit_cast(bf16_t, __builtin_nontemporal_load((const unsigned short*)p));
  }
}
template <int VW>
__device__ __forceinline__ void store_vec_stream(bf16_t* p, const float* in) {
  if constexpr (VW == 4) {
    const bf16x4 x = {(bf16_t)in[0], (bf16_t)in[1], (bf16_t)in[2], (bf16_t)in[3]};
    __builtin_nontemporal_store(__builtin_bit_cast(f32x2, x), (f32x2*)p);
  } else if constexpr (VW == 2) {
    const bf16x2 x = {(bf16_t)in[0], (bf16_t)in[1]};
    __builtin_nontemporal_store(__builtin_bit_cast(float, x), (float*)p);
  } else {
    __builtin_nontemporal_store(__builtin_bit_cast(unsigned short, (bf16_t)in[0]), (unsigned short*)p);
  }
}

// ------------------------------------------------------- cross-lane helpers
// rotate within each row of 16 lanes (DPP row_ror:N)
template <int N>
__device__ __forceinline__ float row_ror(float x) {
  int v = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x120 + N, 0xf, 0xf, false);
  return __builtin_bit_cast(float, v);
}
// sum over the 16 lanes of a row; every lane of the row gets the total
__device__ __forceinline__ float row16_sum(float x) {
  x += row_ror<8>(x);
  x += row_ror<4>(x);
  x += row_ror<2>(x);
  x += row_ror<1>(x);
  return x;
}
// gfx950 lane swaps run in the VALU; the LDS-routed shuffles they replace cost ~64 cycles of latency each.
// Written as inline assembly: with hipcc 7.2 the two results of the __builtin_amdgcn_permlane*_swap
// builtins are merged into one register when both feed the same arithmetic instruction.  The s_nop
// covers the two wait states the instruction needs after a VALU write of its operands.
// a <- {a lanes 0-31, b lanes 0-31}, b <- {a lanes 32-63, b lanes 32-63}
__device__ __forceinline__ void swap_halves(float& a, float& b) {
  asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(a), "+v"(b));
}
// rows of 16 lanes: a <- {a0, b0, a2, b2}, b <- {a1, b1, a3, b3}
__device__ __forceinline__ void swap_rows(float& a, float& b) {
  asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1" : "+v"(a), "+v"(b));
}
// sum over the four 16-lane rows of a wave (same lane-in-row); all lanes get it
__device__ __forceinline__ float rows4_sum(float x) {
  float a = x, b = x;
  swap_halves(a, b);
  a += b;
  b = a;
  swap_rows(a, b);
  return a + b;
}
// four partials, each to be summed over the four rows: the lanes of row g get the total of p_g
__device__ __forceinline__ float rows4_sum_x4(float p0, float p1, float p2, float p3) {
  swap_halves(p0, p2);   // rows 0,1: p0 summed over row pairs; rows 2,3: p2
  swap_halves(p1, p3);
  float s0 = p0 + p2, s1 = p1 + p3;
  swap_rows(s0, s1);
  return s0 + s1;
}
__device__ __forceinline__ float wave_sum(float x) { return rows4_sum(row16_sum(x)); }
// maximum over the 64 lanes of a wave; every lane gets it
__device__ __forceinline__ float wave_max(float x) {
  x = fmaxf(x, row_ror<8>(x));
  x = fmaxf(x, row_ror<4>(x));
  x = fmaxf(x, row_ror<2>(x));
  x = fmaxf(x, row_ror<1>(x));
  float a = x, b = x;
  swap_halves(a, b);
  a = fmaxf(a, b);
  b = a;
  swap_rows(a, b);
  return fmaxf(a, b);
}

// ------------------------------------------------------------------- MFMA
// D[16x16] += A[16x32] * B[32x16], bf16 operands, fp32 accumulate.
// lane l holds: A row (l%16), k = 8*(l/16)+j ; B col (l%16), same k ;
// D col (l%16), rows 4*(l/16)+r.
__device__ __forceinline__ f32x4 mfma16(bf16x8 a, bf16x8 b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}

// same shape with f16 operands (11-bit mantissa; range handled by the caller's block exponent)
__device__ __forceinline__ f32x4 mfma16h(f16x8 a, f16x8 b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
}

// Operands of the fp32-accurate variants of the chunked kernels: a value is carried as the sum of two bf16 numbers
// (16 mantissa bits together) and a product of two such operands as three matrix instructions (the lo x lo term,
// 2^-18 of the result, is dropped); accumulation is fp32 as always.
__device__ __forceinline__ void split_bf16(const float* x, bf16x8& hi, bf16x8& lo) {
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    hi[j] = (bf16_t)x[j];
    lo[j] = (bf16_t)(x[j] - (float)hi[j]);
  }
}
__device__ __forceinline__ f32x4 mfma16_split(bf16x8 ah, bf16x8 al, bf16x8 bh, bf16x8 bl, f32x4 c) {
  c = mfma16(al, bh, c);
  c = mfma16(ah, bl, c);
  return mfma16(ah, bh, c);
}

__device__ __forceinline__ bf16x2 pack2(float lo, float hi) {
  f32x2 x = {lo, hi};
  return __builtin_convertvector(x, bf16x2);
}
template <int VW>
__device__ __forceinline__ void store_vec(bf16_t* p, const float* in) {
  if constexpr (VW == 4) {
    const bf16x2 a = pack2(in[0], in[1]), b = pack2(in[2], in[3]);
    const bf16x4 x = {a[0], a[1], b[0], b[1]};
    *(bf16x4*)p = x;
  } else if constexpr (VW == 2) {
    *(bf16x2*)p = pack2(in[0], in[1]);
  } else {
    *p = (bf16_t)in[0];
  }
}

// ------------------------------------------------------------------ host
#define PAL_HIP_LAUNCH_CHECK()                 \
  do {                                         \
    hipError_t e__ = hipGetLastError();        \
    if (e__ != hipSuccess) return (int)e__;    \
  } while (0)

// LDS of one gfx950 compute unit; a launch asking for more than 64 KiB of dynamic
// LDS has to raise the kernel's limit first.
constexpr size_t kMaxLds = 160 * 1024;
inline int allow_lds(const void* kernel, size_t bytes) {
  if (bytes <= 64 * 1024) return 0;
  hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
  return e == hipSuccess ? 0 : (int)e;
}

inline bool is_aligned16(const void* p) { return (((uintptr_t)p) & 15u) == 0; }
inline bool is_aligned4(const void* p) { return (((uintptr_t)p) & 3u) == 0; }

}  // namespace pal
