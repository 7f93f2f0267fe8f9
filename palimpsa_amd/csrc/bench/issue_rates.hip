// Issue rates of the instructions the chunked kernels are made of, measured on the GPU at hand.
// One workgroup of 4*W waves per compute unit (W waves per SIMD, W = 1, 2, 4), a loop of one kind of
// instruction (or a fixed mix), wall-clock time by HIP events: the figure printed is SIMD cycles per wave64
// instruction at the device's reported clock.  The mixes answer what bounds the chunked kernels: whether a
// matrix instruction's time adds to that of the vector instructions of the same SIMD (same wave, or other
// waves of the SIMD) or hides behind it.
// Build: hipcc --offload-arch=gfx950 -O3 issue_rates.hip -o issue_rates   (palimpsa_amd.build does it)
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4;
#define HIP_OK(x)                                                              \
  do {                                                                         \
    hipError_t e__ = (x);                                                      \
    if (e__ != hipSuccess) { printf("%s: %s\n", #x, hipGetErrorString(e__)); exit(1); } \
  } while (0)
#define REP4(x) x x x x
#define REP16(x) REP4(REP4(x))
#define REP64(x) REP4(REP16(x))
constexpr int ITER = 4096;

template <int MODE> __global__ void k(float* out, long long* cyc, float a, float b) {
  extern __shared__ float lds[];
  float x0 = threadIdx.x, x1 = x0 + 1, x2 = x0 + 2, x3 = x0 + 3;
  f32x4 c0 = {0, 0, 0, 0}, c1 = c0, c2 = c0, c3 = c0;
  bf16x8 A, B;
  for (int j = 0; j < 8; ++j) { A[j] = (__bf16)(float)(threadIdx.x + j); B[j] = (__bf16)1.f; }
  int addr = ((threadIdx.x * 4) & 255) ;
  int addr16 = threadIdx.x * 16 & 1023;
  lds[threadIdx.x] = 0.f;
  __syncthreads();
  long long t0 = clock64();
  for (int it = 0; it < ITER; ++it) {
    if (MODE == 0) {  // dependent fma chain, 64 per iter
      REP64(asm volatile("v_fma_f32 %0, %0, %1, %2" : "+v"(x0) : "v"(a), "v"(b));)
    } else if (MODE == 1) {  // 4 independent chains, 64 per iter
      REP16(asm volatile("v_fma_f32 %0, %0, %4, %5\n v_fma_f32 %1, %1, %4, %5\n v_fma_f32 %2, %2, %4, %5\n v_fma_f32 %3, %3, %4, %5"
                         : "+v"(x0), "+v"(x1), "+v"(x2), "+v"(x3) : "v"(a), "v"(b));)
    } else if (MODE == 2) {  // dependent mfma chain, 16 per iter
      REP16(asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+v"(c0) : "v"(A), "v"(B));)
    } else if (MODE == 3) {  // 4 independent mfma, 16 per iter
      REP4(asm volatile("v_mfma_f32_16x16x32_bf16 %0, %4, %5, %0\n v_mfma_f32_16x16x32_bf16 %1, %4, %5, %1\n v_mfma_f32_16x16x32_bf16 %2, %4, %5, %2\n v_mfma_f32_16x16x32_bf16 %3, %4, %5, %3"
                        : "+v"(c0), "+v"(c1), "+v"(c2), "+v"(c3) : "v"(A), "v"(B));)
    } else if (MODE == 4) {  // 1 independent-ish mfma + 3 fma (independent chains), x16 => 16 mfma + 48 fma
      REP16(asm volatile("v_mfma_f32_16x16x32_bf16 %0, %4, %5, %0\n v_fma_f32 %1, %1, %6, %7\n v_fma_f32 %2, %2, %6, %7\n v_fma_f32 %3, %3, %6, %7"
                         : "+v"(c0), "+v"(x1), "+v"(x2), "+v"(x3) : "v"(A), "v"(B), "v"(a), "v"(b));)
    } else if (MODE == 5) {  // rcp dependent chain 64
      REP64(asm volatile("v_rcp_f32 %0, %0" : "+v"(x0));)
    } else if (MODE == 6) {  // rcp independent 4 chains
      REP16(asm volatile("v_rcp_f32 %0, %0\n v_rcp_f32 %1, %1\n v_rcp_f32 %2, %2\n v_rcp_f32 %3, %3" : "+v"(x0), "+v"(x1), "+v"(x2), "+v"(x3));)
    } else if (MODE == 7) {  // cvt_pk_bf16 independent
      unsigned r0, r1, r2, r3;
      REP16(asm volatile("v_cvt_pk_bf16_f32 %0, %4, %5\n v_cvt_pk_bf16_f32 %1, %5, %6\n v_cvt_pk_bf16_f32 %2, %6, %7\n v_cvt_pk_bf16_f32 %3, %7, %4"
                         : "=v"(r0), "=v"(r1), "=v"(r2), "=v"(r3) : "v"(x0), "v"(x1), "v"(x2), "v"(x3));)
      x0 += __uint_as_float(r0 ^ r1 ^ r2 ^ r3) * 1e-30f;
    } else if (MODE == 8) {  // ds_bpermute dependent chain: 16 per iter
      int v = __float_as_int(x0);
      REP16(asm volatile("ds_bpermute_b32 %0, %1, %0\n s_waitcnt lgkmcnt(0)" : "+v"(v) : "v"(addr));)
      x0 = __int_as_float(v);
    } else if (MODE == 9) {  // 1 mfma + 7 fma (independent chains of 4) x8 => 8 mfma + 56 fma
      REP4(REP4(asm volatile("v_mfma_f32_16x16x32_bf16 %0, %4, %5, %0\n v_fma_f32 %1, %1, %6, %7\n v_fma_f32 %2, %2, %6, %7\n v_fma_f32 %3, %3, %6, %7\n"
                        "v_fma_f32 %8, %8, %6, %7\n v_fma_f32 %1, %1, %6, %7\n v_fma_f32 %2, %2, %6, %7\n v_fma_f32 %3, %3, %6, %7"
                         : "+v"(c0), "+v"(x1), "+v"(x2), "+v"(x3) : "v"(A), "v"(B), "v"(a), "v"(b), "v"(x0));) )
    } else if (MODE == 10) {  // exp independent
      REP16(asm volatile("v_exp_f32 %0, %0\n v_exp_f32 %1, %1\n v_exp_f32 %2, %2\n v_exp_f32 %3, %3" : "+v"(x0), "+v"(x1), "+v"(x2), "+v"(x3));)
    } else if (MODE == 11) {  // dpp row_ror adds, dependent
      REP64(asm volatile("v_add_f32_dpp %0, %0, %0 row_ror:4 row_mask:0xf bank_mask:0xf" : "+v"(x0));)
    } else if (MODE == 12) {  // permlane32 swap dependent
      REP64(asm volatile("v_permlane32_swap_b32 %0, %1" : "+v"(x0), "+v"(x1));)
    } else if (MODE == 14) {  // wave parity: even waves mfma only (16), odd waves fma only (64)
      if ((threadIdx.x >> 6) & 1) {
        REP16(asm volatile("v_fma_f32 %0, %0, %4, %5\n v_fma_f32 %1, %1, %4, %5\n v_fma_f32 %2, %2, %4, %5\n v_fma_f32 %3, %3, %4, %5"
                         : "+v"(x0), "+v"(x1), "+v"(x2), "+v"(x3) : "v"(a), "v"(b));)
      } else {
        REP4(asm volatile("v_mfma_f32_16x16x32_bf16 %0, %4, %5, %0\n v_mfma_f32_16x16x32_bf16 %1, %4, %5, %1\n v_mfma_f32_16x16x32_bf16 %2, %4, %5, %2\n v_mfma_f32_16x16x32_bf16 %3, %4, %5, %3"
                        : "+v"(c0), "+v"(c1), "+v"(c2), "+v"(c3) : "v"(A), "v"(B));)
      }
    } else if (MODE == 15) {
      REP16(asm volatile("v_mul_f32 %0, %0, %4\n v_mul_f32 %1, %1, %4\n v_mul_f32 %2, %2, %4\n v_mul_f32 %3, %3, %4" : "+v"(x0), "+v"(x1), "+v"(x2), "+v"(x3) : "v"(a), "v"(b));)
    } else if (MODE == 16) {
      REP16(asm volatile("v_add_f32 %0, %0, %4\n v_add_f32 %1, %1, %4\n v_add_f32 %2, %2, %4\n v_add_f32 %3, %3, %4" : "+v"(x0), "+v"(x1), "+v"(x2), "+v"(x3) : "v"(a), "v"(b));)
    } else if (MODE == 17) {
      REP16(asm volatile("v_fmac_f32 %0, %4, %5\n v_fmac_f32 %1, %4, %5\n v_fmac_f32 %2, %4, %5\n v_fmac_f32 %3, %4, %5" : "+v"(x0), "+v"(x1), "+v"(x2), "+v"(x3) : "v"(a), "v"(b));)
    } else if (MODE == 18) {
      REP16(asm volatile("v_and_b32 %0, %0, %4\n v_or_b32 %1, %1, %4\n v_lshlrev_b32 %2, 1, %2\n v_perm_b32 %3, %3, %4, %5" : "+v"(x0), "+v"(x1), "+v"(x2), "+v"(x3) : "v"(a), "v"(b));)
    } else if (MODE == 19) {
      REP16(asm volatile("v_cndmask_b32 %0, %0, %4, vcc\n v_max_f32 %1, %1, %4\n v_mov_b32 %2, %3\n v_mov_b32 %3, %2" : "+v"(x0), "+v"(x1), "+v"(x2), "+v"(x3) : "v"(a), "v"(b) : "vcc");)
    } else if (MODE == 20) {  // 8 independent fma chains
      float y0 = x0 * 2, y1 = x1 * 2, y2 = x2 * 2, y3 = x3 * 2;
      REP4(REP4(asm volatile("v_fma_f32 %0, %0, %4, %5\n v_fma_f32 %1, %1, %4, %5\n v_fma_f32 %2, %2, %4, %5\n v_fma_f32 %3, %3, %4, %5"
                         : "+v"(x0), "+v"(x1), "+v"(x2), "+v"(x3) : "v"(a), "v"(b));
           asm volatile("v_fma_f32 %0, %0, %4, %5\n v_fma_f32 %1, %1, %4, %5\n v_fma_f32 %2, %2, %4, %5\n v_fma_f32 %3, %3, %4, %5"
                         : "+v"(y0), "+v"(y1), "+v"(y2), "+v"(y3) : "v"(a), "v"(b));))
      x0 += y0 + y1 + y2 + y3;
    } else if (MODE == 21) {  // ds_read_b128 throughput: 16 independent reads then wait
      f32x4 r0, r1, r2, r3;
      REP4(asm volatile("ds_read_b128 %0, %4\n ds_read_b128 %1, %4 offset:1024\n ds_read_b128 %2, %4 offset:2048\n ds_read_b128 %3, %4 offset:3072\n s_waitcnt lgkmcnt(0)"
                        : "=v"(r0), "=v"(r1), "=v"(r2), "=v"(r3) : "v"(addr16));
           x0 += r0[0] + r1[1] + r2[2] + r3[3];)
    } else if (MODE == 22) {  // v_pk_mul_f16 4 chains
      REP16(asm volatile("v_pk_mul_f16 %0, %0, %4\n v_pk_mul_f16 %1, %1, %4\n v_pk_mul_f16 %2, %2, %4\n v_pk_mul_f16 %3, %3, %4" : "+v"(x0), "+v"(x1), "+v"(x2), "+v"(x3) : "v"(a), "v"(b));)
    } else if (MODE == 23) {  // f16 mfma 4 indep
      typedef _Float16 h8 __attribute__((ext_vector_type(8)));
      h8 HA, HB; for (int j = 0; j < 8; ++j) { HA[j] = (_Float16)(float)(threadIdx.x + j); HB[j] = (_Float16)1.f; }
      REP4(asm volatile("v_mfma_f32_16x16x32_f16 %0, %4, %5, %0\n v_mfma_f32_16x16x32_f16 %1, %4, %5, %1\n v_mfma_f32_16x16x32_f16 %2, %4, %5, %2\n v_mfma_f32_16x16x32_f16 %3, %4, %5, %3"
                        : "+v"(c0), "+v"(c1), "+v"(c2), "+v"(c3) : "v"(HA), "v"(HB));)
    } else if (MODE == 24) {  // v_cvt_pk_f16_f32 (rtz) indep
      unsigned r0, r1, r2, r3;
      REP16(asm volatile("v_cvt_pkrtz_f16_f32 %0, %4, %5\n v_cvt_pkrtz_f16_f32 %1, %5, %6\n v_cvt_pkrtz_f16_f32 %2, %6, %7\n v_cvt_pkrtz_f16_f32 %3, %7, %4"
                         : "=v"(r0), "=v"(r1), "=v"(r2), "=v"(r3) : "v"(x0), "v"(x1), "v"(x2), "v"(x3));)
      x0 += __uint_as_float(r0 ^ r1 ^ r2 ^ r3) * 1e-30f;
    } else if (MODE == 25) {  // legacy-shape mfma 16x16x16 bf16, 4 independent
      typedef __bf16 b4 __attribute__((ext_vector_type(4)));
      b4 A4, B4; for (int j = 0; j < 4; ++j) { A4[j] = (__bf16)(float)(threadIdx.x + j); B4[j] = (__bf16)1.f; }
      REP4(asm volatile("v_mfma_f32_16x16x16_bf16 %0, %4, %5, %0\n v_mfma_f32_16x16x16_bf16 %1, %4, %5, %1\n v_mfma_f32_16x16x16_bf16 %2, %4, %5, %2\n v_mfma_f32_16x16x16_bf16 %3, %4, %5, %3"
                        : "+v"(c0), "+v"(c1), "+v"(c2), "+v"(c3) : "v"(A4), "v"(B4));)
    } else if (MODE == 26) {  // v_dot2_f32_bf16, 4 chains
      REP16(asm volatile("v_dot2_f32_bf16 %0, %4, %5, %0\n v_dot2_f32_bf16 %1, %4, %5, %1\n v_dot2_f32_bf16 %2, %4, %5, %2\n v_dot2_f32_bf16 %3, %4, %5, %3"
                         : "+v"(x0), "+v"(x1), "+v"(x2), "+v"(x3) : "v"(a), "v"(b));)
    } else if (MODE == 27) {  // one wave in four issues mfma only (16), the other three fma only (64 each)
      if (((threadIdx.x >> 6) >> 2) == 0) {
        REP4(asm volatile("v_mfma_f32_16x16x32_bf16 %0, %4, %5, %0\n v_mfma_f32_16x16x32_bf16 %1, %4, %5, %1\n v_mfma_f32_16x16x32_bf16 %2, %4, %5, %2\n v_mfma_f32_16x16x32_bf16 %3, %4, %5, %3"
                        : "+v"(c0), "+v"(c1), "+v"(c2), "+v"(c3) : "v"(A), "v"(B));)
      } else {
        REP16(asm volatile("v_fma_f32 %0, %0, %4, %5\n v_fma_f32 %1, %1, %4, %5\n v_fma_f32 %2, %2, %4, %5\n v_fma_f32 %3, %3, %4, %5"
                         : "+v"(x0), "+v"(x1), "+v"(x2), "+v"(x3) : "v"(a), "v"(b));)
      }
    } else if (MODE == 28) {  // 4 independent mfma then 28 independent fma per block (same 1:7 mix, mfma back to back)
      REP4(asm volatile("v_mfma_f32_16x16x32_bf16 %0, %4, %5, %0\n v_mfma_f32_16x16x32_bf16 %1, %4, %5, %1\n v_mfma_f32_16x16x32_bf16 %2, %4, %5, %2\n v_mfma_f32_16x16x32_bf16 %3, %4, %5, %3"
                        : "+v"(c0), "+v"(c1), "+v"(c2), "+v"(c3) : "v"(A), "v"(B));
           REP4(asm volatile("v_fma_f32 %0, %0, %4, %5\n v_fma_f32 %1, %1, %4, %5\n v_fma_f32 %2, %2, %4, %5\n v_fma_f32 %3, %3, %4, %5\n v_fma_f32 %0, %0, %4, %5\n v_fma_f32 %1, %1, %4, %5\n v_fma_f32 %2, %2, %4, %5"
                         : "+v"(x0), "+v"(x1), "+v"(x2), "+v"(x3) : "v"(a), "v"(b));))
    } else if (MODE == 29) {  // mfma 32x32x16 bf16, 2 independent (16 accumulator registers each)
      typedef float f16v __attribute__((ext_vector_type(16)));
      f16v d0 = {0}, d1 = {0};
      REP4(REP4(asm volatile("v_mfma_f32_32x32x16_bf16 %0, %2, %3, %0\n v_mfma_f32_32x32x16_bf16 %1, %2, %3, %1"
                        : "+v"(d0), "+v"(d1) : "v"(A), "v"(B));))
      x0 += d0[0] + d1[5];
    } else if (MODE == 30) {  // 1 mfma + 7 salu-free "cheap" valu of mixed kinds (mul, add, fma, cvt_pk) as in the kernels
      unsigned r0;
      REP4(REP4(asm volatile("v_mfma_f32_16x16x32_bf16 %0, %5, %6, %0\n v_mul_f32 %1, %1, %7\n v_fma_f32 %2, %2, %7, %8\n v_add_f32 %3, %3, %8\n"
                        "v_cvt_pk_bf16_f32 %4, %1, %2\n v_mul_f32 %1, %1, %7\n v_fma_f32 %2, %2, %7, %8\n v_rcp_f32 %3, %3"
                         : "+v"(c0), "+v"(x1), "+v"(x2), "+v"(x3), "=v"(r0) : "v"(A), "v"(B), "v"(a), "v"(b));) )
      x0 += __uint_as_float(r0) * 1e-30f;
    } else if (MODE == 31) {  // the same 7 valu without the mfma
      unsigned r0;
      REP4(REP4(asm volatile("v_mul_f32 %1, %1, %7\n v_fma_f32 %2, %2, %7, %8\n v_add_f32 %3, %3, %8\n"
                        "v_cvt_pk_bf16_f32 %4, %1, %2\n v_mul_f32 %1, %1, %7\n v_fma_f32 %2, %2, %7, %8\n v_rcp_f32 %3, %3"
                         : "+v"(c0), "+v"(x1), "+v"(x2), "+v"(x3), "=v"(r0) : "v"(A), "v"(B), "v"(a), "v"(b));) )
      x0 += __uint_as_float(r0) * 1e-30f;
    } else if (MODE == 32) {  // matrix instructions of two operand types in turn (bf16, f16, bf16, f16), independent
      REP4(asm volatile("v_mfma_f32_16x16x32_bf16 %0, %4, %5, %0\n v_mfma_f32_16x16x32_f16 %1, %4, %5, %1\n v_mfma_f32_16x16x32_bf16 %2, %4, %5, %2\n v_mfma_f32_16x16x32_f16 %3, %4, %5, %3"
                        : "+v"(c0), "+v"(c1), "+v"(c2), "+v"(c3) : "v"(A), "v"(B));)
    } else if (MODE == 33) {  // half of the waves issue bf16 matrix instructions, the other half f16
      if ((threadIdx.x >> 6) & 4) {
        REP4(asm volatile("v_mfma_f32_16x16x32_bf16 %0, %4, %5, %0\n v_mfma_f32_16x16x32_bf16 %1, %4, %5, %1\n v_mfma_f32_16x16x32_bf16 %2, %4, %5, %2\n v_mfma_f32_16x16x32_bf16 %3, %4, %5, %3"
                          : "+v"(c0), "+v"(c1), "+v"(c2), "+v"(c3) : "v"(A), "v"(B));)
      } else {
        REP4(asm volatile("v_mfma_f32_16x16x32_f16 %0, %4, %5, %0\n v_mfma_f32_16x16x32_f16 %1, %4, %5, %1\n v_mfma_f32_16x16x32_f16 %2, %4, %5, %2\n v_mfma_f32_16x16x32_f16 %3, %4, %5, %3"
                          : "+v"(c0), "+v"(c1), "+v"(c2), "+v"(c3) : "v"(A), "v"(B));)
      }
    } else if (MODE == 34) {  // packed f16 multiply feeding a matrix instruction: 4 products + 1 matrix instruction, x4
      REP4(asm volatile("v_pk_mul_f16 %1, %1, %5\n v_pk_mul_f16 %2, %2, %5\n v_pk_mul_f16 %3, %3, %5\n v_pk_mul_f16 %4, %4, %5\n v_mfma_f32_16x16x32_f16 %0, %6, %7, %0"
                        : "+v"(c0), "+v"(x0), "+v"(x1), "+v"(x2), "+v"(x3) : "v"(a), "v"(A), "v"(B));)
    } else if (MODE == 40) {  // one wave in four issues matrix instructions only (16), the other three v_rcp_f32 (64 each)
      if (((threadIdx.x >> 6) >> 2) == 0) {
        REP4(asm volatile("v_mfma_f32_16x16x32_bf16 %0, %4, %5, %0\n v_mfma_f32_16x16x32_bf16 %1, %4, %5, %1\n v_mfma_f32_16x16x32_bf16 %2, %4, %5, %2\n v_mfma_f32_16x16x32_bf16 %3, %4, %5, %3"
                        : "+v"(c0), "+v"(c1), "+v"(c2), "+v"(c3) : "v"(A), "v"(B));)
      } else {
        REP16(asm volatile("v_rcp_f32 %0, %0\n v_rcp_f32 %1, %1\n v_rcp_f32 %2, %2\n v_rcp_f32 %3, %3" : "+v"(x0), "+v"(x1), "+v"(x2), "+v"(x3));)
      }
    } else if (MODE == 41) {  // one wave in four issues matrix instructions only (16), the other three v_cvt_pk_bf16_f32 (64 each)
      if (((threadIdx.x >> 6) >> 2) == 0) {
        REP4(asm volatile("v_mfma_f32_16x16x32_bf16 %0, %4, %5, %0\n v_mfma_f32_16x16x32_bf16 %1, %4, %5, %1\n v_mfma_f32_16x16x32_bf16 %2, %4, %5, %2\n v_mfma_f32_16x16x32_bf16 %3, %4, %5, %3"
                        : "+v"(c0), "+v"(c1), "+v"(c2), "+v"(c3) : "v"(A), "v"(B));)
      } else {
        unsigned r0, r1, r2, r3;
        REP16(asm volatile("v_cvt_pk_bf16_f32 %0, %4, %5\n v_cvt_pk_bf16_f32 %1, %5, %6\n v_cvt_pk_bf16_f32 %2, %6, %7\n v_cvt_pk_bf16_f32 %3, %7, %4" : "=v"(r0), "=v"(r1), "=v"(r2), "=v"(r3) : "v"(x0), "v"(x1), "v"(x2), "v"(x3));)
        x0 += __uint_as_float(r0 ^ r1 ^ r2 ^ r3) * 1e-30f;
      }
    } else if (MODE == 42) {  // one wave in four issues matrix instructions only (16), the other three v_pk_mul_f16 (64 each)
      if (((threadIdx.x >> 6) >> 2) == 0) {
        REP4(asm volatile("v_mfma_f32_16x16x32_bf16 %0, %4, %5, %0\n v_mfma_f32_16x16x32_bf16 %1, %4, %5, %1\n v_mfma_f32_16x16x32_bf16 %2, %4, %5, %2\n v_mfma_f32_16x16x32_bf16 %3, %4, %5, %3"
                        : "+v"(c0), "+v"(c1), "+v"(c2), "+v"(c3) : "v"(A), "v"(B));)
      } else {
        REP16(asm volatile("v_pk_mul_f16 %0, %0, %4\n v_pk_mul_f16 %1, %1, %4\n v_pk_mul_f16 %2, %2, %4\n v_pk_mul_f16 %3, %3, %4" : "+v"(x0), "+v"(x1), "+v"(x2), "+v"(x3) : "v"(a));)
      }
    } else if (MODE == 43) {  // one wave in four issues matrix instructions only (16), the other three v_and_b32 / v_lshlrev_b32 (64 each)
      if (((threadIdx.x >> 6) >> 2) == 0) {
        REP4(asm volatile("v_mfma_f32_16x16x32_bf16 %0, %4, %5, %0\n v_mfma_f32_16x16x32_bf16 %1, %4, %5, %1\n v_mfma_f32_16x16x32_bf16 %2, %4, %5, %2\n v_mfma_f32_16x16x32_bf16 %3, %4, %5, %3"
                        : "+v"(c0), "+v"(c1), "+v"(c2), "+v"(c3) : "v"(A), "v"(B));)
      } else {
        REP16(asm volatile("v_and_b32 %0, %0, %4\n v_lshlrev_b32 %1, 1, %1\n v_and_b32 %2, %2, %4\n v_lshlrev_b32 %3, 1, %3" : "+v"(x0), "+v"(x1), "+v"(x2), "+v"(x3) : "v"(a));)
      }
    } else if (MODE == 44) {  // one wave in four issues matrix instructions only (16), the other three v_permlane32_swap (64 each)
      if (((threadIdx.x >> 6) >> 2) == 0) {
        REP4(asm volatile("v_mfma_f32_16x16x32_bf16 %0, %4, %5, %0\n v_mfma_f32_16x16x32_bf16 %1, %4, %5, %1\n v_mfma_f32_16x16x32_bf16 %2, %4, %5, %2\n v_mfma_f32_16x16x32_bf16 %3, %4, %5, %3"
                        : "+v"(c0), "+v"(c1), "+v"(c2), "+v"(c3) : "v"(A), "v"(B));)
      } else {
        REP16(asm volatile("v_permlane32_swap_b32 %0, %1\n v_permlane32_swap_b32 %2, %3\n v_permlane32_swap_b32 %0, %1\n v_permlane32_swap_b32 %2, %3" : "+v"(x0), "+v"(x1), "+v"(x2), "+v"(x3));)
      }
    } else if (MODE == 13) {  // ds_read_b128 dependent latency (pointer chase on zeroed lds)
      int p = addr;
      REP16(asm volatile("ds_read_b32 %0, %0\n s_waitcnt lgkmcnt(0)" : "+v"(p));)
      x0 += p;
    }
  }
  long long t1 = clock64();
  out[blockIdx.x * blockDim.x + threadIdx.x] = x0 + x1 + x2 + x3 + c0[0] + c1[1] + c2[2] + c3[3];
  if (threadIdx.x == 0 && blockIdx.x == 0) *cyc = t1 - t0;
}

static double g_ghz = 2.4;
template <int MODE> void run(const char* name, int wps, int n_instr_per_iter, float* out, long long* cyc) {
  hipEvent_t e0, e1; HIP_OK(hipEventCreate(&e0)); HIP_OK(hipEventCreate(&e1));
  const int threads = wps * 256;
  HIP_OK(hipFuncSetAttribute((const void*)k<MODE>, hipFuncAttributeMaxDynamicSharedMemorySize, 100 * 1024));
  k<MODE><<<256, threads, 100 * 1024>>>(out, cyc, 0.999f, 0.001f);
  HIP_OK(hipEventRecord(e0));
  k<MODE><<<256, threads, 100 * 1024>>>(out, cyc, 0.999f, 0.001f);
  HIP_OK(hipEventRecord(e1)); HIP_OK(hipEventSynchronize(e1));
  float ms; HIP_OK(hipEventElapsedTime(&ms, e0, e1));
  long long c; HIP_OK(hipMemcpy(&c, cyc, 8, hipMemcpyDeviceToHost));
  const double n = (double)ITER * n_instr_per_iter;
  // n = instructions per wave; a SIMD runs wps waves, so SIMD cycles per instruction = cycles / (n * wps)
  printf("%-44s waves/SIMD=%d  ms=%.4f  SIMD cycles per wave instruction=%.2f\n", name, wps, ms,
         ms * 1e-3 * g_ghz * 1e9 / (n * wps));
  fflush(stdout);
}

// ---- LDS access patterns: LDS cycles per wave64 instruction when all 16 waves of a compute unit issue the same kind of
// access with a given lane -> byte address map (bank conflicts show as multiples of the contiguous case)
typedef __attribute__((__vector_size__(2 * sizeof(float)))) float f32x2;
enum LdsOp { kRead128, kRead64, kReadU16, kWrite32, kWrite64 };
template <int OP> __global__ void lds_pattern_kernel(float* out, const int* addr_of_lane) {
  extern __shared__ float lds[];
  for (int i = threadIdx.x; i < 16384; i += blockDim.x) lds[i] = 0.f;
  __syncthreads();
  const int addr = addr_of_lane[threadIdx.x & 63];
  float acc = 0.f;
  for (int it = 0; it < ITER / 2; ++it) {
    if (OP == kRead128) {
      f32x4 r0, r1, r2, r3;
      asm volatile("ds_read_b128 %0, %4\n ds_read_b128 %1, %4 offset:16384\n ds_read_b128 %2, %4 offset:32768\n ds_read_b128 %3, %4 offset:49152\n s_waitcnt lgkmcnt(0)"
                   : "=v"(r0), "=v"(r1), "=v"(r2), "=v"(r3) : "v"(addr));
      acc += r0[0] + r1[1] + r2[2] + r3[3];
    } else if (OP == kRead64) {
      f32x2 r0, r1, r2, r3;
      asm volatile("ds_read_b64 %0, %4\n ds_read_b64 %1, %4 offset:16384\n ds_read_b64 %2, %4 offset:32768\n ds_read_b64 %3, %4 offset:49152\n s_waitcnt lgkmcnt(0)"
                   : "=v"(r0), "=v"(r1), "=v"(r2), "=v"(r3) : "v"(addr));
      acc += r0[0] + r1[1] + r2[0] + r3[1];
    } else if (OP == kReadU16) {
      float r0, r1, r2, r3;
      asm volatile("ds_read_u16 %0, %4\n ds_read_u16 %1, %4 offset:16384\n ds_read_u16 %2, %4 offset:32768\n ds_read_u16 %3, %4 offset:49152\n s_waitcnt lgkmcnt(0)"
                   : "=v"(r0), "=v"(r1), "=v"(r2), "=v"(r3) : "v"(addr));
      acc += r0 + r1 + r2 + r3;
    } else if (OP == kWrite32) {
      asm volatile("ds_write_b32 %0, %1\n ds_write_b32 %0, %1 offset:16384\n ds_write_b32 %0, %1 offset:32768\n ds_write_b32 %0, %1 offset:49152\n s_waitcnt lgkmcnt(0)"
                   :: "v"(addr), "v"(acc));
    } else {
      f32x2 v = {acc, acc};
      asm volatile("ds_write_b64 %0, %1\n ds_write_b64 %0, %1 offset:16384\n ds_write_b64 %0, %1 offset:32768\n ds_write_b64 %0, %1 offset:49152\n s_waitcnt lgkmcnt(0)"
                   :: "v"(addr), "v"(v));
    }
  }
  out[blockIdx.x * blockDim.x + threadIdx.x] = acc;
}
template <int OP> void run_lds(const char* name, int (*addr)(int), float* out, int* table) {
  int h[64];
  for (int l = 0; l < 64; ++l) h[l] = addr(l);
  HIP_OK(hipMemcpy(table, h, sizeof(h), hipMemcpyHostToDevice));
  HIP_OK(hipFuncSetAttribute((const void*)lds_pattern_kernel<OP>, hipFuncAttributeMaxDynamicSharedMemorySize, 66 * 1024));
  hipEvent_t e0, e1; HIP_OK(hipEventCreate(&e0)); HIP_OK(hipEventCreate(&e1));
  lds_pattern_kernel<OP><<<256, 1024, 66 * 1024>>>(out, table);
  HIP_OK(hipEventRecord(e0));
  lds_pattern_kernel<OP><<<256, 1024, 66 * 1024>>>(out, table);
  HIP_OK(hipEventRecord(e1)); HIP_OK(hipEventSynchronize(e1));
  float ms; HIP_OK(hipEventElapsedTime(&ms, e0, e1));
  printf("%-78s %6.2f LDS cycles per wave instruction\n", name, ms * 1e-3 * g_ghz * 1e9 / ((double)(ITER / 2) * 4 * 16));
  fflush(stdout);
}
#define LDS_ROWS(OP, S, PIECE) \
  run_lds<OP>(#OP " rows " #S " bytes apart: (lane & 15) * " #S " + (lane >> 4) * " #PIECE, [](int l) { return (l & 15) * S + (l >> 4) * PIECE; }, out, table)
static void lds_patterns(float* out) {
  int* table;
  HIP_OK(hipMalloc(&table, 64 * sizeof(int)));
  printf("LDS access patterns, 16 waves per compute unit\n");
  run_lds<kRead128>("kRead128 contiguous: lane * 16", [](int l) { return l * 16; }, out, table);
  LDS_ROWS(kRead128, 96, 16); LDS_ROWS(kRead128, 144, 16); LDS_ROWS(kRead128, 160, 16); LDS_ROWS(kRead128, 176, 16);
  LDS_ROWS(kRead128, 224, 16); LDS_ROWS(kRead128, 272, 16); LDS_ROWS(kRead128, 288, 16); LDS_ROWS(kRead128, 544, 16);
  run_lds<kRead64>("kRead64 contiguous: lane * 8", [](int l) { return l * 8; }, out, table);
  LDS_ROWS(kRead64, 136, 8); LDS_ROWS(kRead64, 144, 8); LDS_ROWS(kRead64, 160, 8); LDS_ROWS(kRead64, 176, 8);
  run_lds<kReadU16>("kReadU16 contiguous: lane * 2", [](int l) { return l * 2; }, out, table);
  run_lds<kReadU16>("kReadU16 columns of rows 144 bytes apart, lane groups 8 rows apart", [](int l) { return 8 * (l >> 4) * 144 + (l & 15) * 2; }, out, table);
  run_lds<kReadU16>("kReadU16 the same with the 32-byte groups of a row exchanged per lane group", [](int l) { return 8 * (l >> 4) * 144 + (((l & 15) ^ ((l >> 4) << 4)) * 2); }, out, table);
  run_lds<kWrite32>("kWrite32 contiguous: lane * 4", [](int l) { return l * 4; }, out, table);
  run_lds<kWrite32>("kWrite32 transposing: column 8 (lane & 7), word lane >> 3, columns 144 bytes apart", [](int l) { return 8 * (l & 7) * 144 + (l >> 3) * 4; }, out, table);
  run_lds<kWrite32>("kWrite32 transposing: column 8 (lane & 7), word lane >> 3, columns 136 bytes apart", [](int l) { return 8 * (l & 7) * 136 + (l >> 3) * 4; }, out, table);
  run_lds<kWrite32>("kWrite32 transposing: column 8 (lane & 7), word lane >> 3, columns 140 bytes apart", [](int l) { return 8 * (l & 7) * 140 + (l >> 3) * 4; }, out, table);
  run_lds<kWrite64>("kWrite64 contiguous: lane * 8", [](int l) { return l * 8; }, out, table);
  LDS_ROWS(kWrite64, 136, 8); LDS_ROWS(kWrite64, 144, 8); LDS_ROWS(kWrite64, 160, 8);
  HIP_OK(hipFree(table));
}

int main() {
  int khz = 0;
  HIP_OK(hipDeviceGetAttribute(&khz, hipDeviceAttributeClockRate, 0));
  if (khz > 0) g_ghz = khz * 1e-6;
  printf("device clock %.3f GHz (reported); 256 workgroups, one per compute unit\n", g_ghz);
  float* out; long long* cyc;
  HIP_OK(hipMalloc(&out, 256 * 1024 * 4)); HIP_OK(hipMalloc(&cyc, 8));
  for (int wps = 1; wps <= 4; wps *= 2) {
    run<0>("fma dependent", wps, 64, out, cyc);
    run<1>("fma 4 chains", wps, 64, out, cyc);
    run<2>("mfma dependent", wps, 16, out, cyc);
    run<3>("mfma 4 indep", wps, 16, out, cyc);
    run<4>("1 mfma + 3 fma (per 4)", wps, 64, out, cyc);
    run<9>("1 mfma + 7 fma (per 8)", wps, 128, out, cyc);
    run<5>("rcp dependent", wps, 64, out, cyc);
    run<6>("rcp 4 chains", wps, 64, out, cyc);
    run<10>("exp 4 chains", wps, 64, out, cyc);
    run<7>("cvt_pk_bf16 indep", wps, 64, out, cyc);
    run<8>("ds_bpermute dep", wps, 16, out, cyc);
    run<13>("ds_read_b32 dep", wps, 16, out, cyc);
    run<11>("add dpp row_ror dep", wps, 64, out, cyc);
    run<12>("permlane32_swap dep", wps, 64, out, cyc);
    run<14>("even:mfma odd:fma waves", wps, 40, out, cyc);
    run<15>("mul 4 chains", wps, 64, out, cyc);
    run<16>("add 4 chains", wps, 64, out, cyc);
    run<17>("fmac 4 chains", wps, 64, out, cyc);
    run<18>("and/or/shl/perm", wps, 64, out, cyc);
    run<19>("cndmask/max/mov/mov", wps, 64, out, cyc);
    run<20>("fma 8 chains", wps, 128, out, cyc);
    run<21>("ds_read_b128 x4 + wait", wps, 16, out, cyc);
    run<22>("v_pk_mul_f16 4 chains", wps, 64, out, cyc);
    run<23>("mfma f16 4 indep", wps, 16, out, cyc);
    run<24>("cvt_pkrtz_f16_f32", wps, 64, out, cyc);
    run<25>("mfma 16x16x16 bf16 4 indep", wps, 16, out, cyc);
    run<29>("mfma 32x32x16 bf16 2 indep", wps, 32, out, cyc);
    run<26>("v_dot2_f32_bf16 4 chains", wps, 64, out, cyc);
    run<28>("4 mfma back to back + 28 fma", wps, 128, out, cyc);
    run<30>("1 mfma + 7 mixed valu (per 8)", wps, 128, out, cyc);
    run<31>("7 mixed valu alone (per 7)", wps, 112, out, cyc);
    run<32>("mfma bf16, f16 in turn, 4 indep", wps, 16, out, cyc);
    if (wps >= 2) run<33>("half the waves mfma bf16, half f16", wps, 16, out, cyc);
    run<34>("4 v_pk_mul_f16 + 1 mfma f16 (per 5)", wps, 20, out, cyc);
    if (wps == 4) {
      run<40>("1 wave mfma only, 3 waves rcp only", wps, 52, out, cyc);
      run<41>("1 wave mfma only, 3 waves cvt_pk only", wps, 52, out, cyc);
      run<42>("1 wave mfma only, 3 waves pk_mul_f16 only", wps, 52, out, cyc);
      run<43>("1 wave mfma only, 3 waves and/shl only", wps, 52, out, cyc);
      run<44>("1 wave mfma only, 3 waves permlane32_swap", wps, 52, out, cyc);
    }
    if (wps == 4) run<27>("1 wave mfma only, 3 waves fma only", wps, 52, out, cyc);
  }
  lds_patterns(out);
  return 0;
}
