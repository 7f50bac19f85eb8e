// Shared device helpers for the gfx950 kernels: element types, conversions,
// wavefront (64 lanes) and workgroup reductions, and the host-side error slot.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

#define RA_WAVE 64

// element-type tags of the C interface
enum { RA_F32 = 0, RA_BF16 = 1 };

// XCDs of the chip: workgroups are dealt round them in the order of their numbers, each XCD has an L2 of its own
#define RA_XCDS 8

typedef __bf16 bf16_t;
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4_t __attribute__((ext_vector_type(4)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));

__device__ __forceinline__ float to_f32(float v) { return v; }
__device__ __forceinline__ float to_f32(bf16_t v) { return (float)v; }

template <typename T> __device__ __forceinline__ T from_f32(float v);
template <> __device__ __forceinline__ float from_f32<float>(float v) { return v; }
// round to nearest even; the hardware conversion of gfx950
template <> __device__ __forceinline__ bf16_t from_f32<bf16_t>(float v) { return (bf16_t)v; }

// Eight consecutive elements as floats through 16-byte accesses; `p` is 16-byte aligned.
template <typename T> struct Vec8;
template <> struct Vec8<float> {
  static __device__ __forceinline__ void load(const float* p, float (&v)[8]) {
    const f32x4_t a = *(const f32x4_t*)p, b = *(const f32x4_t*)(p + 4);
#pragma unroll
    for (int i = 0; i < 4; ++i) { v[i] = a[i]; v[4 + i] = b[i]; }
  }
  static __device__ __forceinline__ void store(float* p, const float (&v)[8]) {
    *(f32x4_t*)p = (f32x4_t){v[0], v[1], v[2], v[3]};
    *(f32x4_t*)(p + 4) = (f32x4_t){v[4], v[5], v[6], v[7]};
  }
};
template <> struct Vec8<bf16_t> {
  static __device__ __forceinline__ void load(const bf16_t* p, float (&v)[8]) {
    const bf16x8_t a = *(const bf16x8_t*)p;
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = (float)a[i];
  }
  static __device__ __forceinline__ void store(bf16_t* p, const float (&v)[8]) {
    bf16x8_t a;
#pragma unroll
    for (int i = 0; i < 8; ++i) a[i] = (bf16_t)v[i];
    *(bf16x8_t*)p = a;
  }
};
// whether rows of `ld` elements of `bytes` each that start at `p` can be read in 16-byte pieces
static inline bool ra_rows_16b(const void* p, long ld, int bytes) {
  return p == nullptr || (((uintptr_t)p % 16) == 0 && (ld * bytes) % 16 == 0);
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int m = RA_WAVE / 2; m > 0; m >>= 1) v += __shfl_xor(v, m, RA_WAVE);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int m = RA_WAVE / 2; m > 0; m >>= 1) v = fmaxf(v, __shfl_xor(v, m, RA_WAVE));
  return v;
}

// Sum over a workgroup of up to 1024 threads; every thread gets the result.
// `red` is LDS for 17 floats. All threads of the workgroup must call it.
__device__ __forceinline__ float block_sum(float v, float* red) {
  const int lane = threadIdx.x & (RA_WAVE - 1);
  const int wave = threadIdx.x / RA_WAVE;
  const int nwave = (blockDim.x + RA_WAVE - 1) / RA_WAVE;
  v = wave_sum(v);
  __syncthreads();               // red may still be read from an earlier call
  if (lane == 0) red[wave] = v;
  __syncthreads();
  float t = 0.f;
  for (int i = 0; i < nwave; ++i) t += red[i];   // fixed order: deterministic
  return t;
}

// ---- what attention does to a score between the scaled product and the softmax -------------------------------
// softcap > 0: s <- softcap * tanh(s / softcap); r1, r2 (float, one entry a query head; both or neither):
// s <- s - r1[h] * ln(1 + r2[h] * (query position - key position)). The cap comes first.
struct RaScoreMod {
  float softcap;
  const float* r1;
  const float* r2;
};
__device__ __forceinline__ float ra_mod_score(float s, float softcap, bool biased, float r1, float r2, int dist) {
  if (softcap > 0.f) s = softcap * tanhf(s / softcap);
  if (biased) s -= r1 * logf(1.f + r2 * (float)dist);
  return s;
}
// The same through the hardware's exponential, logarithm and reciprocal (an ulp or two each), for the kernels whose
// operands are bfloat16: tanh(x) = 1 - 2 / (1 + e^(2x)), the argument bounded so that e^(2x) stays finite.
__device__ __forceinline__ float ra_mod_score_fast(float s, float softcap, float inv_softcap, bool biased, float r1,
                                                   float r2, int dist) {
  if (softcap > 0.f) {
    const float x = fminf(fmaxf(s * inv_softcap, -15.f), 15.f);
    s = softcap * (1.f - __fdividef(2.f, 1.f + __expf(2.f * x)));
  }
  if (biased) s -= r1 * 0.6931471805599453f * __log2f(fmaf(r2, (float)dist, 1.f));
  return s;
}

// ---- cache layout -----------------------------------------------------------
// A block of the cache holds block_size (a multiple of 16) slots of one KV head
// as block_size/16 tiles of 16 slots x d elements, 16*d elements each, laid out
// in the order the MFMA operands want them, so that a wave's load of a tile is
// one contiguous run and LDS copies of it have no bank conflicts:
//   K tile: [d/8][16 slots][8]      element (slot, e) at ((e/8)*16 + slot)*8 + e%8
//   V tile: [d/16][4][16][4]        element (slot, e) at (((e/16)*4 + slot/4)*16 + e%16)*4 + slot%4
// `off` is the slot inside the block; d is a multiple of 16.
__host__ __device__ __forceinline__ size_t cache_k_index(int off, int e, int d) {
  return (size_t)(off >> 4) * 16 * d + (size_t)(((e >> 3) * 16 + (off & 15)) * 8 + (e & 7));
}
__host__ __device__ __forceinline__ size_t cache_v_index(int off, int e, int d) {
  const int s = off & 15;
  return (size_t)(off >> 4) * 16 * d + (size_t)((((e >> 4) * 4 + (s >> 2)) * 16 + (e & 15)) * 4 + (s & 3));
}

// ---- host side -------------------------------------------------------------
// One message slot per thread; ra_last_error() hands it to the caller.
extern thread_local char ra_error_text[512];
int ra_fail(const char* fmt, ...);

// Compute units of the current device (cached per device; 256 if the device cannot be asked).
int ra_cu_count(void);

#define RA_CHECK(cond, ...)                    \
  do {                                         \
    if (!(cond)) return ra_fail(__VA_ARGS__);  \
  } while (0)

#define RA_LAUNCH_CHECK(name)                                                   \
  do {                                                                          \
    hipError_t e_ = hipGetLastError();                                          \
    if (e_ != hipSuccess) return ra_fail("%s: launch failed: %s", name, hipGetErrorString(e_)); \
  } while (0)
