// Attention over a low-rank latent: every token keeps one vector c (the RMS-normed down projection, `rank`
// wide) and one rotated key part (`R` wide) that all heads share. Keys and values of a head are linear in c,
// so a head's query is taken through its key matrix once (q' = W_uk,h^T q) and its output through its value
// matrix once (o = W_uv,h o'), and the attention itself runs over the cached rows [c | rotated part] as one
// shared KV head of size Dp = rank + R rounded up to the cache's tile of 16: the framework's paged kernels
// do that part. Here: the kernel that prepares queries and cache rows, and the per-head products.
// Sums of squares, the norm's factor, angles, sines and all accumulation are float.
#include "common.h"
#include "reinfer_hip.h"

// ---------------------------------------------------------------------------
// One workgroup a token. proj row = [... q heads (each D unrotated | R rotated) ... | c_raw (rank) | kr (R) ...]
//   c  = c_raw * rsqrt(mean(c_raw^2) + eps) * w
//   rotation of the first rot_dims of an R-wide part: pair (i, i + rot_dims/2) by angle pos * inv_freq[i]
//   cache row (K and V layout alike) = [c | rot(kr) | 0 ...]            at slots[t] (-1: store nothing)
//   q_lat[t, h, rank : Dp] = [rot(q_h rotated part) | 0 ...]            (columns below rank: head products)
// ---------------------------------------------------------------------------
template <typename TA>
__device__ __forceinline__ float latent_rot(const TA* vec, int i, int half, int rot_dims, const float* cs,
                                            const float* sn) {
  if (i < half) return to_f32(vec[i]) * cs[i] - to_f32(vec[i + half]) * sn[i];
  if (i < rot_dims) {
    const int j = i - half;
    return to_f32(vec[i]) * cs[j] + to_f32(vec[j]) * sn[j];
  }
  return to_f32(vec[i]);
}

template <typename TA, typename TW>
__global__ void latent_prep_kernel(const TA* __restrict__ proj, int ld, int q_off, int dkv_off,
                                   const TW* __restrict__ cw, float eps, const int* __restrict__ positions,
                                   const float* __restrict__ inv_freq, int rot_dims, int R, int rank, int H, int D,
                                   TA* __restrict__ q_lat, int Dp, const int* __restrict__ slots,
                                   TA* __restrict__ kcache, TA* __restrict__ vcache, int block_size) {
  extern __shared__ float sm[];          // cos [half], sin [half]
  __shared__ float red[17];
  const int t = blockIdx.x;
  const int half = rot_dims / 2;
  float* cs = sm;
  float* sn = sm + half;
  const TA* row = proj + (size_t)t * ld;
  const TA* craw = row + dkv_off;
  const TA* kr = craw + rank;
  const float pos = (float)positions[t];
  for (int j = threadIdx.x; j < half; j += blockDim.x) sincosf(pos * inv_freq[j], &sn[j], &cs[j]);
  float ss = 0.f;
  for (int i = threadIdx.x; i < rank; i += blockDim.x) {
    const float v = to_f32(craw[i]);
    ss += v * v;
  }
  const float total = block_sum(ss, red);          // its barriers also publish cs / sn
  const float rstd = rsqrtf(total / (float)rank + eps);
  const int slot = slots[t];
  if (slot >= 0) {
    const int blk = slot / block_size, off = slot % block_size;
    TA* kb = kcache + (size_t)blk * block_size * Dp;
    TA* vb = vcache + (size_t)blk * block_size * Dp;
    for (int e = threadIdx.x; e < Dp; e += blockDim.x) {
      float v = 0.f;
      if (e < rank) v = to_f32(craw[e]) * rstd * to_f32(cw[e]);
      else if (e < rank + R) v = latent_rot(kr, e - rank, half, rot_dims, cs, sn);
      const TA o = from_f32<TA>(v);
      kb[cache_k_index(off, e, Dp)] = o;
      vb[cache_v_index(off, e, Dp)] = o;
    }
  }
  const int tail = Dp - rank;
  TA* qo = q_lat + (size_t)t * H * Dp;
  for (int idx = threadIdx.x; idx < H * tail; idx += blockDim.x) {
    const int h = idx / tail, i = idx % tail;
    float v = 0.f;
    if (i < R) v = latent_rot(row + q_off + (size_t)h * (D + R) + D, i, half, rot_dims, cs, sn);
    qo[(size_t)h * Dp + rank + i] = from_f32<TA>(v);
  }
}

extern "C" int ra_latent_prep(const void* proj, int act_dtype, int ld, int q_off, int dkv_off, const void* c_weight,
                              int weight_dtype, float eps, const int* positions, const float* inv_freq,
                              int rot_dims, int R, int rank, int H, int D, void* q_lat, int Dp, const int* slots,
                              void* kcache, void* vcache, int block_size, int n_tokens, hipStream_t stream) {
  RA_CHECK(n_tokens > 0 && H > 0 && D >= 0 && R >= 0 && rank > 0, "latent_prep: %d tokens, %d heads of %d + %d, rank %d",
           n_tokens, H, D, R, rank);
  RA_CHECK(rot_dims >= 0 && rot_dims % 2 == 0 && rot_dims <= R, "latent_prep: %d rotated of %d", rot_dims, R);
  RA_CHECK(Dp % 16 == 0 && Dp >= rank + R && block_size > 0 && block_size % 16 == 0,
           "latent_prep: cache rows of %d for rank %d + %d, blocks of %d", Dp, rank, R, block_size);
  RA_CHECK(q_off >= 0 && dkv_off >= 0 && q_off + H * (D + R) <= ld && dkv_off + rank + R <= ld,
           "latent_prep: the row of %d does not hold queries at %d and the latent at %d", ld, q_off, dkv_off);
  const size_t lds = (size_t)(rot_dims > 0 ? rot_dims : 2) * sizeof(float);
#define RA_LP(TA, TW)                                                                                          \
  latent_prep_kernel<TA, TW><<<n_tokens, 256, lds, stream>>>(                                                  \
      (const TA*)proj, ld, q_off, dkv_off, (const TW*)c_weight, eps, positions, inv_freq, rot_dims, R, rank, H, D, \
      (TA*)q_lat, Dp, slots, (TA*)kcache, (TA*)vcache, block_size)
  if (act_dtype == RA_F32 && weight_dtype == RA_F32) RA_LP(float, float);
  else if (act_dtype == RA_BF16 && weight_dtype == RA_BF16) RA_LP(bf16_t, bf16_t);
  else if (act_dtype == RA_BF16 && weight_dtype == RA_F32) RA_LP(bf16_t, float);
  else return ra_fail("latent_prep: unsupported dtypes (activations %d, weight %d)", act_dtype, weight_dtype);
#undef RA_LP
  RA_LAUNCH_CHECK("latent_prep");
  return 0;
}

// ---------------------------------------------------------------------------
// Products head by head: out[t, h, n] = sum_k x[t, h, k] * W[h, n, k]   (W: [H, N, K], k contiguous)
// optionally times sigmoid(gate[t, h * N + n]). x, out and gate are rows with strides of their own, a head
// of x at h * x_head, of out at h * o_head.
//
// bfloat16 with K, the row strides and the head offsets of x in steps of 8 elements: matrix cores. A wave
// owns 16 output columns of one head for MT tiles of 16 tokens and walks K in steps of 32; both operands come
// straight from memory in operand layout (lane (r, g): row r, elements 8g .. 8g + 7 of the step, one 16-byte
// load), the weights of a head being small enough to stay in the caches while the token tiles pass. The four
// waves of a workgroup take four column tiles. Lane (r, g) ends with out[token r][column 4g .. 4g + 3].
// Anything else (float, odd sizes): a plain kernel, 16 tokens of one head a workgroup, x in LDS as float.
// ---------------------------------------------------------------------------
template <int MT>
__global__ void __launch_bounds__(256)
head_linear_mfma_kernel(const bf16_t* __restrict__ x, int ldx, int x_head, const bf16_t* __restrict__ W,
                        bf16_t* __restrict__ out, int ldo, int o_head, const bf16_t* __restrict__ gate, int ldg,
                        int gate_per_head, int T, int N, int K) {
  const int lane = threadIdx.x & (RA_WAVE - 1);
  const int wave = threadIdx.x / RA_WAVE;
  const int r = lane & 15, g = lane >> 4;
  const int h = blockIdx.z;
  const int n0 = (blockIdx.x * 4 + wave) * 16;
  const int t0 = blockIdx.y * 16 * MT;
  if (n0 >= N) return;
  const bf16_t* wrow = W + ((size_t)h * N + (n0 + r < N ? n0 + r : 0)) * K;
  const bool w_ok = n0 + r < N;
  const bf16_t* xrow[MT];
  bool x_ok[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int t = t0 + mt * 16 + r;
    x_ok[mt] = t < T;
    xrow[mt] = x + (size_t)(x_ok[mt] ? t : 0) * ldx + (size_t)h * x_head;
  }
  f32x4_t acc[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) acc[mt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  const bf16x8_t zero = {0, 0, 0, 0, 0, 0, 0, 0};
  for (int k0 = 0; k0 < K; k0 += 32) {
    const int k = k0 + g * 8;
    const bool k_ok = k < K;                          // K is a multiple of 8: a chunk is whole or absent
    const bf16x8_t a = (w_ok && k_ok) ? *(const bf16x8_t*)(wrow + k) : zero;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const bf16x8_t b = (x_ok[mt] && k_ok) ? *(const bf16x8_t*)(xrow[mt] + k) : zero;
      acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc[mt], 0, 0, 0);
    }
  }
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int t = t0 + mt * 16 + r;
    if (t >= T) continue;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int n = n0 + 4 * g + i;
      if (n >= N) continue;
      float v = acc[mt][i];
      if (gate) {
        const float gv = to_f32(gate[(size_t)t * ldg + (gate_per_head ? (size_t)h : (size_t)h * N + n)]);
        v *= 1.f / (1.f + expf(-gv));
      }
      out[(size_t)t * ldo + (size_t)h * o_head + n] = from_f32<bf16_t>(v);
    }
  }
}

#define HL_TOKENS 16
template <typename TA>
__global__ void head_linear_kernel(const TA* __restrict__ x, int ldx, int x_head, const TA* __restrict__ W,
                                   TA* __restrict__ out, int ldo, int o_head, const TA* __restrict__ gate,
                                   int ldg, int gate_per_head, int T, int N, int K) {
  extern __shared__ float xs[];          // [K][HL_TOKENS]
  const int h = blockIdx.x;
  const int t0 = blockIdx.y * HL_TOKENS;
  const int nt = (T - t0 < HL_TOKENS) ? T - t0 : HL_TOKENS;
  for (int idx = threadIdx.x; idx < K * HL_TOKENS; idx += blockDim.x) {
    const int tt = idx / K, k = idx % K;
    xs[k * HL_TOKENS + tt] = (tt < nt) ? to_f32(x[(size_t)(t0 + tt) * ldx + (size_t)h * x_head + k]) : 0.f;
  }
  __syncthreads();
  const TA* Wh = W + (size_t)h * K * N;
  for (int n = blockIdx.z * blockDim.x + threadIdx.x; n < N; n += gridDim.z * blockDim.x) {
    float acc[HL_TOKENS];
#pragma unroll
    for (int i = 0; i < HL_TOKENS; ++i) acc[i] = 0.f;
    const TA* wr = Wh + (size_t)n * K;
    for (int k = 0; k < K; ++k) {
      const float w = to_f32(wr[k]);
      const f32x4_t* xr = (const f32x4_t*)(xs + k * HL_TOKENS);
#pragma unroll
      for (int g = 0; g < HL_TOKENS / 4; ++g) {
        const f32x4_t v = xr[g];
        acc[4 * g + 0] += w * v[0];
        acc[4 * g + 1] += w * v[1];
        acc[4 * g + 2] += w * v[2];
        acc[4 * g + 3] += w * v[3];
      }
    }
#pragma unroll
    for (int i = 0; i < HL_TOKENS; ++i) {
      if (i < nt) {
        float v = acc[i];
        if (gate) {
          const float g = to_f32(gate[(size_t)(t0 + i) * ldg + (gate_per_head ? (size_t)h : (size_t)h * N + n)]);
          v *= 1.f / (1.f + expf(-g));
        }
        out[(size_t)(t0 + i) * ldo + (size_t)h * o_head + n] = from_f32<TA>(v);
      }
    }
  }
}

extern "C" int ra_head_linear(const void* x, int ldx, int x_head, const void* W, void* out, int ldo, int o_head,
                              const void* gate, int ldg, int gate_per_head, int act_dtype, int n_tokens, int H,
                              int N, int K, hipStream_t stream) {
  RA_CHECK(n_tokens > 0 && H > 0 && N > 0 && K > 0, "head_linear: %d tokens, %d heads, %d x %d", n_tokens, H, N, K);
  RA_CHECK(ldx >= (H - 1) * x_head + K && ldo >= (H - 1) * o_head + N && x_head >= 0 && o_head >= N,
           "head_linear: rows of %d / %d do not hold %d heads of %d / %d", ldx, ldo, H, K, N);
  RA_CHECK(gate == nullptr || ldg >= (gate_per_head ? H : H * N), "head_linear: gate rows of %d for %d heads of %d", ldg, H, N);
  RA_CHECK(H <= 65535, "head_linear: %d heads in one launch", H);
  if (act_dtype == RA_BF16 && K % 8 == 0 && ldx % 8 == 0 && x_head % 8 == 0 && ((uintptr_t)x % 16) == 0 &&
      ((uintptr_t)W % 16) == 0) {
    const int col_groups = (N + 63) / 64;
    if (n_tokens <= 16) {
      dim3 grid(col_groups, 1, H);
      head_linear_mfma_kernel<1><<<grid, 256, 0, stream>>>((const bf16_t*)x, ldx, x_head, (const bf16_t*)W,
                                                           (bf16_t*)out, ldo, o_head, (const bf16_t*)gate, ldg,
                                                           gate_per_head, n_tokens, N, K);
    } else {
      const int tiles = (n_tokens + 63) / 64;
      RA_CHECK(tiles <= 65535, "head_linear: %d tokens in one launch", n_tokens);
      dim3 grid(col_groups, tiles, H);
      head_linear_mfma_kernel<4><<<grid, 256, 0, stream>>>((const bf16_t*)x, ldx, x_head, (const bf16_t*)W,
                                                           (bf16_t*)out, ldo, o_head, (const bf16_t*)gate, ldg,
                                                           gate_per_head, n_tokens, N, K);
    }
    RA_LAUNCH_CHECK("head_linear");
    return 0;
  }
  const size_t lds = (size_t)K * HL_TOKENS * sizeof(float);
  RA_CHECK(lds <= 64 * 1024, "head_linear: K = %d is more than the 1024 a workgroup stages", K);
  const int tiles = (n_tokens + HL_TOKENS - 1) / HL_TOKENS;
  RA_CHECK(tiles <= 65535, "head_linear: %d tokens in one launch", n_tokens);
  const int threads = N >= 256 ? 256 : ((N + 63) / 64) * 64;
  // few tokens: the columns of a head are spread over several workgroups as well
  const int col_groups = tiles * H >= 256 ? 1 : (N + threads - 1) / threads;
  dim3 grid(H, tiles, col_groups);
  if (act_dtype == RA_F32)
    head_linear_kernel<float><<<grid, threads, lds, stream>>>((const float*)x, ldx, x_head, (const float*)W,
                                                              (float*)out, ldo, o_head, (const float*)gate, ldg,
                                                              gate_per_head, n_tokens, N, K);
  else if (act_dtype == RA_BF16)
    head_linear_kernel<bf16_t><<<grid, threads, lds, stream>>>((const bf16_t*)x, ldx, x_head, (const bf16_t*)W,
                                                               (bf16_t*)out, ldo, o_head, (const bf16_t*)gate, ldg,
                                                               gate_per_head, n_tokens, N, K);
  else
    return ra_fail("head_linear: unknown dtype tag %d", act_dtype);
  RA_LAUNCH_CHECK("head_linear");
  return 0;
}
