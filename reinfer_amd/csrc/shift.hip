// Row kernels around a mixer that reads its neighbours in time and whose result enters the stream through a
// gate: the token shift (mixes of a row with the row of the token before it, the last row of a portion kept in
// the request's state), the gated add into the float residual stream, an RMSNorm over rows of activations
// (strided, for a latent inside a wider projection), and tanh in place. Sums, mixes, sigmoids and the residual
// are float whatever the activations' type.
#include "common.h"
#include "reinfer_hip.h"

namespace {

// ---------------------------------------------------------------------------
// out[t, j * width + e] = h[t, e] + (prev(t)[e] - h[t, e]) * mu[j, e],  j < n_mix
// prev(t) = h[t - 1] inside a portion; for a portion's first row the row kept at keep_off in the request's state
// slot (zeros at a request's start). One workgroup a token. With `keep` set (a step of single tokens only: the
// workgroup that reads the kept row is the one that replaces it) the row is stored behind the read.
// ---------------------------------------------------------------------------
template <typename TA, typename TM>
__global__ void token_shift_kernel(const TA* __restrict__ h, int ldh, const TM* __restrict__ mu, int n_mix,
                                   float* __restrict__ state, long slot_stride, long keep_off,
                                   const int* __restrict__ seq_of_token, const int* __restrict__ cu_tokens,
                                   const int* __restrict__ state_slots, const int* __restrict__ fresh,
                                   TA* __restrict__ out, int ldo, int width, int keep) {
  const int t = blockIdx.x;
  const int seq = seq_of_token[t];
  const int first = cu_tokens[seq];
  const int slot = state_slots[seq];
  const TA* row = h + (size_t)t * ldh;
  const bool from_state = t == first;
  const bool zero = from_state && (slot < 0 || fresh[seq] != 0);
  float* kept = slot >= 0 ? state + (size_t)slot * slot_stride + keep_off : nullptr;
  const TA* before = row - ldh;
  for (int e = threadIdx.x; e < width; e += blockDim.x) {
    const float x = to_f32(row[e]);
    const float p = zero ? 0.f : from_state ? kept[e] : to_f32(before[e]);
    const float d = p - x;
    for (int j = 0; j < n_mix; ++j)
      out[(size_t)t * ldo + (size_t)j * width + e] = from_f32<TA>(x + d * to_f32(mu[(size_t)j * width + e]));
    if (keep && kept) kept[e] = x;            // this thread alone reads and writes element e of the kept row
  }
}

// The same, eight elements a thread through 16-byte accesses, a row split over blockIdx.y: a decode step has a
// handful of rows, and one workgroup walking a whole row is a chain of memory round trips.
template <typename TA, typename TM>
__global__ void token_shift_vec_kernel(const TA* __restrict__ h, int ldh, const TM* __restrict__ mu, int n_mix,
                                       float* __restrict__ state, long slot_stride, long keep_off,
                                       const int* __restrict__ seq_of_token, const int* __restrict__ cu_tokens,
                                       const int* __restrict__ state_slots, const int* __restrict__ fresh,
                                       TA* __restrict__ out, int ldo, int width, int keep) {
  const int t = blockIdx.x;
  const int e = (blockIdx.y * blockDim.x + threadIdx.x) * 8;
  if (e >= width) return;
  const int seq = seq_of_token[t];
  const int slot = state_slots[seq];
  const bool from_state = t == cu_tokens[seq];
  const bool zero = from_state && (slot < 0 || fresh[seq] != 0);
  float* kept = slot >= 0 ? state + (size_t)slot * slot_stride + keep_off : nullptr;
  const TA* row = h + (size_t)t * ldh;
  float x[8], d[8], m[8], o[8];
  Vec8<TA>::load(row + e, x);
  if (zero) {
#pragma unroll
    for (int i = 0; i < 8; ++i) d[i] = 0.f;
  } else if (from_state) {
    Vec8<float>::load(kept + e, d);
  } else {
    Vec8<TA>::load(row - ldh + e, d);
  }
#pragma unroll
  for (int i = 0; i < 8; ++i) d[i] -= x[i];
  for (int j = 0; j < n_mix; ++j) {
    Vec8<TM>::load(mu + (size_t)j * width + e, m);
#pragma unroll
    for (int i = 0; i < 8; ++i) o[i] = x[i] + d[i] * m[i];
    Vec8<TA>::store(out + (size_t)t * ldo + (size_t)j * width + e, o);
  }
  if (keep && kept) Vec8<float>::store(kept + e, x);   // this thread alone reads and writes these eight of the kept row
}

// The kept row moves on: a request's state takes the last row of its portion. Runs behind token_shift_kernel in
// stream order, after every read of the old row.
template <typename TA>
__global__ void token_shift_keep_kernel(const TA* __restrict__ h, int ldh, float* __restrict__ state, long slot_stride,
                                        long keep_off, const int* __restrict__ cu_tokens,
                                        const int* __restrict__ state_slots, int width) {
  const int seq = blockIdx.x;
  const int slot = state_slots[seq];
  const int first = cu_tokens[seq], last = cu_tokens[seq + 1];
  if (slot < 0 || last <= first) return;
  const TA* row = h + (size_t)(last - 1) * ldh;
  float* kept = state + (size_t)slot * slot_stride + keep_off;
  for (int e = blockIdx.y * blockDim.x + threadIdx.x; e < width; e += gridDim.y * blockDim.x) kept[e] = to_f32(row[e]);
}

// ---------------------------------------------------------------------------
// resid[t, e] += sigmoid(g[t, e]) * a[t, e] + sigmoid(g[t, width + e]) * b[t, e]      (b optional)
// g holds the gates' pre-activations side by side, rows ldg apart; a and b are contiguous [T, width].
// ---------------------------------------------------------------------------
template <typename TG, typename TA, typename TB>
__global__ void gated_stream_add_kernel(float* __restrict__ resid, const TG* __restrict__ g, int ldg,
                                        const TA* __restrict__ a, const TB* __restrict__ b, int width) {
  const size_t t = blockIdx.x;
  for (int e = threadIdx.x; e < width; e += blockDim.x) {
    float v = resid[t * width + e];
    const float ga = to_f32(g[t * ldg + e]);
    v += to_f32(a[t * width + e]) / (1.f + expf(-ga));
    if (b) {
      const float gb = to_f32(g[t * ldg + width + e]);
      v += to_f32(b[t * width + e]) / (1.f + expf(-gb));
    }
    resid[t * width + e] = v;
  }
}

template <typename TG, typename TA, typename TB>
__global__ void gated_stream_add_vec_kernel(float* __restrict__ resid, const TG* __restrict__ g, int ldg,
                                            const TA* __restrict__ a, const TB* __restrict__ b, int width) {
  const size_t t = blockIdx.x;
  const int e = (blockIdx.y * blockDim.x + threadIdx.x) * 8;
  if (e >= width) return;
  float v[8], gv[8], av[8];
  Vec8<float>::load(resid + t * width + e, v);
  Vec8<TG>::load(g + t * ldg + e, gv);
  Vec8<TA>::load(a + t * width + e, av);
#pragma unroll
  for (int i = 0; i < 8; ++i) v[i] += av[i] / (1.f + expf(-gv[i]));
  if (b) {
    Vec8<TG>::load(g + t * ldg + width + e, gv);
    Vec8<TB>::load(b + t * width + e, av);
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] += av[i] / (1.f + expf(-gv[i]));
  }
  Vec8<float>::store(resid + t * width + e, v);
}

// ---------------------------------------------------------------------------
// out[r, :] = x[r, :] * rsqrt(mean(x[r, :]^2) + eps) * w   over rows of activations, ldx / ldo apart.
// One wave a row.
// ---------------------------------------------------------------------------
template <typename TA, typename TW>
__global__ void rows_rmsnorm_kernel(const TA* __restrict__ x, int ldx, const TW* __restrict__ w, TA* __restrict__ out,
                                    int ldo, int n_rows, int width, float eps) {
  const int lane = threadIdx.x & (RA_WAVE - 1);
  const int r = blockIdx.x * (blockDim.x / RA_WAVE) + threadIdx.x / RA_WAVE;
  if (r >= n_rows) return;
  const TA* row = x + (size_t)r * ldx;
  float ss = 0.f;
  for (int e = lane; e < width; e += RA_WAVE) {
    const float v = to_f32(row[e]);
    ss += v * v;
  }
  ss = wave_sum(ss);
  const float rstd = 1.f / sqrtf(ss / (float)width + eps);
  TA* o = out + (size_t)r * ldo;
  for (int e = lane; e < width; e += RA_WAVE) o[e] = from_f32<TA>(to_f32(row[e]) * rstd * to_f32(w[e]));
}

// The same through 16-byte accesses, the row kept in registers (at most ROWS_CH * 512 wide).
#define ROWS_CH 4
template <typename TA, typename TW>
__global__ void rows_rmsnorm_vec_kernel(const TA* __restrict__ x, int ldx, const TW* __restrict__ w, TA* __restrict__ out,
                                        int ldo, int n_rows, int width, float eps) {
  const int lane = threadIdx.x & (RA_WAVE - 1);
  const int r = blockIdx.x * (blockDim.x / RA_WAVE) + threadIdx.x / RA_WAVE;
  if (r >= n_rows) return;
  const TA* row = x + (size_t)r * ldx;
  float v[ROWS_CH][8];
  float ss = 0.f;
#pragma unroll
  for (int c = 0; c < ROWS_CH; ++c) {
    const int e = (c * RA_WAVE + lane) * 8;
    if (e < width) {
      Vec8<TA>::load(row + e, v[c]);
#pragma unroll
      for (int i = 0; i < 8; ++i) ss += v[c][i] * v[c][i];
    }
  }
  ss = wave_sum(ss);
  const float rstd = 1.f / sqrtf(ss / (float)width + eps);
  TA* o = out + (size_t)r * ldo;
#pragma unroll
  for (int c = 0; c < ROWS_CH; ++c) {
    const int e = (c * RA_WAVE + lane) * 8;
    if (e < width) {
      float wv[8];
      Vec8<TW>::load(w + e, wv);
#pragma unroll
      for (int i = 0; i < 8; ++i) v[c][i] = v[c][i] * rstd * wv[i];
      Vec8<TA>::store(o + e, v[c]);
    }
  }
}

template <typename TA>
__global__ void tanh_rows_kernel(TA* __restrict__ x, long n) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) x[i] = from_f32<TA>(tanhf(to_f32(x[i])));
}

}  // namespace

extern "C" int ra_token_shift(const void* h, int ldh, const void* mu, int mu_dtype, int n_mix, float* state,
                              long slot_stride, long keep_off, const int* seq_of_token, const int* cu_tokens,
                              const int* state_slots, const int* fresh, void* out, int ldo, int act_dtype,
                              int n_seqs, int n_tokens, int width, int single_tokens, hipStream_t stream) {
  RA_CHECK(n_tokens > 0 && n_seqs > 0 && width > 0 && n_mix >= 1, "token_shift: %d tokens of %d requests, width %d, %d mixes",
           n_tokens, n_seqs, width, n_mix);
  RA_CHECK(ldh >= width && ldo >= n_mix * width, "token_shift: rows of %d / %d for width %d and %d mixes", ldh, ldo,
           width, n_mix);
  RA_CHECK(slot_stride >= keep_off + width && keep_off >= 0, "token_shift: a state slot of %ld floats, the kept row at %ld",
           slot_stride, keep_off);
  RA_CHECK(n_seqs <= 65535, "token_shift: %d requests in one launch", n_seqs);
  const int threads = width >= 1024 ? 256 : width >= 256 ? 128 : 64;
  const int ab = act_dtype == RA_F32 ? 4 : 2, mb = mu_dtype == RA_F32 ? 4 : 2;
  const bool vec = width % 8 == 0 && ra_rows_16b(h, ldh, ab) && ra_rows_16b(out, ldo, ab) && ra_rows_16b(mu, width, mb) &&
                   ra_rows_16b(state, slot_stride, 4) && keep_off % 4 == 0;
  const int vthreads = width >= 2048 ? 128 : 64;
  const dim3 vgrid(n_tokens, (width / 8 + vthreads - 1) / vthreads);
  const dim3 kgrid(n_seqs, (width + 4 * threads - 1) / (4 * threads));
#define RA_TS(TA, TM)                                                                                                \
  do {                                                                                                               \
    if (vec)                                                                                                         \
      token_shift_vec_kernel<TA, TM><<<vgrid, vthreads, 0, stream>>>(                                                \
          (const TA*)h, ldh, (const TM*)mu, n_mix, state, slot_stride, keep_off, seq_of_token, cu_tokens,            \
          state_slots, fresh, (TA*)out, ldo, width, single_tokens ? 1 : 0);                                          \
    else                                                                                                             \
      token_shift_kernel<TA, TM><<<n_tokens, threads, 0, stream>>>(                                                  \
          (const TA*)h, ldh, (const TM*)mu, n_mix, state, slot_stride, keep_off, seq_of_token, cu_tokens,            \
          state_slots, fresh, (TA*)out, ldo, width, single_tokens ? 1 : 0);                                          \
    if (!single_tokens)                                                                                              \
      token_shift_keep_kernel<TA><<<kgrid, threads, 0, stream>>>((const TA*)h, ldh, state, slot_stride, keep_off,    \
                                                                 cu_tokens, state_slots, width);                     \
  } while (0)
  if (act_dtype == RA_F32 && mu_dtype == RA_F32) RA_TS(float, float);
  else if (act_dtype == RA_BF16 && mu_dtype == RA_BF16) RA_TS(bf16_t, bf16_t);
  else if (act_dtype == RA_BF16 && mu_dtype == RA_F32) RA_TS(bf16_t, float);
  else return ra_fail("token_shift: unsupported dtypes (activations %d, factors %d)", act_dtype, mu_dtype);
#undef RA_TS
  RA_LAUNCH_CHECK("token_shift");
  return 0;
}

extern "C" int ra_gated_stream_add(float* resid, const void* gates, int ldg, int gate_dtype, const void* a, int a_dtype,
                                   const void* b, int b_dtype, int n_tokens, int width, hipStream_t stream) {
  RA_CHECK(n_tokens > 0 && width > 0 && a != nullptr, "gated_stream_add: %d tokens, width %d", n_tokens, width);
  RA_CHECK(ldg >= (b ? 2 : 1) * width, "gated_stream_add: gate rows of %d for width %d", ldg, width);
  const int threads = width >= 1024 ? 256 : width >= 256 ? 128 : 64;
  const int bd = b ? b_dtype : a_dtype;
  const bool vec = width % 8 == 0 && ra_rows_16b(resid, width, 4) && ra_rows_16b(gates, ldg, gate_dtype == RA_F32 ? 4 : 2) &&
                   ra_rows_16b(a, width, a_dtype == RA_F32 ? 4 : 2) && ra_rows_16b(b, width, bd == RA_F32 ? 4 : 2);
  const int vthreads = width >= 2048 ? 128 : 64;
  const dim3 vgrid(n_tokens, (width / 8 + vthreads - 1) / vthreads);
#define RA_GA(TG, TA, TB)                                                                                            \
  do {                                                                                                               \
    if (vec)                                                                                                         \
      gated_stream_add_vec_kernel<TG, TA, TB><<<vgrid, vthreads, 0, stream>>>(resid, (const TG*)gates, ldg,          \
                                                                             (const TA*)a, (const TB*)b, width);     \
    else                                                                                                             \
      gated_stream_add_kernel<TG, TA, TB><<<n_tokens, threads, 0, stream>>>(resid, (const TG*)gates, ldg,            \
                                                                          (const TA*)a, (const TB*)b, width);        \
  } while (0)
  if (gate_dtype == RA_F32 && a_dtype == RA_F32 && bd == RA_F32) RA_GA(float, float, float);
  else if (gate_dtype == RA_BF16 && a_dtype == RA_BF16 && bd == RA_BF16) RA_GA(bf16_t, bf16_t, bf16_t);
  else if (gate_dtype == RA_BF16 && a_dtype == RA_BF16 && bd == RA_F32) RA_GA(bf16_t, bf16_t, float);
  else if (gate_dtype == RA_BF16 && a_dtype == RA_F32 && bd == RA_BF16) RA_GA(bf16_t, float, bf16_t);
  else if (gate_dtype == RA_BF16 && a_dtype == RA_F32 && bd == RA_F32) RA_GA(bf16_t, float, float);
  else return ra_fail("gated_stream_add: unsupported dtypes (gates %d, addends %d, %d)", gate_dtype, a_dtype, bd);
#undef RA_GA
  RA_LAUNCH_CHECK("gated_stream_add");
  return 0;
}

extern "C" int ra_rows_rmsnorm(const void* x, int ldx, const void* weight, int weight_dtype, void* out, int ldo,
                               int act_dtype, int n_rows, int width, float eps, hipStream_t stream) {
  RA_CHECK(n_rows > 0 && width > 0 && ldx >= width && ldo >= width, "rows_rmsnorm: %d rows of %d (strides %d, %d)",
           n_rows, width, ldx, ldo);
  const int ab = act_dtype == RA_F32 ? 4 : 2;
  const bool vec = width % 8 == 0 && width <= ROWS_CH * RA_WAVE * 8 && ra_rows_16b(x, ldx, ab) && ra_rows_16b(out, ldo, ab) &&
                   ra_rows_16b(weight, width, weight_dtype == RA_F32 ? 4 : 2);
  // few rows: a wave a workgroup, so that the rows spread over the compute units
  const int waves = n_rows <= 256 ? 1 : 4;
  const unsigned blocks = (unsigned)((n_rows + waves - 1) / waves);
#define RA_RN(TA, TW)                                                                                                \
  do {                                                                                                               \
    if (vec)                                                                                                         \
      rows_rmsnorm_vec_kernel<TA, TW><<<blocks, waves * RA_WAVE, 0, stream>>>((const TA*)x, ldx, (const TW*)weight,  \
                                                                              (TA*)out, ldo, n_rows, width, eps);    \
    else                                                                                                             \
      rows_rmsnorm_kernel<TA, TW><<<blocks, waves * RA_WAVE, 0, stream>>>((const TA*)x, ldx, (const TW*)weight,      \
                                                                          (TA*)out, ldo, n_rows, width, eps);        \
  } while (0)
  if (act_dtype == RA_F32 && weight_dtype == RA_F32) RA_RN(float, float);
  else if (act_dtype == RA_BF16 && weight_dtype == RA_BF16) RA_RN(bf16_t, bf16_t);
  else if (act_dtype == RA_BF16 && weight_dtype == RA_F32) RA_RN(bf16_t, float);
  else return ra_fail("rows_rmsnorm: unsupported dtypes (activations %d, weight %d)", act_dtype, weight_dtype);
#undef RA_RN
  RA_LAUNCH_CHECK("rows_rmsnorm");
  return 0;
}

extern "C" int ra_tanh_rows(void* x, int act_dtype, long n, hipStream_t stream) {
  RA_CHECK(n > 0, "tanh_rows: empty input");
  const unsigned blocks = (unsigned)((n + 255) / 256);
  if (act_dtype == RA_F32) tanh_rows_kernel<float><<<blocks, 256, 0, stream>>>((float*)x, n);
  else if (act_dtype == RA_BF16) tanh_rows_kernel<bf16_t><<<blocks, 256, 0, stream>>>((bf16_t*)x, n);
  else return ra_fail("tanh_rows: unknown dtype tag %d", act_dtype);
  RA_LAUNCH_CHECK("tanh_rows");
  return 0;
}
