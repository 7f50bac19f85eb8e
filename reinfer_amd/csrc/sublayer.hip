// Row kernels of a layer whose sublayers read the residual stream itself and whose results enter it behind a norm,
// and of an attention whose queries and keys are normed over their whole projection and whose values turn with
// their position. Sums, norms, angles and the stream are float whatever the activations' type.
//
//   stream_cast     out[t, :] = TA(x[t, :])                            the stream as the products' operand
//   sum_norm_add    y = sum_i s_i x_i;  y <- y / rms(y) * w (optional);  x += y (optional);  copy = TA(x or y)
//   span_rmsnorm    a run of columns of every row, in place: v / sqrt(sum v^2 / count + eps) * w
//   turn_heads      every head's first `width` entries turned by sign * position (pairs (m, m + width / 2) or
//                   (2m, 2m + 1), angle position * inv_freq[m]), in place, optionally times sigmoid(gate)
#include "common.h"
#include "reinfer_hip.h"

namespace {

template <typename TA>
__global__ void stream_cast_kernel(const float* __restrict__ x, TA* __restrict__ out, size_t n) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (; i < n; i += stride) out[i] = from_f32<TA>(x[i]);
}

template <typename TA>
__global__ void stream_cast_vec_kernel(const float* __restrict__ x, TA* __restrict__ out, size_t n8) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (; i < n8; i += stride) {
    float v[8];
    Vec8<float>::load(x + i * 8, v);
    Vec8<TA>::store(out + i * 8, v);
  }
}

#define SNA_MAX 4
struct SumInputs {
  const void* x[SNA_MAX];
  float s[SNA_MAX];
};

// One workgroup a row. The row's sum is kept in LDS as floats between the two passes (rows up to SNA_LDS wide),
// or formed again from the inputs.
#define SNA_LDS 8192
template <typename TX, typename TO, int N>
__global__ void sum_norm_add_kernel(SumInputs in, const float* __restrict__ weight, int weight_stride, int normed,
                                    float eps, int h, float* __restrict__ resid, TO* __restrict__ copy) {
  __shared__ float red[17];
  __shared__ float row_y[SNA_LDS];
  const size_t row = (size_t)blockIdx.x * h;
  const bool keep = h <= SNA_LDS;
  auto value = [&](int e) -> float {
    float y = 0.f;
#pragma unroll
    for (int i = 0; i < N; ++i) y += in.s[i] * to_f32(((const TX*)in.x[i])[row + e]);
    return y;
  };
  float rstd = 1.f;
  if (normed) {
    float ss = 0.f;
    for (int e = threadIdx.x; e < h; e += blockDim.x) {
      const float y = value(e);
      if (keep) row_y[e] = y;
      ss += y * y;
    }
    const float total = block_sum(ss, red);
    rstd = 1.f / sqrtf(total / (float)h + eps);
  }
  for (int e = threadIdx.x; e < h; e += blockDim.x) {
    float y = (normed && keep) ? row_y[e] : value(e);      // a thread reads back what it wrote itself
    if (normed) y = y * rstd * weight[(size_t)e * weight_stride];
    if (resid) {
      y += resid[row + e];
      resid[row + e] = y;
    }
    if (copy) copy[row + e] = from_f32<TO>(y);
  }
}

// The same with rows whose width is a multiple of 8 and at most 8 * SNA_CHUNKS * 1024: a thread holds CH (1, 2 or 4)
// runs of eight neighbouring elements in registers, everything it reads (the inputs, the stream, the weight) is
// asked for in one trip through 16-byte accesses, and nothing is read twice. (CH is a template parameter so that a
// row of 2,048 or 4,096 costs the registers of one or two runs, not of four, and more workgroups share a CU.)
#define SNA_CHUNKS 4
template <typename TX, typename TO, int N, int CH>
__global__ void sum_norm_add_vec_kernel(SumInputs in, const float* __restrict__ weight, int weight_stride, int normed,
                                        float eps, int h, float* __restrict__ resid, TO* __restrict__ copy) {
  __shared__ float red[17];
  const size_t row = (size_t)blockIdx.x * h;
  float y[CH][8], add[CH][8], w[CH][8];
  bool live[CH];
  float ss = 0.f;
#pragma unroll
  for (int r = 0; r < CH; ++r) {
    const int c = (threadIdx.x + r * blockDim.x) * 8;
    live[r] = c < h;
#pragma unroll
    for (int e = 0; e < 8; ++e) { y[r][e] = 0.f; add[r][e] = 0.f; w[r][e] = 1.f; }
    if (!live[r]) continue;
#pragma unroll
    for (int i = 0; i < N; ++i) {
      float v[8];
      Vec8<TX>::load((const TX*)in.x[i] + row + c, v);
#pragma unroll
      for (int e = 0; e < 8; ++e) y[r][e] += in.s[i] * v[e];
    }
    if (resid) Vec8<float>::load(resid + row + c, add[r]);
    if (normed && weight_stride) Vec8<float>::load(weight + c, w[r]);
#pragma unroll
    for (int e = 0; e < 8; ++e) ss += y[r][e] * y[r][e];
  }
  float rstd = 1.f;
  if (normed) {
    const float total = block_sum(ss, red);
    rstd = 1.f / sqrtf(total / (float)h + eps);
    if (!weight_stride) rstd *= weight[0];
  }
#pragma unroll
  for (int r = 0; r < CH; ++r) {
    if (!live[r]) continue;
    const int c = (threadIdx.x + r * blockDim.x) * 8;
    float o[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) o[e] = (normed ? y[r][e] * rstd * w[r][e] : y[r][e]) + add[r][e];
    if (resid) Vec8<float>::store(resid + row + c, o);
    if (copy) Vec8<TO>::store(copy + row + c, o);
  }
}

// One workgroup a (row, span): blockIdx.y picks the span.
struct NormSpans {
  int col0[2], width[2], count[2];
  const float* w[2];
};
template <typename TA>
__global__ void span_rmsnorm_kernel(TA* __restrict__ x, long ld, NormSpans sp, float eps) {
  __shared__ float red[17];
  const int k = blockIdx.y;
  TA* v = x + (size_t)blockIdx.x * ld + sp.col0[k];
  const int n = sp.width[k];
  float ss = 0.f;
  for (int e = threadIdx.x; e < n; e += blockDim.x) {
    const float a = to_f32(v[e]);
    ss += a * a;
  }
  const float total = block_sum(ss, red);
  const float rstd = 1.f / sqrtf(total / (float)sp.count[k] + eps);
  const float* w = sp.w[k];
  for (int e = threadIdx.x; e < n; e += blockDim.x) v[e] = from_f32<TA>(to_f32(v[e]) * rstd * w[e]);
}

// The same for runs that start and end on multiples of 8 columns and are at most 8 * SNA_CHUNKS * 1024 wide: a run in
// registers, 16-byte accesses, one trip to memory.
template <typename TA>
__global__ void span_rmsnorm_vec_kernel(TA* __restrict__ x, long ld, NormSpans sp, float eps) {
  __shared__ float red[17];
  const int k = blockIdx.y;
  TA* v = x + (size_t)blockIdx.x * ld + sp.col0[k];
  const int n = sp.width[k];
  const float* wt = sp.w[k];
  float a[SNA_CHUNKS][8], w[SNA_CHUNKS][8];
  float ss = 0.f;
#pragma unroll
  for (int r = 0; r < SNA_CHUNKS; ++r) {
    const int c = (threadIdx.x + r * blockDim.x) * 8;
#pragma unroll
    for (int e = 0; e < 8; ++e) a[r][e] = 0.f;
    if (c >= n) continue;
    Vec8<TA>::load(v + c, a[r]);
    Vec8<float>::load(wt + c, w[r]);
#pragma unroll
    for (int e = 0; e < 8; ++e) ss += a[r][e] * a[r][e];
  }
  const float total = block_sum(ss, red);
  const float rstd = 1.f / sqrtf(total / (float)sp.count[k] + eps);
#pragma unroll
  for (int r = 0; r < SNA_CHUNKS; ++r) {
    const int c = (threadIdx.x + r * blockDim.x) * 8;
    if (c >= n) continue;
    float o[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) o[e] = a[r][e] * rstd * w[r][e];
    Vec8<TA>::store(v + c, o);
  }
}

// One thread a (token, head, pair).
template <typename TA>
__global__ void turn_heads_kernel(TA* __restrict__ x, long ld, int heads, int head_stride, int width, int style,
                                  const int* __restrict__ positions, const float* __restrict__ inv_freq, float sign,
                                  const TA* __restrict__ gate, long ldg, int gate_stride, long total) {
  const long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const int half = width / 2;
  const int per_head = gate ? head_stride - half : half;   // with a gate the entries past the turned ones are visited too
  const int m = (int)(idx % per_head);
  const int hd = (int)((idx / per_head) % heads);
  const long t = idx / per_head / heads;
  TA* v = x + (size_t)t * ld + (size_t)hd * head_stride;
  const TA* gp = gate ? gate + (size_t)t * ldg + (size_t)hd * gate_stride : nullptr;
  if (m >= half) {                                         // an entry that does not turn: the gate alone
    const int e = m + half;
    if (e < head_stride) {
      const float z = to_f32(gp[e]);
      v[e] = from_f32<TA>(to_f32(v[e]) / (1.f + expf(-z)));
    }
    return;
  }
  const int i0 = style == 0 ? m : 2 * m, i1 = style == 0 ? m + half : 2 * m + 1;
  const float ang = (float)positions[t] * inv_freq[m];
  float sn, cs;
  sincosf(ang, &sn, &cs);
  sn *= sign;
  const float a = to_f32(v[i0]), b = to_f32(v[i1]);
  float ra = a * cs - b * sn, rb = b * cs + a * sn;
  if (gp) {
    ra = ra / (1.f + expf(-to_f32(gp[i0])));
    rb = rb / (1.f + expf(-to_f32(gp[i1])));
  }
  v[i0] = from_f32<TA>(ra);
  v[i1] = from_f32<TA>(rb);
}

}  // namespace

extern "C" int ra_stream_cast(const float* x, void* out, int act_dtype, long n, hipStream_t stream) {
  RA_CHECK(n > 0, "stream_cast: nothing to copy");
  RA_CHECK(act_dtype == RA_F32 || act_dtype == RA_BF16, "stream_cast: unknown dtype tag %d", act_dtype);
  if (n % 8 == 0 && ((uintptr_t)x % 16) == 0 && ((uintptr_t)out % 16) == 0) {
    size_t blocks = ((size_t)n / 8 + 255) / 256;
    if (blocks > 65535 * 4) blocks = 65535 * 4;
    if (act_dtype == RA_F32) stream_cast_vec_kernel<float><<<(unsigned)blocks, 256, 0, stream>>>(x, (float*)out, (size_t)n / 8);
    else stream_cast_vec_kernel<bf16_t><<<(unsigned)blocks, 256, 0, stream>>>(x, (bf16_t*)out, (size_t)n / 8);
  } else {
    size_t blocks = ((size_t)n + 255) / 256;
    if (blocks > 65535 * 4) blocks = 65535 * 4;
    if (act_dtype == RA_F32) stream_cast_kernel<float><<<(unsigned)blocks, 256, 0, stream>>>(x, (float*)out, (size_t)n);
    else stream_cast_kernel<bf16_t><<<(unsigned)blocks, 256, 0, stream>>>(x, (bf16_t*)out, (size_t)n);
  }
  RA_LAUNCH_CHECK("stream_cast");
  return 0;
}

// xs: n inputs [n_tokens, hidden] of type in_dtype, each times scales[i]; weight float, `weight_stride` 1 (a vector
// over the width) or 0 (one number); normed 0: the sum enters as it is; resid float or null; copy of type
// copy_dtype or null: the new stream (or, without resid, the result) in that type.
extern "C" int ra_sum_norm_add(const void* const* xs, const float* scales, int n, int in_dtype, const float* weight,
                               int weight_stride, int normed, float eps, int n_tokens, int hidden, float* resid,
                               void* copy, int copy_dtype, hipStream_t stream) {
  RA_CHECK(n >= 1 && n <= SNA_MAX, "sum_norm_add: %d inputs (1 to %d)", n, SNA_MAX);
  RA_CHECK(n_tokens > 0 && hidden > 0, "sum_norm_add: %d tokens, width %d", n_tokens, hidden);
  RA_CHECK(resid != nullptr || copy != nullptr, "sum_norm_add: the result goes into the stream or into a copy");
  RA_CHECK(!normed || weight != nullptr, "sum_norm_add: a norm needs its weight");
  RA_CHECK(weight_stride == 0 || weight_stride == 1, "sum_norm_add: the weight is one number or a vector");
  SumInputs in;
  for (int i = 0; i < SNA_MAX; ++i) {
    in.x[i] = i < n ? xs[i] : nullptr;
    in.s[i] = i < n ? scales[i] : 0.f;
  }
  int threads = hidden >= 2048 ? 512 : 256;
  // rows of whole 16-byte pieces in every operand: the form that keeps a row in registers
  bool vec = hidden % 8 == 0 && hidden <= 8 * SNA_CHUNKS * 1024 && ((uintptr_t)resid % 16) == 0 &&
             ((uintptr_t)copy % 16) == 0 && (!normed || weight_stride == 0 || ((uintptr_t)weight % 16) == 0);
  for (int i = 0; i < n; ++i) vec = vec && ((uintptr_t)xs[i] % 16) == 0;
  int chunks = 1;
  if (vec) {
    // rows up to 2,048 wide: one run a thread; from there workgroups of 256 threads with two or four runs each, and
    // beyond 8,192 more threads
    chunks = hidden <= 2048 ? 1 : hidden <= 4096 ? 2 : 4;
    threads = (hidden / (8 * chunks) + RA_WAVE - 1) / RA_WAVE * RA_WAVE;
  }
#define RA_SNA_VEC(TX, TO, N, CH)                                                                                      \
  sum_norm_add_vec_kernel<TX, TO, N, CH><<<n_tokens, threads, 0, stream>>>(in, weight, weight_stride, normed, eps,     \
                                                                           hidden, resid, (TO*)copy)
#define RA_SNA(TX, TO, N)                                                                                          \
  do {                                                                                                             \
    if (vec && chunks == 1) RA_SNA_VEC(TX, TO, N, 1);                                                              \
    else if (vec && chunks == 2) RA_SNA_VEC(TX, TO, N, 2);                                                         \
    else if (vec) RA_SNA_VEC(TX, TO, N, 4);                                                                        \
    else                                                                                                           \
      sum_norm_add_kernel<TX, TO, N><<<n_tokens, threads, 0, stream>>>(in, weight, weight_stride, normed, eps,     \
                                                                       hidden, resid, (TO*)copy);                  \
  } while (0)
#define RA_SNA_N(TX, TO)                \
  do {                                  \
    if (n == 1) RA_SNA(TX, TO, 1);      \
    else if (n == 2) RA_SNA(TX, TO, 2); \
    else if (n == 3) RA_SNA(TX, TO, 3); \
    else RA_SNA(TX, TO, 4);             \
  } while (0)
  const int cd = copy ? copy_dtype : RA_F32;
  if (in_dtype == RA_F32 && cd == RA_F32) RA_SNA_N(float, float);
  else if (in_dtype == RA_F32 && cd == RA_BF16) RA_SNA_N(float, bf16_t);
  else if (in_dtype == RA_BF16 && cd == RA_BF16) RA_SNA_N(bf16_t, bf16_t);
  else if (in_dtype == RA_BF16 && cd == RA_F32) RA_SNA_N(bf16_t, float);
  else return ra_fail("sum_norm_add: unknown dtype tags %d, %d", in_dtype, copy_dtype);
#undef RA_SNA_N
#undef RA_SNA
#undef RA_SNA_VEC
  RA_LAUNCH_CHECK("sum_norm_add");
  return 0;
}

// Up to two runs of columns of x [n_tokens rows, ld apart]: run k starts at col0[k], is width[k] wide, and is divided
// by sqrt(sum of its squares / count[k] + eps) and multiplied by the float vector w[k] (count: the entries that
// carry values, where the run holds rows of zeros between them).
extern "C" int ra_span_rmsnorm(void* x, int act_dtype, long ld, int n_tokens, int n_spans, const int* col0,
                               const int* width, const int* count, const float* const* w, float eps,
                               hipStream_t stream) {
  RA_CHECK(n_tokens > 0 && n_spans >= 1 && n_spans <= 2, "span_rmsnorm: %d tokens, %d runs (1 or 2)", n_tokens, n_spans);
  NormSpans sp = {};
  for (int k = 0; k < n_spans; ++k) {
    RA_CHECK(col0[k] >= 0 && width[k] > 0 && count[k] > 0 && col0[k] + width[k] <= ld && w[k] != nullptr,
             "span_rmsnorm: run %d: columns %d..%d of %ld, %d values", k, col0[k], col0[k] + width[k], ld, count[k]);
    sp.col0[k] = col0[k]; sp.width[k] = width[k]; sp.count[k] = count[k]; sp.w[k] = w[k];
  }
  RA_CHECK(n_tokens <= 0x7fffffff / 1, "span_rmsnorm: too many rows");
  const dim3 grid(n_tokens, n_spans);
  const int es = act_dtype == RA_F32 ? 4 : 2;
  bool vec = ((uintptr_t)x % 16) == 0 && (ld * es) % 16 == 0;
  int widest = 0;
  for (int k = 0; k < n_spans; ++k) {
    vec = vec && col0[k] % 8 == 0 && width[k] % 8 == 0 && width[k] <= 8 * SNA_CHUNKS * 1024 && ((uintptr_t)w[k] % 16) == 0;
    widest = width[k] > widest ? width[k] : widest;
  }
  int threads = (widest / 8 + RA_WAVE - 1) / RA_WAVE * RA_WAVE;
  if (threads > 1024) threads = 1024;
  if (act_dtype == RA_F32) {
    if (vec) span_rmsnorm_vec_kernel<float><<<grid, threads, 0, stream>>>((float*)x, ld, sp, eps);
    else span_rmsnorm_kernel<float><<<grid, 256, 0, stream>>>((float*)x, ld, sp, eps);
  } else if (act_dtype == RA_BF16) {
    if (vec) span_rmsnorm_vec_kernel<bf16_t><<<grid, threads, 0, stream>>>((bf16_t*)x, ld, sp, eps);
    else span_rmsnorm_kernel<bf16_t><<<grid, 256, 0, stream>>>((bf16_t*)x, ld, sp, eps);
  } else return ra_fail("span_rmsnorm: unknown dtype tag %d", act_dtype);
  RA_LAUNCH_CHECK("span_rmsnorm");
  return 0;
}

// x [n_tokens rows, ld apart] holds `heads` heads head_stride apart from column 0; the first `width` (even) entries
// of each turn by sign * positions[t] * inv_freq[m], pair m being (m, m + width / 2) (style 0) or (2m, 2m + 1)
// (style 1). gate (or null; rows ldg apart, heads gate_stride apart, the activations' type): every entry of a head,
// turned or not, is then multiplied by the sigmoid of the gate's entry at the same place.
extern "C" int ra_turn_heads(void* x, int act_dtype, long ld, int n_tokens, int heads, int head_stride, int width,
                             int style, const int* positions, const float* inv_freq, float sign, const void* gate,
                             long ldg, int gate_stride, hipStream_t stream) {
  RA_CHECK(n_tokens > 0 && heads > 0 && head_stride > 0, "turn_heads: %d tokens, %d heads of %d", n_tokens, heads, head_stride);
  RA_CHECK(width >= 0 && width % 2 == 0 && width <= head_stride, "turn_heads: %d turned entries of %d", width, head_stride);
  RA_CHECK((long)heads * head_stride <= ld, "turn_heads: %d heads of %d in rows of %ld", heads, head_stride, ld);
  RA_CHECK(style == 0 || style == 1, "turn_heads: pair layout %d", style);
  RA_CHECK(width == 0 || (positions && inv_freq), "turn_heads: positions and frequencies are needed");
  RA_CHECK(width > 0 || gate, "turn_heads: nothing to do");
  const int per_head = gate ? head_stride - width / 2 : width / 2;
  const long total = (long)n_tokens * heads * per_head;
  const unsigned blocks = (unsigned)((total + 255) / 256);
  if (act_dtype == RA_F32)
    turn_heads_kernel<float><<<blocks, 256, 0, stream>>>((float*)x, ld, heads, head_stride, width, style, positions,
                                                         inv_freq, sign, (const float*)gate, ldg, gate_stride, total);
  else if (act_dtype == RA_BF16)
    turn_heads_kernel<bf16_t><<<blocks, 256, 0, stream>>>((bf16_t*)x, ld, heads, head_stride, width, style, positions,
                                                          inv_freq, sign, (const bf16_t*)gate, ldg, gate_stride, total);
  else return ra_fail("turn_heads: unknown dtype tag %d", act_dtype);
  RA_LAUNCH_CHECK("turn_heads");
  return 0;
}
