// Mixture of experts: the router's choice (the `top` largest float logits, softmax over those alone) and the
// activation of the experts' up projections with the routing weights applied. Logits, their order, the
// exponentials and the weights are float whatever the activations' type.
#include "common.h"
#include "reinfer_hip.h"

// ---------------------------------------------------------------------------
// One wave a token: its float router logits z[0..E) (a product made them) go to LDS, then `top` rounds of a
// wave-wide maximum (ties go to the lower expert), then p_j = exp(z_j - z_0) / sum over the chosen.
// ids[t, j] and weights[t, j] come out in falling order of z.
// ---------------------------------------------------------------------------
#define MOE_TOPK_WAVES 4
__global__ void moe_topk_kernel(const float* __restrict__ logits, int ld, int E, int top, int* __restrict__ ids,
                                float* __restrict__ weights, int T) {
  extern __shared__ float zs[];          // [MOE_TOPK_WAVES][E]
  const int lane = threadIdx.x & (RA_WAVE - 1);
  const int wave = threadIdx.x / RA_WAVE;
  const int t = blockIdx.x * MOE_TOPK_WAVES + wave;
  if (t >= T) return;                    // whole waves leave; no workgroup barrier below
  float* z = zs + (size_t)wave * E;
  for (int e = lane; e < E; e += RA_WAVE) z[e] = logits[(size_t)t * ld + e];
  float z0 = 0.f, denom = 0.f, mine = 0.f;
  int mine_id = 0;
  for (int j = 0; j < top; ++j) {
    float best = -INFINITY;
    int at = 0x7fffffff;
    for (int e = lane; e < E; e += RA_WAVE) {      // a lane reads back only what it wrote itself
      const float v = z[e];
      if (at == 0x7fffffff || v > best) { best = v; at = e; }       // ascending e: the first of equals stays
    }
#pragma unroll
    for (int m = RA_WAVE / 2; m > 0; m >>= 1) {
      const float ob = __shfl_xor(best, m, RA_WAVE);
      const int oa = __shfl_xor(at, m, RA_WAVE);
      if (ob > best || (ob == best && oa < at)) { best = ob; at = oa; }
    }
    if (j == 0) z0 = best;
    const float p = expf(best - z0);
    denom += p;
    if (lane == j) { mine = p; mine_id = at; }    // lane j keeps the j-th choice (top <= 64)
    if (at < E && (at & (RA_WAVE - 1)) == lane) z[at] = -INFINITY;   // taken: its own lane strikes it
  }
  if (lane < top) {
    weights[(size_t)t * top + lane] = mine / denom;
    ids[(size_t)t * top + lane] = mine_id;
  }
}

extern "C" int ra_moe_topk(const float* logits, int ld, int experts, int top, int* ids, float* weights,
                           int n_tokens, hipStream_t stream) {
  RA_CHECK(n_tokens > 0 && experts > 0, "moe_topk: %d tokens, %d experts", n_tokens, experts);
  RA_CHECK(top > 0 && top <= experts && top <= RA_WAVE, "moe_topk: %d of %d experts (at most 64 chosen)", top, experts);
  RA_CHECK(ld >= experts, "moe_topk: rows of %d for %d experts", ld, experts);
  const size_t lds = (size_t)MOE_TOPK_WAVES * experts * sizeof(float);
  RA_CHECK(lds <= 64 * 1024, "moe_topk: %d experts", experts);
  const int groups = (n_tokens + MOE_TOPK_WAVES - 1) / MOE_TOPK_WAVES;
  moe_topk_kernel<<<groups, MOE_TOPK_WAVES * RA_WAVE, lds, stream>>>(logits, ld, experts, top, ids, weights, n_tokens);
  RA_LAUNCH_CHECK("moe_topk");
  return 0;
}

// ---------------------------------------------------------------------------
// Sigmoid scores with groups of experts. One wave a token: s_e = sigmoid(z_e) goes to LDS; with more than one
// group (equal runs of neighbours) a group's score is the sum of its `group_top` largest s, the `kept` groups
// with the highest scores stay (ties: the lower group) and the experts of the others are struck; then `top`
// rounds of a wave-wide maximum as above. weights[t, j] = s * scale, not renormalised.
// ---------------------------------------------------------------------------
__global__ void moe_route_sigmoid_kernel(const float* __restrict__ logits, int ld, int E, int top, int groups,
                                         int kept, int group_top, float scale, int* __restrict__ ids,
                                         float* __restrict__ weights, int T) {
  extern __shared__ float zs[];          // [MOE_TOPK_WAVES][E + groups]
  const int lane = threadIdx.x & (RA_WAVE - 1);
  const int wave = threadIdx.x / RA_WAVE;
  const int t = blockIdx.x * MOE_TOPK_WAVES + wave;
  if (t >= T) return;                    // whole waves leave; no workgroup barrier below
  float* s = zs + (size_t)wave * (E + groups);
  float* gs = s + E;
  for (int e = lane; e < E; e += RA_WAVE) s[e] = 1.f / (1.f + expf(-logits[(size_t)t * ld + e]));
  __builtin_amdgcn_wave_barrier();
  if (groups > 1) {
    const int size = E / groups;
    // a lane scores whole groups: the sum of the group's `group_top` largest, each round taking the largest that
    // comes behind the round before's in the order (score falling, index rising)
    for (int g = lane; g < groups; g += RA_WAVE) {
      float sum = 0.f, prev = INFINITY;
      int prev_at = -1;
      for (int r = 0; r < group_top && r < size; ++r) {
        float best = -INFINITY;
        int at = -1;
        for (int i = 0; i < size; ++i) {
          const float v = s[g * size + i];
          const bool behind = v < prev || (v == prev && i > prev_at);
          if (behind && (at < 0 || v > best)) { best = v; at = i; }
        }
        sum += best;
        prev = best;
        prev_at = at;
      }
      gs[g] = sum;
    }
    __builtin_amdgcn_wave_barrier();
    // keep the best `kept` groups: rounds of a wave-wide maximum over the group scores; a kept group's score
    // becomes +inf, and what is not +inf at the end is struck
    for (int j = 0; j < kept; ++j) {
      float best = -INFINITY;
      int at = 0x7fffffff;
      for (int g = lane; g < groups; g += RA_WAVE) {
        const float v = gs[g];
        if (v != INFINITY && (at == 0x7fffffff || v > best)) { best = v; at = g; }
      }
#pragma unroll
      for (int m = RA_WAVE / 2; m > 0; m >>= 1) {
        const float ob = __shfl_xor(best, m, RA_WAVE);
        const int oa = __shfl_xor(at, m, RA_WAVE);
        if (oa != 0x7fffffff && (at == 0x7fffffff || ob > best || (ob == best && oa < at))) { best = ob; at = oa; }
      }
      if (at < groups && (at & (RA_WAVE - 1)) == lane) gs[at] = INFINITY;
      __builtin_amdgcn_wave_barrier();
    }
    for (int e = lane; e < E; e += RA_WAVE)
      if (gs[e / size] != INFINITY) s[e] = -INFINITY;
    __builtin_amdgcn_wave_barrier();
  }
  float mine = 0.f;
  int mine_id = 0;
  for (int j = 0; j < top; ++j) {
    float best = -INFINITY;
    int at = 0x7fffffff;
    for (int e = lane; e < E; e += RA_WAVE) {      // a lane reads back only what it wrote itself
      const float v = s[e];
      if (at == 0x7fffffff || v > best) { best = v; at = e; }
    }
#pragma unroll
    for (int m = RA_WAVE / 2; m > 0; m >>= 1) {
      const float ob = __shfl_xor(best, m, RA_WAVE);
      const int oa = __shfl_xor(at, m, RA_WAVE);
      if (ob > best || (ob == best && oa < at)) { best = ob; at = oa; }
    }
    if (lane == j) { mine = best * scale; mine_id = at; }
    if (at < E && (at & (RA_WAVE - 1)) == lane) s[at] = -INFINITY;
  }
  if (lane < top) {
    weights[(size_t)t * top + lane] = mine;
    ids[(size_t)t * top + lane] = mine_id;
  }
}

extern "C" int ra_moe_route_sigmoid(const float* logits, int ld, int experts, int top, int groups, int kept,
                                    int group_top, float scale, int* ids, float* weights, int n_tokens,
                                    hipStream_t stream) {
  RA_CHECK(n_tokens > 0 && experts > 0, "moe_route_sigmoid: %d tokens, %d experts", n_tokens, experts);
  RA_CHECK(groups >= 1 && experts % groups == 0 && kept >= 1 && kept <= groups && group_top >= 1,
           "moe_route_sigmoid: %d experts in %d groups, %d kept, scored by %d", experts, groups, kept, group_top);
  RA_CHECK(top > 0 && top <= RA_WAVE && top <= kept * (experts / groups),
           "moe_route_sigmoid: %d of %d experts that can be chosen (at most 64)", top, kept * (experts / groups));
  RA_CHECK(ld >= experts, "moe_route_sigmoid: rows of %d for %d experts", ld, experts);
  const size_t lds = (size_t)MOE_TOPK_WAVES * (experts + groups) * sizeof(float);
  RA_CHECK(lds <= 64 * 1024, "moe_route_sigmoid: %d experts", experts);
  const int blocks = (n_tokens + MOE_TOPK_WAVES - 1) / MOE_TOPK_WAVES;
  moe_route_sigmoid_kernel<<<blocks, MOE_TOPK_WAVES * RA_WAVE, lds, stream>>>(logits, ld, experts, top, groups, kept,
                                                                              group_top, scale, ids, weights, n_tokens);
  RA_LAUNCH_CHECK("moe_route_sigmoid");
  return 0;
}

// ---------------------------------------------------------------------------
// Softmax scores over all E outputs of the router with a correction that only the choice sees. One wave a
// token: s = softmax(z) and the choice score c = s + correction go to LDS; with more than one group (equal runs
// of neighbours) a group's score is its largest c, the `kept` best groups stay (ties: the lower group) and the
// others' c become -inf; `top` rounds of a wave-wide maximum over c (ties: the lower index) choose; the weights
// are the chosen s over their sum + norm_eps.
// ---------------------------------------------------------------------------
__global__ void moe_route_softmax_kernel(const float* __restrict__ logits, int ld, int E, int top, int groups,
                                         int kept, const float* __restrict__ correction, float norm_eps,
                                         int* __restrict__ ids, float* __restrict__ weights, int T) {
  extern __shared__ float zs[];          // [MOE_TOPK_WAVES][2 E + groups]
  const int lane = threadIdx.x & (RA_WAVE - 1);
  const int wave = threadIdx.x / RA_WAVE;
  const int t = blockIdx.x * MOE_TOPK_WAVES + wave;
  if (t >= T) return;                    // whole waves leave; no workgroup barrier below
  float* s = zs + (size_t)wave * (2 * E + groups);
  float* c = s + E;
  float* gs = c + E;
  float m = -INFINITY;
  for (int e = lane; e < E; e += RA_WAVE) m = fmaxf(m, logits[(size_t)t * ld + e]);
  m = wave_max(m);
  float sum = 0.f;
  for (int e = lane; e < E; e += RA_WAVE) {
    const float p = expf(logits[(size_t)t * ld + e] - m);
    s[e] = p;
    sum += p;
  }
  sum = wave_sum(sum);
  for (int e = lane; e < E; e += RA_WAVE) {      // a lane reads back only what it wrote itself
    const float p = s[e] / sum;
    s[e] = p;
    c[e] = p + (correction ? correction[e] : 0.f);
  }
  __builtin_amdgcn_wave_barrier();
  if (groups > 1) {
    const int size = E / groups;
    for (int g = lane; g < groups; g += RA_WAVE) {
      float best = -INFINITY;
      for (int i = 0; i < size; ++i) best = fmaxf(best, c[g * size + i]);
      gs[g] = best;
    }
    __builtin_amdgcn_wave_barrier();
    for (int j = 0; j < kept; ++j) {
      float best = -INFINITY;
      int at = 0x7fffffff;
      for (int g = lane; g < groups; g += RA_WAVE) {
        const float v = gs[g];
        if (v != INFINITY && (at == 0x7fffffff || v > best)) { best = v; at = g; }
      }
#pragma unroll
      for (int mm = RA_WAVE / 2; mm > 0; mm >>= 1) {
        const float ob = __shfl_xor(best, mm, RA_WAVE);
        const int oa = __shfl_xor(at, mm, RA_WAVE);
        if (oa != 0x7fffffff && (at == 0x7fffffff || ob > best || (ob == best && oa < at))) { best = ob; at = oa; }
      }
      if (at < groups && (at & (RA_WAVE - 1)) == lane) gs[at] = INFINITY;
      __builtin_amdgcn_wave_barrier();
    }
    for (int e = lane; e < E; e += RA_WAVE)
      if (gs[e / size] != INFINITY) c[e] = -INFINITY;
    __builtin_amdgcn_wave_barrier();
  }
  float mine = 0.f, total = 0.f;
  int mine_id = 0;
  for (int j = 0; j < top; ++j) {
    float best = -INFINITY;
    int at = 0x7fffffff;
    for (int e = lane; e < E; e += RA_WAVE) {
      const float v = c[e];
      if (at == 0x7fffffff || v > best) { best = v; at = e; }
    }
#pragma unroll
    for (int mm = RA_WAVE / 2; mm > 0; mm >>= 1) {
      const float ob = __shfl_xor(best, mm, RA_WAVE);
      const int oa = __shfl_xor(at, mm, RA_WAVE);
      if (ob > best || (ob == best && oa < at)) { best = ob; at = oa; }
    }
    const float p = s[at];                 // every lane reads the winner's score: written before the barrier above
    total += p;
    if (lane == j) { mine = p; mine_id = at; }
    if ((at & (RA_WAVE - 1)) == lane) c[at] = -INFINITY;
  }
  if (lane < top) {
    weights[(size_t)t * top + lane] = mine / (total + norm_eps);
    ids[(size_t)t * top + lane] = mine_id;
  }
}

extern "C" int ra_moe_route_softmax(const float* logits, int ld, int experts, int top, int groups, int kept,
                                    const float* correction, float norm_eps, int* ids, float* weights, int n_tokens,
                                    hipStream_t stream) {
  RA_CHECK(n_tokens > 0 && experts > 0, "moe_route_softmax: %d tokens, %d experts", n_tokens, experts);
  RA_CHECK(groups >= 1 && experts % groups == 0 && kept >= 1 && kept <= groups,
           "moe_route_softmax: %d experts in %d groups, %d kept", experts, groups, kept);
  RA_CHECK(top > 0 && top <= RA_WAVE && top <= kept * (experts / groups),
           "moe_route_softmax: %d of %d experts that can be chosen (at most 64)", top, kept * (experts / groups));
  RA_CHECK(ld >= experts, "moe_route_softmax: rows of %d for %d experts", ld, experts);
  const size_t lds = (size_t)MOE_TOPK_WAVES * (2 * experts + groups) * sizeof(float);
  RA_CHECK(lds <= 64 * 1024, "moe_route_softmax: %d experts", experts);
  const int blocks = (n_tokens + MOE_TOPK_WAVES - 1) / MOE_TOPK_WAVES;
  moe_route_softmax_kernel<<<blocks, MOE_TOPK_WAVES * RA_WAVE, lds, stream>>>(logits, ld, experts, top, groups, kept,
                                                                              correction, norm_eps, ids, weights,
                                                                              n_tokens);
  RA_LAUNCH_CHECK("moe_route_softmax");
  return 0;
}

// ---------------------------------------------------------------------------
// Identity experts: a chosen id of E or more names no matrices; its output is the token's input row. One
// workgroup a token: y[t, :] += (sum of the weights of such choices) * x[t, :], the sum and product in float.
// ---------------------------------------------------------------------------
template <typename TA>
__global__ void moe_identity_add_kernel(TA* __restrict__ y, int ldy, const TA* __restrict__ x, int ldx,
                                        const int* __restrict__ ids, const float* __restrict__ weights, int top, int E,
                                        int width) {
  const size_t t = blockIdx.x;
  float coef = 0.f;
  for (int j = 0; j < top; ++j)
    if (ids[t * top + j] >= E) coef += weights[t * top + j];
  if (coef == 0.f) return;
  for (int e = threadIdx.x; e < width; e += blockDim.x)
    y[t * ldy + e] = from_f32<TA>(to_f32(y[t * ldy + e]) + coef * to_f32(x[t * ldx + e]));
}

// the same, eight columns a thread through 16-byte accesses, a row split over blockIdx.y
template <typename TA>
__global__ void moe_identity_add_x8_kernel(TA* __restrict__ y, int ldy, const TA* __restrict__ x, int ldx,
                                           const int* __restrict__ ids, const float* __restrict__ weights, int top,
                                           int E, int width) {
  const size_t t = blockIdx.x;
  const int e = (blockIdx.y * blockDim.x + threadIdx.x) * 8;
  if (e >= width) return;
  float coef = 0.f;
  for (int j = 0; j < top; ++j)
    if (ids[t * top + j] >= E) coef += weights[t * top + j];
  if (coef == 0.f) return;
  float a[8], b[8];
  Vec8<TA>::load(y + t * ldy + e, a);
  Vec8<TA>::load(x + t * ldx + e, b);
#pragma unroll
  for (int i = 0; i < 8; ++i) a[i] += coef * b[i];
  Vec8<TA>::store(y + t * ldy + e, a);
}

extern "C" int ra_moe_identity_add(void* y, int ldy, const void* x, int ldx, int act_dtype, const int* ids,
                                   const float* weights, int top, int experts, int n_tokens, int width,
                                   hipStream_t stream) {
  RA_CHECK(n_tokens > 0 && width > 0 && top > 0 && ldy >= width && ldx >= width,
           "moe_identity_add: %d tokens, width %d, %d choices", n_tokens, width, top);
  const int threads = width >= 1024 ? 256 : width >= 256 ? 128 : 64;
  const int ab = act_dtype == RA_F32 ? 4 : 2;
  if (width % 8 == 0 && ra_rows_16b(y, ldy, ab) && ra_rows_16b(x, ldx, ab) && (act_dtype == RA_F32 || act_dtype == RA_BF16)) {
    const int vthreads = width >= 2048 ? 128 : 64;
    const dim3 vgrid(n_tokens, (width / 8 + vthreads - 1) / vthreads);
    if (act_dtype == RA_F32)
      moe_identity_add_x8_kernel<float><<<vgrid, vthreads, 0, stream>>>((float*)y, ldy, (const float*)x, ldx, ids, weights,
                                                                        top, experts, width);
    else
      moe_identity_add_x8_kernel<bf16_t><<<vgrid, vthreads, 0, stream>>>((bf16_t*)y, ldy, (const bf16_t*)x, ldx, ids,
                                                                         weights, top, experts, width);
    RA_LAUNCH_CHECK("moe_identity_add");
    return 0;
  }
  if (act_dtype == RA_F32)
    moe_identity_add_kernel<float><<<n_tokens, threads, 0, stream>>>((float*)y, ldy, (const float*)x, ldx, ids, weights,
                                                                     top, experts, width);
  else if (act_dtype == RA_BF16)
    moe_identity_add_kernel<bf16_t><<<n_tokens, threads, 0, stream>>>((bf16_t*)y, ldy, (const bf16_t*)x, ldx, ids,
                                                                      weights, top, experts, width);
  else
    return ra_fail("moe_identity_add: unknown dtype tag %d", act_dtype);
  RA_LAUNCH_CHECK("moe_identity_add");
  return 0;
}

// ---------------------------------------------------------------------------
// Gated experts side by side: gu[t, e * 2 ff + j] is expert e's gate projection of token t and
// gu[t, e * 2 ff + ff + j] its up projection; behind the experts a shared expert's [gate | up] of `shared` each.
// act[t, e * ff + j] = p(t, e) * silu(gate) * up for the chosen experts and 0 for the others;
// act[t, E * ff + j] = silu(gate) * up of the shared expert.
// ---------------------------------------------------------------------------
template <typename TA>
__global__ void moe_silu_gate_scale_kernel(const TA* __restrict__ gu, TA* __restrict__ act,
                                           const int* __restrict__ ids, const float* __restrict__ weights, int top,
                                           int E, int ff, int shared, const float* __restrict__ shared_logit,
                                           int ld_logit) {
  extern __shared__ float gate[];        // [E]
  const int t = blockIdx.y;
  for (int e = threadIdx.x; e < E; e += blockDim.x) gate[e] = 0.f;
  __syncthreads();
  for (int j = threadIdx.x; j < top; j += blockDim.x) {
    const int id = ids[(size_t)t * top + j];
    if (id < E) gate[id] = weights[(size_t)t * top + j];     // an id past the experts names no matrices (an identity expert)
  }
  __syncthreads();
  const int n = E * ff + shared;
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const TA* row = gu + (size_t)t * 2 * n;
  float p, g, u;
  if (i < E * ff) {
    const int e = i / ff, j = i - e * ff;
    p = gate[e];
    if (p == 0.f) {
      act[(size_t)t * n + i] = from_f32<TA>(0.f);
      return;
    }
    g = to_f32(row[(size_t)e * 2 * ff + j]);
    u = to_f32(row[(size_t)e * 2 * ff + ff + j]);
  } else {
    const int j = i - E * ff;
    p = shared_logit ? 1.f / (1.f + expf(-shared_logit[(size_t)t * ld_logit])) : 1.f;
    g = to_f32(row[(size_t)E * 2 * ff + j]);
    u = to_f32(row[(size_t)E * 2 * ff + shared + j]);
  }
  act[(size_t)t * n + i] = from_f32<TA>(p * (g / (1.f + expf(-g))) * u);
}

// the same, eight columns a thread through 16-byte accesses (ff and shared multiples of 8: the eight lie in one
// expert, or in the shared one)
template <typename TA>
__global__ void moe_silu_gate_scale_x8_kernel(const TA* __restrict__ gu, TA* __restrict__ act,
                                              const int* __restrict__ ids, const float* __restrict__ weights, int top,
                                              int E, int ff, int shared, const float* __restrict__ shared_logit,
                                              int ld_logit) {
  extern __shared__ float gate[];        // [E]
  const int t = blockIdx.y;
  for (int e = threadIdx.x; e < E; e += blockDim.x) gate[e] = 0.f;
  __syncthreads();
  for (int j = threadIdx.x; j < top; j += blockDim.x) {
    const int id = ids[(size_t)t * top + j];
    if (id < E) gate[id] = weights[(size_t)t * top + j];
  }
  __syncthreads();
  const int n = E * ff + shared;
  const int i = (blockIdx.x * blockDim.x + threadIdx.x) * 8;
  if (i >= n) return;
  const TA* row = gu + (size_t)t * 2 * n;
  float p, g[8], u[8];
  if (i < E * ff) {
    const int e = i / ff, j = i - e * ff;
    p = gate[e];
    if (p == 0.f) {
#pragma unroll
      for (int k = 0; k < 8; ++k) g[k] = 0.f;
      Vec8<TA>::store(act + (size_t)t * n + i, g);
      return;
    }
    Vec8<TA>::load(row + (size_t)e * 2 * ff + j, g);
    Vec8<TA>::load(row + (size_t)e * 2 * ff + ff + j, u);
  } else {
    const int j = i - E * ff;
    p = shared_logit ? 1.f / (1.f + expf(-shared_logit[(size_t)t * ld_logit])) : 1.f;
    Vec8<TA>::load(row + (size_t)E * 2 * ff + j, g);
    Vec8<TA>::load(row + (size_t)E * 2 * ff + shared + j, u);
  }
#pragma unroll
  for (int k = 0; k < 8; ++k) g[k] = p * (g[k] / (1.f + expf(-g[k]))) * u[k];
  Vec8<TA>::store(act + (size_t)t * n + i, g);
}

extern "C" int ra_moe_silu_gate_scale(const void* gu, void* act, int act_dtype, const int* ids, const float* weights,
                                      int top, int experts, int ff, int shared, int n_tokens, hipStream_t stream) {
  return ra_moe_silu_gate_scale_shared(gu, act, act_dtype, ids, weights, top, experts, ff, shared, nullptr, 0, n_tokens,
                                       stream);
}

extern "C" int ra_moe_silu_gate_scale_shared(const void* gu, void* act, int act_dtype, const int* ids,
                                             const float* weights, int top, int experts, int ff, int shared,
                                             const float* shared_logit, int ld_logit, int n_tokens,
                                             hipStream_t stream) {
  RA_CHECK(n_tokens > 0 && experts > 0 && ff > 0 && top > 0 && shared >= 0,
           "moe_silu_gate_scale: %d tokens, %d of %d experts of %d, shared %d", n_tokens, top, experts, ff, shared);
  RA_CHECK(n_tokens <= 65535, "moe_silu_gate_scale: %d tokens in one launch (max 65535)", n_tokens);
  const size_t lds = (size_t)experts * sizeof(float);
  RA_CHECK(lds <= 64 * 1024, "moe_silu_gate_scale: %d experts", experts);
  const int n = experts * ff + shared;
  dim3 grid((n + 255) / 256, n_tokens);
  if (ff % 8 == 0 && shared % 8 == 0 && ((uintptr_t)gu % 16) == 0 && ((uintptr_t)act % 16) == 0 &&
      (act_dtype == RA_F32 || act_dtype == RA_BF16)) {
    dim3 grid8((n / 8 + 255) / 256, n_tokens);
    if (act_dtype == RA_F32)
      moe_silu_gate_scale_x8_kernel<float><<<grid8, 256, lds, stream>>>((const float*)gu, (float*)act, ids, weights, top,
                                                                        experts, ff, shared, shared_logit, ld_logit);
    else
      moe_silu_gate_scale_x8_kernel<bf16_t><<<grid8, 256, lds, stream>>>((const bf16_t*)gu, (bf16_t*)act, ids, weights,
                                                                         top, experts, ff, shared, shared_logit, ld_logit);
    RA_LAUNCH_CHECK("moe_silu_gate_scale");
    return 0;
  }
  if (act_dtype == RA_F32)
    moe_silu_gate_scale_kernel<float><<<grid, 256, lds, stream>>>((const float*)gu, (float*)act, ids, weights, top,
                                                                   experts, ff, shared, shared_logit, ld_logit);
  else if (act_dtype == RA_BF16)
    moe_silu_gate_scale_kernel<bf16_t><<<grid, 256, lds, stream>>>((const bf16_t*)gu, (bf16_t*)act, ids, weights, top,
                                                                    experts, ff, shared, shared_logit, ld_logit);
  else
    return ra_fail("moe_silu_gate_scale: unknown dtype tag %d", act_dtype);
  RA_LAUNCH_CHECK("moe_silu_gate_scale");
  return 0;
}

// ---------------------------------------------------------------------------
// Experts side by side: up[t, e * ff + j] is expert e's up projection of token t. act[t, e * ff + j] =
// p(t, e) * relu(up)^2 for the chosen experts, 0 for the others, so that one product with the down
// projections laid side by side, [width, E * ff], is the weighted sum of the chosen experts' outputs.
// ---------------------------------------------------------------------------
template <typename TA>
__global__ void moe_relu2_scale_kernel(const TA* __restrict__ up, TA* __restrict__ act, const int* __restrict__ ids,
                                       const float* __restrict__ weights, int top, int E, int ff) {
  extern __shared__ float gate[];        // [E]
  const int t = blockIdx.y;
  for (int e = threadIdx.x; e < E; e += blockDim.x) gate[e] = 0.f;
  __syncthreads();
  for (int j = threadIdx.x; j < top; j += blockDim.x) gate[ids[(size_t)t * top + j]] = weights[(size_t)t * top + j];
  __syncthreads();
  const int n = E * ff;
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) {
    const float g = gate[i / ff];
    float v = 0.f;
    if (g != 0.f) {
      const float u = fmaxf(to_f32(up[(size_t)t * n + i]), 0.f);
      v = g * (u * u);
    }
    act[(size_t)t * n + i] = from_f32<TA>(v);
  }
}

// the same, eight bfloat16 columns a thread (ff a multiple of 8: the eight lie in one expert)
__global__ void moe_relu2_scale_x8_kernel(const bf16_t* __restrict__ up, bf16_t* __restrict__ act,
                                          const int* __restrict__ ids, const float* __restrict__ weights, int top,
                                          int E, int ff) {
  extern __shared__ float gate[];        // [E]
  const int t = blockIdx.y;
  for (int e = threadIdx.x; e < E; e += blockDim.x) gate[e] = 0.f;
  __syncthreads();
  for (int j = threadIdx.x; j < top; j += blockDim.x) gate[ids[(size_t)t * top + j]] = weights[(size_t)t * top + j];
  __syncthreads();
  const int n = E * ff;
  const int i = (blockIdx.x * blockDim.x + threadIdx.x) * 8;
  if (i < n) {
    const float g = gate[i / ff];
    bf16x8_t o = {0, 0, 0, 0, 0, 0, 0, 0};
    if (g != 0.f) {
      const bf16x8_t u = *(const bf16x8_t*)(up + (size_t)t * n + i);
#pragma unroll
      for (int k = 0; k < 8; ++k) {
        const float v = fmaxf((float)u[k], 0.f);
        o[k] = (bf16_t)(g * (v * v));
      }
    }
    *(bf16x8_t*)(act + (size_t)t * n + i) = o;
  }
}

extern "C" int ra_moe_relu2_scale(const void* up, void* act, int act_dtype, const int* ids, const float* weights,
                                  int top, int experts, int ff, int n_tokens, hipStream_t stream) {
  RA_CHECK(n_tokens > 0 && experts > 0 && ff > 0 && top > 0 && top <= experts,
           "moe_relu2_scale: %d tokens, %d of %d experts of %d", n_tokens, top, experts, ff);
  RA_CHECK(n_tokens <= 65535, "moe_relu2_scale: %d tokens in one launch (max 65535)", n_tokens);
  const size_t lds = (size_t)experts * sizeof(float);
  RA_CHECK(lds <= 64 * 1024, "moe_relu2_scale: %d experts", experts);
  dim3 grid((experts * ff + 255) / 256, n_tokens);
  if (act_dtype == RA_BF16 && ff % 8 == 0 && ((uintptr_t)up % 16) == 0 && ((uintptr_t)act % 16) == 0) {
    dim3 grid8((experts * ff / 8 + 255) / 256, n_tokens);
    moe_relu2_scale_x8_kernel<<<grid8, 256, lds, stream>>>((const bf16_t*)up, (bf16_t*)act, ids, weights, top, experts, ff);
  } else if (act_dtype == RA_F32)
    moe_relu2_scale_kernel<float><<<grid, 256, lds, stream>>>((const float*)up, (float*)act, ids, weights, top, experts, ff);
  else if (act_dtype == RA_BF16)
    moe_relu2_scale_kernel<bf16_t><<<grid, 256, lds, stream>>>((const bf16_t*)up, (bf16_t*)act, ids, weights, top, experts, ff);
  else
    return ra_fail("moe_relu2_scale: unknown dtype tag %d", act_dtype);
  RA_LAUNCH_CHECK("moe_relu2_scale");
  return 0;
}

// ---------------------------------------------------------------------------
// Few tokens (a decode step of one or two requests): only the chosen experts' rows are read. Pair p = (token
// t, choice j) with expert e = ids[p] and weight g = weights[p]:
//   act[p, f]   = g * relu(W_up[e * ff + f, :] . x[t, :])^2          one wave a row f, lanes split the width
//   y[t, n]     = sum_j W_down[n, e_j * ff : (e_j + 1) * ff] . act[p_j, :]   one wave a column n, added into the
//                 float stream (resid) or written to out
// bfloat16 rows in steps of 8 are read 16 bytes a lane; anything else element by element. Sums are float.
// ---------------------------------------------------------------------------
// s[r] += w_r . v for four rows w_0..w_3 that share v: the lanes split K; rows of bfloat16 in steps of 8 are
// read 16 bytes a lane, four loads in flight beside the shared one
template <typename TA>
__device__ __forceinline__ void moe_dot4(const TA* const (&w)[4], const TA* __restrict__ v, int K, int lane, bool vec,
                                         float (&s)[4]) {
  for (int k = lane; k < K; k += RA_WAVE) {
    const float b = to_f32(v[k]);
#pragma unroll
    for (int r = 0; r < 4; ++r) s[r] += to_f32(w[r][k]) * b;
  }
}
template <>
__device__ __forceinline__ void moe_dot4<bf16_t>(const bf16_t* const (&w)[4], const bf16_t* __restrict__ v, int K,
                                                 int lane, bool vec, float (&s)[4]) {
  if (vec) {
    for (int k = lane * 8; k < K; k += RA_WAVE * 8) {
      const bf16x8_t b = *(const bf16x8_t*)(v + k);
      bf16x8_t a[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) a[r] = *(const bf16x8_t*)(w[r] + k);
#pragma unroll
      for (int r = 0; r < 4; ++r)
#pragma unroll
        for (int i = 0; i < 8; ++i) s[r] += (float)a[r][i] * (float)b[i];
    }
  } else {
    for (int k = lane; k < K; k += RA_WAVE) {
      const float b = (float)v[k];
#pragma unroll
      for (int r = 0; r < 4; ++r) s[r] += (float)w[r][k] * b;
    }
  }
}

#define MOE_ROWS 16          // rows (or columns) a workgroup of four waves takes, four a wave
template <typename TA>
__global__ void __launch_bounds__(256)
moe_up_chosen_kernel(const TA* __restrict__ x, int ldx, const TA* __restrict__ Wup, const int* __restrict__ ids,
                     const float* __restrict__ weights, TA* __restrict__ act, int ff, int width, int top, int vec) {
  const int lane = threadIdx.x & (RA_WAVE - 1);
  const int wave = threadIdx.x / RA_WAVE;
  const int p = blockIdx.y;
  const int t = p / top;
  const int e = ids[p];
  const float g = weights[p];
  const int f0 = blockIdx.x * MOE_ROWS + wave * 4;
  if (f0 >= ff) return;
  const TA* w[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) w[r] = Wup + ((size_t)e * ff + (f0 + r < ff ? f0 + r : f0)) * width;   // past the end: a row again, not stored
  float s[4] = {0.f, 0.f, 0.f, 0.f};
  moe_dot4<TA>(w, x + (size_t)t * ldx, width, lane, vec != 0, s);
#pragma unroll
  for (int r = 0; r < 4; ++r) s[r] = wave_sum(s[r]);
  if (lane < 4 && f0 + lane < ff) {
    const float u = fmaxf(lane == 0 ? s[0] : lane == 1 ? s[1] : lane == 2 ? s[2] : s[3], 0.f);
    act[(size_t)p * ff + f0 + lane] = from_f32<TA>(g * (u * u));
  }
}

template <typename TA>
__global__ void __launch_bounds__(256)
moe_down_chosen_kernel(const TA* __restrict__ act, const TA* __restrict__ Wdown, const int* __restrict__ ids,
                       float* __restrict__ resid, TA* __restrict__ out, int ff, int width, int E, int top, int vec) {
  const int lane = threadIdx.x & (RA_WAVE - 1);
  const int wave = threadIdx.x / RA_WAVE;
  const int t = blockIdx.y;
  const int n0 = blockIdx.x * MOE_ROWS + wave * 4;
  if (n0 >= width) return;
  float s[4] = {0.f, 0.f, 0.f, 0.f};
  for (int j = 0; j < top; ++j) {               // choice order: the same sum whatever else is in the step
    const int p = t * top + j;
    const TA* w[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) w[r] = Wdown + (size_t)(n0 + r < width ? n0 + r : n0) * E * ff + (size_t)ids[p] * ff;
    moe_dot4<TA>(w, act + (size_t)p * ff, ff, lane, vec != 0, s);
  }
#pragma unroll
  for (int r = 0; r < 4; ++r) s[r] = wave_sum(s[r]);
  if (lane < 4 && n0 + lane < width) {
    const float v = lane == 0 ? s[0] : lane == 1 ? s[1] : lane == 2 ? s[2] : s[3];
    const size_t at = (size_t)t * width + n0 + lane;
    if (resid) resid[at] += v;                   // this thread alone owns (t, n)
    else out[at] = from_f32<TA>(v);
  }
}

extern "C" int ra_moe_up_chosen(const void* x, int ldx, const void* w_up, const int* ids, const float* weights,
                                void* act, int act_dtype, int n_tokens, int top, int experts, int ff, int width,
                                hipStream_t stream) {
  RA_CHECK(n_tokens > 0 && top > 0 && top <= experts && ff > 0 && width > 0 && ldx >= width,
           "moe_up_chosen: %d tokens, %d of %d experts of %d x %d", n_tokens, top, experts, ff, width);
  RA_CHECK((long)n_tokens * top <= 65535, "moe_up_chosen: %d pairs in one launch", n_tokens * top);
  const int vec = (width % 8 == 0 && ldx % 8 == 0 && ((uintptr_t)x % 16) == 0 && ((uintptr_t)w_up % 16) == 0) ? 1 : 0;
  dim3 grid((ff + MOE_ROWS - 1) / MOE_ROWS, n_tokens * top);
  if (act_dtype == RA_F32)
    moe_up_chosen_kernel<float><<<grid, 256, 0, stream>>>((const float*)x, ldx, (const float*)w_up, ids, weights,
                                                          (float*)act, ff, width, top, 0);
  else if (act_dtype == RA_BF16)
    moe_up_chosen_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)x, ldx, (const bf16_t*)w_up, ids, weights,
                                                           (bf16_t*)act, ff, width, top, vec);
  else
    return ra_fail("moe_up_chosen: unknown dtype tag %d", act_dtype);
  RA_LAUNCH_CHECK("moe_up_chosen");
  return 0;
}

extern "C" int ra_moe_down_chosen(const void* act, const void* w_down, const int* ids, float* resid, void* out,
                                  int act_dtype, int n_tokens, int top, int experts, int ff, int width,
                                  hipStream_t stream) {
  RA_CHECK(n_tokens > 0 && top > 0 && top <= experts && ff > 0 && width > 0,
           "moe_down_chosen: %d tokens, %d of %d experts of %d x %d", n_tokens, top, experts, ff, width);
  RA_CHECK((resid != nullptr) != (out != nullptr), "moe_down_chosen: the result goes into the stream or into out");
  RA_CHECK(n_tokens <= 65535, "moe_down_chosen: %d tokens in one launch", n_tokens);
  const int vec = (ff % 8 == 0 && ((uintptr_t)act % 16) == 0 && ((uintptr_t)w_down % 16) == 0) ? 1 : 0;
  dim3 grid((width + MOE_ROWS - 1) / MOE_ROWS, n_tokens);
  if (act_dtype == RA_F32)
    moe_down_chosen_kernel<float><<<grid, 256, 0, stream>>>((const float*)act, (const float*)w_down, ids, resid,
                                                            (float*)out, ff, width, experts, top, 0);
  else if (act_dtype == RA_BF16)
    moe_down_chosen_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)act, (const bf16_t*)w_down, ids, resid,
                                                             (bf16_t*)out, ff, width, experts, top, vec);
  else
    return ra_fail("moe_down_chosen: unknown dtype tag %d", act_dtype);
  RA_LAUNCH_CHECK("moe_down_chosen");
  return 0;
}

// ---------------------------------------------------------------------------
// The same for gated experts whose [gate; up] rows lie one expert after the other in one matrix, a shared
// expert's behind them, and whose down projections lie side by side, the shared one's last. Pair p = (token t,
// choice j), j < top; with a shared expert one more pair a token, j = top. act is [T, top * ff + shared]:
//   act[t, j * ff + f]   = g * silu(W[e 2 ff + f, :] . x[t]) * (W[e 2 ff + ff + f, :] . x[t])     e = ids[t, j], g = weights[t, j]
//   act[t, top * ff + f] = g_s * silu(W[E 2 ff + f, :] . x[t]) * (W[E 2 ff + shared + f, :] . x[t])
//                          g_s = sigmoid(shared_logit[t]) or 1
//   y[t, n] = sum_j Wd[n, e_j ff : (e_j + 1) ff] . act[t, j ff : ...] + Wd[n, E ff :] . act[t, top ff :]
//             + (sum of g over choices with e >= E) * x[t, n]
// A chosen id of E or more names no matrices (an identity expert): its part of act is zero and not read.
// ---------------------------------------------------------------------------
template <typename TA>
__global__ void __launch_bounds__(256)
moe_gate_up_chosen_kernel(const TA* __restrict__ x, int ldx, const TA* __restrict__ Wgu, const int* __restrict__ ids,
                          const float* __restrict__ weights, const float* __restrict__ shared_logit, int ld_logit,
                          TA* __restrict__ act, int ff, int shared, int E, int width, int top, int vec) {
  const int lane = threadIdx.x & (RA_WAVE - 1);
  const int wave = threadIdx.x / RA_WAVE;
  const int per_token = top + (shared > 0 ? 1 : 0);
  const int t = blockIdx.y / per_token, j = blockIdx.y - t * per_token;
  const bool is_shared = j == top;
  const int rows = is_shared ? shared : ff;
  const int f0 = blockIdx.x * MOE_ROWS + wave * 4;
  if (f0 >= rows) return;
  TA* o = act + (size_t)t * ((size_t)top * ff + shared) + (size_t)j * ff;
  const int e = is_shared ? E : ids[t * top + j];
  if (e > E || (e == E && !is_shared)) {          // an identity expert
    if (lane < 4 && f0 + lane < rows) o[f0 + lane] = from_f32<TA>(0.f);
    return;
  }
  const float g = is_shared ? (shared_logit ? 1.f / (1.f + expf(-shared_logit[(size_t)t * ld_logit])) : 1.f)
                            : weights[t * top + j];
  const TA* base = Wgu + (size_t)e * 2 * ff * width;          // the shared expert's rows lie behind E experts'
  const TA* wg[4];
  const TA* wu[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int f = f0 + r < rows ? f0 + r : f0;                 // past the end: a row again, not stored
    wg[r] = base + (size_t)f * width;
    wu[r] = base + (size_t)(rows + f) * width;
  }
  float sg[4] = {0.f, 0.f, 0.f, 0.f}, su[4] = {0.f, 0.f, 0.f, 0.f};
  moe_dot4<TA>(wg, x + (size_t)t * ldx, width, lane, vec != 0, sg);
  moe_dot4<TA>(wu, x + (size_t)t * ldx, width, lane, vec != 0, su);
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    sg[r] = wave_sum(sg[r]);
    su[r] = wave_sum(su[r]);
  }
  if (lane < 4 && f0 + lane < rows) {
    const float a = lane == 0 ? sg[0] : lane == 1 ? sg[1] : lane == 2 ? sg[2] : sg[3];
    const float u = lane == 0 ? su[0] : lane == 1 ? su[1] : lane == 2 ? su[2] : su[3];
    o[f0 + lane] = from_f32<TA>(g * (a / (1.f + expf(-a))) * u);
  }
}

template <typename TA>
__global__ void __launch_bounds__(256)
moe_down_gated_chosen_kernel(const TA* __restrict__ act, const TA* __restrict__ Wdown, const int* __restrict__ ids,
                             const float* __restrict__ weights, const TA* __restrict__ x, int ldx,
                             TA* __restrict__ out, int ff, int shared, int width, int E, int top, int vec) {
  const int lane = threadIdx.x & (RA_WAVE - 1);
  const int wave = threadIdx.x / RA_WAVE;
  const int t = blockIdx.y;
  const int n0 = blockIdx.x * MOE_ROWS + wave * 4;
  if (n0 >= width) return;
  const size_t ldw = (size_t)E * ff + shared, lda = (size_t)top * ff + shared;
  float s[4] = {0.f, 0.f, 0.f, 0.f};
  float coef = 0.f;
  const TA* w[4];
  for (int j = 0; j < top; ++j) {               // choice order: the same sum whatever else is in the step
    const int e = ids[t * top + j];
    if (e >= E) {
      coef += weights[t * top + j];
      continue;
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) w[r] = Wdown + (size_t)(n0 + r < width ? n0 + r : n0) * ldw + (size_t)e * ff;
    moe_dot4<TA>(w, act + t * lda + (size_t)j * ff, ff, lane, vec != 0, s);
  }
  if (shared > 0) {
#pragma unroll
    for (int r = 0; r < 4; ++r) w[r] = Wdown + (size_t)(n0 + r < width ? n0 + r : n0) * ldw + (size_t)E * ff;
    moe_dot4<TA>(w, act + t * lda + (size_t)top * ff, shared, lane, vec != 0, s);
  }
#pragma unroll
  for (int r = 0; r < 4; ++r) s[r] = wave_sum(s[r]);
  if (lane < 4 && n0 + lane < width) {
    float v = lane == 0 ? s[0] : lane == 1 ? s[1] : lane == 2 ? s[2] : s[3];
    if (coef != 0.f) v += coef * to_f32(x[(size_t)t * ldx + n0 + lane]);
    out[(size_t)t * width + n0 + lane] = from_f32<TA>(v);
  }
}

extern "C" int ra_moe_gate_up_chosen(const void* x, int ldx, const void* w_gate_up, const int* ids, const float* weights,
                                     const float* shared_logit, int ld_logit, void* act, int act_dtype, int n_tokens,
                                     int top, int experts, int ff, int shared, int width, hipStream_t stream) {
  RA_CHECK(n_tokens > 0 && top > 0 && experts > 0 && ff > 0 && shared >= 0 && width > 0 && ldx >= width,
           "moe_gate_up_chosen: %d tokens, %d of %d experts of %d x %d, shared %d", n_tokens, top, experts, ff, width, shared);
  const long pairs = (long)n_tokens * (top + (shared > 0 ? 1 : 0));
  RA_CHECK(pairs <= 65535, "moe_gate_up_chosen: %ld pairs in one launch", pairs);
  const int vec = (width % 8 == 0 && ldx % 8 == 0 && ((uintptr_t)x % 16) == 0 && ((uintptr_t)w_gate_up % 16) == 0) ? 1 : 0;
  const int rows = ff > shared ? ff : shared;
  dim3 grid((rows + MOE_ROWS - 1) / MOE_ROWS, (unsigned)pairs);
  if (act_dtype == RA_F32)
    moe_gate_up_chosen_kernel<float><<<grid, 256, 0, stream>>>((const float*)x, ldx, (const float*)w_gate_up, ids, weights,
                                                               shared_logit, ld_logit, (float*)act, ff, shared, experts,
                                                               width, top, 0);
  else if (act_dtype == RA_BF16)
    moe_gate_up_chosen_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)x, ldx, (const bf16_t*)w_gate_up, ids,
                                                                weights, shared_logit, ld_logit, (bf16_t*)act, ff, shared,
                                                                experts, width, top, vec);
  else
    return ra_fail("moe_gate_up_chosen: unknown dtype tag %d", act_dtype);
  RA_LAUNCH_CHECK("moe_gate_up_chosen");
  return 0;
}

extern "C" int ra_moe_down_gated_chosen(const void* act, const void* w_down, const int* ids, const float* weights,
                                        const void* x, int ldx, void* out, int act_dtype, int n_tokens, int top,
                                        int experts, int ff, int shared, int width, hipStream_t stream) {
  RA_CHECK(n_tokens > 0 && top > 0 && experts > 0 && ff > 0 && shared >= 0 && width > 0 && ldx >= width,
           "moe_down_gated_chosen: %d tokens, %d of %d experts of %d x %d, shared %d", n_tokens, top, experts, ff, width, shared);
  RA_CHECK(n_tokens <= 65535, "moe_down_gated_chosen: %d tokens in one launch", n_tokens);
  RA_CHECK(act != nullptr && out != nullptr && x != nullptr, "moe_down_gated_chosen: act, x and out are given");
  const int vec = (ff % 8 == 0 && shared % 8 == 0 && ((uintptr_t)act % 16) == 0 && ((uintptr_t)w_down % 16) == 0) ? 1 : 0;
  dim3 grid((width + MOE_ROWS - 1) / MOE_ROWS, n_tokens);
  if (act_dtype == RA_F32)
    moe_down_gated_chosen_kernel<float><<<grid, 256, 0, stream>>>((const float*)act, (const float*)w_down, ids, weights,
                                                                  (const float*)x, ldx, (float*)out, ff, shared, width,
                                                                  experts, top, 0);
  else if (act_dtype == RA_BF16)
    moe_down_gated_chosen_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)act, (const bf16_t*)w_down, ids, weights,
                                                                   (const bf16_t*)x, ldx, (bf16_t*)out, ff, shared, width,
                                                                   experts, top, vec);
  else
    return ra_fail("moe_down_gated_chosen: unknown dtype tag %d", act_dtype);
  RA_LAUNCH_CHECK("moe_down_gated_chosen");
  return 0;
}

// ---------------------------------------------------------------------------
// No router: an integer table [vocabulary, top] gives each token id its experts; each weighs 1 / top.
// ---------------------------------------------------------------------------
__global__ void moe_table_route_kernel(const int* __restrict__ token_ids, const int* __restrict__ table, int top,
                                       int* __restrict__ ids, float* __restrict__ weights, long total) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const long t = i / top;
  const int j = (int)(i - t * top);
  ids[i] = table[(size_t)token_ids[t] * top + j];
  weights[i] = 1.f / (float)top;
}

extern "C" int ra_moe_table_route(const int* token_ids, const int* table, int top, int* ids, float* weights,
                                  int n_tokens, hipStream_t stream) {
  RA_CHECK(n_tokens > 0 && top > 0, "moe_table_route: %d tokens, %d choices", n_tokens, top);
  const long total = (long)n_tokens * top;
  moe_table_route_kernel<<<(unsigned)((total + 255) / 256), 256, 0, stream>>>(token_ids, table, top, ids, weights, total);
  RA_LAUNCH_CHECK("moe_table_route");
  return 0;
}
