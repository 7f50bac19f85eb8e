// Recurrent token mixers: a matrix memory with exponential gates and a gated delta rule, both a float matrix
// state [key_dim, value_dim] a head that is carried from token to token, and the row kernels around them
// (gate preparation, the short causal filter with its unit norms, the per-head norm and output gate, the mean of
// several mixers' normed outputs). Everything here computes in float whatever the activations' type.
//
// The scans. A column of the state (one value index) evolves on its own given the token's k, q and gates, so
// the columns are spread over lanes, waves and workgroups and every wave walks the request's tokens in order:
// R lanes share a column, each holding a run of NPL of its elements; a wave holds 64 / R columns. The two dot products a token needs (with k or n, and with q) are sums over a lane's elements
// and a butterfly over the R lanes. The next token's operands are asked for before the current token's
// arithmetic. The state of a request lives in its slot in the waves' own order, [NPL][64] floats a wave, so
// that loading and storing it are whole lines; nothing else reads it.
#include "common.h"
#include "reinfer_hip.h"

namespace {

struct ScanGeom {
  int R, NPL, CPW, waves;      // lanes a column, elements a lane, columns a wave, waves a head
  int wave_floats;             // floats of state a wave
};

// kind 0: matrix memory (S, the normaliser n once a wave, the running maximum m); kind 1: delta rule (S);
// kind 2: wkv (S); kind 3: a memory that fades by a constant a head (S)
bool scan_geom(int kind, int dk, int dv, ScanGeom* g) {
  if (dk <= 0 || dv <= 0 || dk > 512) return false;
  // at most 8 elements a lane: the per-token chain of multiply-adds stays short, and a head has enough waves to
  // spread over the chip when one request's prompt is all there is
  g->R = dk <= 32 ? 8 : dk <= 128 ? 16 : dk <= 256 ? 32 : 64;
  const int per = (dk + g->R - 1) / g->R;
  g->NPL = per <= 2 ? 2 : per <= 4 ? 4 : 8;
  g->CPW = RA_WAVE / g->R;
  g->waves = (dv + g->CPW - 1) / g->CPW;
  g->wave_floats = g->NPL * RA_WAVE + (kind == 0 ? g->NPL * g->R + 4 : 0);
  return true;
}

// Sum over runs of R neighbouring lanes, every lane of a run getting the sum. Inside a row of 16 lanes the
// exchanges are DPP operands of the adds (pairs, quads, the mirrored half row and row); only beyond 16 lanes does
// a value travel through the LDS crossbar.
template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}
template <int R>
__device__ __forceinline__ float group_sum(float v) {
  v += dpp_move<0xB1>(v);                    // quad_perm [1, 0, 3, 2]
  v += dpp_move<0x4E>(v);                    // quad_perm [2, 3, 0, 1]
  v += dpp_move<0x141>(v);                   // row_half_mirror: the other quad of the 8
  if (R >= 16) v += dpp_move<0x140>(v);      // row_mirror: the other half of the 16
  if (R >= 32) v += __shfl_xor(v, 16, RA_WAVE);
  if (R >= 64) v += __shfl_xor(v, 32, RA_WAVE);
  return v;
}

__device__ __forceinline__ float softplus_f(float x) { return x > 20.f ? x : log1pf(expf(x)); }
__device__ __forceinline__ float logsigmoid_f(float x) { return -softplus_f(-x); }

// ---------------------------------------------------------------------------
// The scan of either mixer. A workgroup (up to 4 waves: 32 or 8 columns of one head of one request) walks the
// request's tokens in chunks: the chunk's k and q rows of the head (as floats, q scaled), the v entries of the
// workgroup's columns and the two gate values a token are fetched into registers while the chunk before is
// computed, written to LDS behind it, and read from there token by token (a lane's NPL elements of k and of q
// are one run of LDS, rows padded so that the 16-byte reads of a wave fall on different banks). One barrier a
// chunk; every wave of the workgroup takes part in the staging, also those past the head's last column.
//
// Matrix memory (MEMORY): gt[t, j H + h], j = 0, 1, 2: keep = exp(b + m - m'), take = exp(a - m') and exp(-m') with
// m' = max(b + m, a) the running maximum of the log gates (all three prepared below, where the maximum is kept)
//   S <- keep S + take k v^T;  n <- keep n + take k;  o = S^T q / (max(|n . q|, exp(-m')) + eps)
// Gated delta rule: gt[t, h] = beta, gt[t, H + h] = decay g (prepared below).
//   S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q
// computed from the state before the decay: a = S^T k, b = S^T q, kq = k . q in one butterfly, then
// u = beta (v - g a), o = g b + u kq, S <- g S + k u.
// A memory that fades by a constant (DECAY): no gates; q, k and v pass silu as they are staged (float);
//   S <- head_decay[h] S + k v^T;  o = S^T q   (the read-out sees the token's own write)
// ---------------------------------------------------------------------------
#define SCAN_KQ_REGS 8         // k (and q) values a thread fetches for a chunk
#define SCAN_V_REGS 2
#define SCAN_CHUNK_MAX 16
#define SCAN_LDS_FLOATS 6144   // of one of the two buffers

enum { SCAN_DELTA = 0, SCAN_MEMORY = 1, SCAN_WKV = 2, SCAN_DECAY = 3 };

struct ScanArgs {
  const void* q; const void* k; const void* v;     // column 0 of each in row 0; rows ld elements apart
  int ld;
  int q_heads;                                       // heads of q and k (value heads share them in equal runs)
  const float* gates;                                // [T, NG H], NG = 3 (matrix memory) or 2 (delta rule)
  float* state; long slot_stride;
  const int* cu_tokens; const int* state_slots; const int* fresh;
  int H, dk, dv, waves_per_head, wave_floats, chunk;
  float q_scale, denom_eps;
  float* out;
  // wkv: the decays' pre-activations, float [T, H dk] with rows ldw apart, their bias w0 [H dk] and the bonus u [H dk]
  const float* w; int ldw; const float* w0; const float* u;
  const float* head_decay;                           // the fading memory: one factor a head
};

template <typename TA, int R, int NPL, int MODE>
__global__ __launch_bounds__(256) void scan_kernel(ScanArgs p) {
  constexpr bool MEMORY = MODE == SCAN_MEMORY, WKV = MODE == SCAN_WKV, DECAY = MODE == SCAN_DECAY;
  constexpr int CPW = RA_WAVE / R;
  constexpr int PITCH = NPL + 4;                     // floats of a lane's run of k (or q) in LDS, padded
  constexpr int NG = MEMORY ? 3 : (WKV || DECAY) ? 0 : 2;       // gate values a token
  constexpr int NGD = NG ? NG : 1;
  constexpr int NV = WKV ? 3 : 2;                    // vectors over the key size a token: k, q and, for wkv, the decay
  extern __shared__ __attribute__((aligned(16))) float lds[];
  const int seq = blockIdx.x, head = blockIdx.y;
  const int tid = threadIdx.x, nthreads = blockDim.x;
  const int lane = tid & (RA_WAVE - 1);
  const int waves = nthreads / RA_WAVE;
  const int cols = waves * CPW;                      // columns of this workgroup
  const int w = blockIdx.z * waves + tid / RA_WAVE;
  const bool active = w < p.waves_per_head;
  const int c = lane / R, r = lane % R;
  const int col = w * CPW + c;
  const bool col_ok = active && col < p.dv;
  const int first = p.cu_tokens[seq], last = p.cu_tokens[seq + 1];
  const int slot = p.state_slots[seq];
  const int ow = p.H * p.dv;
  const int H = p.H, dk = p.dk, dv = p.dv, CT = p.chunk;
  if (slot < 0) {                                    // a padding row: no state, a defined result
    if (col_ok && r == 0)
      for (int t = first; t < last; ++t) p.out[(size_t)t * ow + head * dv + col] = 0.f;
    return;
  }
  if (first >= last) return;
  // LDS: two buffers of [CT][NV][R][PITCH] k, q (and the decay), [CT][cols] v, [CT][NG] gates
  const int kq_floats = CT * NV * R * PITCH, v_floats = CT * cols;
  const int buf_floats = kq_floats + v_floats + CT * NG;
  const int qh = head / (H / p.q_heads);
  const TA* qg = (const TA*)p.q + (size_t)qh * dk;
  const TA* kg = (const TA*)p.k + (size_t)qh * dk;
  const TA* vg = (const TA*)p.v + (size_t)head * dv + (size_t)blockIdx.z * cols;
  const int v_left = dv - blockIdx.z * cols;         // columns of this workgroup that exist
  float fk[SCAN_KQ_REGS], fq[SCAN_KQ_REGS], fw[WKV ? SCAN_KQ_REGS : 1], fv[SCAN_V_REGS], fg = 0.f;
  const float* wg = WKV ? p.w + (size_t)head * dk : nullptr;
  const float* w0 = WKV ? p.w0 + (size_t)head * dk : nullptr;
  int kq_w[WKV ? SCAN_KQ_REGS : 1];                  // the decay's place: rows of its own pitch, the bias by element
  // what this thread fetches for a chunk is the same for every chunk: token (of the chunk), offset behind the
  // chunk's first row, and place in LDS are worked out once
  int kq_t[SCAN_KQ_REGS], kq_g[SCAN_KQ_REGS], kq_l[SCAN_KQ_REGS];
  bool kq_e[SCAN_KQ_REGS];
#pragma unroll
  for (int j = 0; j < SCAN_KQ_REGS; ++j) {
    const int idx = tid + j * nthreads;
    const int t = idx / (R * NPL), e = idx - t * (R * NPL);      // e runs over the lanes' runs: past dk they hold zeros
    kq_t[j] = t < CT ? t : SCAN_CHUNK_MAX;           // past the chunk: never fetched, never stored
    kq_e[j] = e < dk;
    kq_g[j] = t * p.ld + e;
    kq_l[j] = t * NV * R * PITCH + (e / NPL) * PITCH + (e % NPL);
    if (WKV) kq_w[j] = e;
  }
  int v_t[SCAN_V_REGS], v_g[SCAN_V_REGS];
#pragma unroll
  for (int j = 0; j < SCAN_V_REGS; ++j) {
    const int idx = tid + j * nthreads;
    const int t = idx / cols, cc = idx - t * cols;
    v_t[j] = (t < CT && cc < v_left) ? t : SCAN_CHUNK_MAX;
    v_g[j] = t * p.ld + cc;
  }
  const int g_t = tid < NG * CT ? tid / NGD : SCAN_CHUNK_MAX;
  const int g_g = g_t * NG * H + (tid - g_t * NG) * H + head;
  auto fetch = [&](int t0) {                         // chunk starting at token t0 -> registers
    const int n = min(CT, last - t0);
    const size_t row0 = (size_t)t0 * p.ld;
#pragma unroll
    for (int j = 0; j < SCAN_KQ_REGS; ++j) {
      fk[j] = fq[j] = 0.f;
      if (kq_t[j] < n && kq_e[j]) {
        fk[j] = to_f32(kg[row0 + kq_g[j]]);
        fq[j] = to_f32(qg[row0 + kq_g[j]]) * p.q_scale;
        if (DECAY) {                                   // silu through the hardware's exponential and reciprocal
          fk[j] = __fdividef(fk[j], 1.f + __expf(-fk[j]));
          fq[j] = __fdividef(fq[j], 1.f + __expf(-fq[j]));
        }
      }
      if (WKV) {                                     // the decay exp(-exp(z + w0)), float from its pre-activation on
        fw[j] = 0.f;
        if (kq_t[j] < n && kq_e[j])
          fw[j] = expf(-expf(wg[(size_t)(t0 + kq_t[j]) * p.ldw + kq_w[j]] + w0[kq_w[j]]));
      }
    }
#pragma unroll
    for (int j = 0; j < SCAN_V_REGS; ++j) {
      fv[j] = v_t[j] < n ? to_f32(vg[row0 + v_g[j]]) : 0.f;
      if (DECAY) fv[j] = __fdividef(fv[j], 1.f + __expf(-fv[j]));
    }
    fg = (NG && g_t < n) ? p.gates[(size_t)t0 * NG * H + g_g] : 0.f;
  };
  auto stage = [&](float* buf) {                     // registers -> LDS
#pragma unroll
    for (int j = 0; j < SCAN_KQ_REGS; ++j) {
      if (kq_t[j] < SCAN_CHUNK_MAX) {
        buf[kq_l[j]] = fk[j];
        buf[kq_l[j] + R * PITCH] = fq[j];
        if (WKV) buf[kq_l[j] + 2 * R * PITCH] = fw[j];
      }
    }
#pragma unroll
    for (int j = 0; j < SCAN_V_REGS; ++j) {
      const int idx = tid + j * nthreads;
      if (idx < v_floats) buf[kq_floats + idx] = fv[j];
    }
    if (NG && tid < NG * CT) buf[kq_floats + v_floats + tid] = fg;
  };
  float* st = p.state + (size_t)slot * p.slot_stride + (size_t)(head * p.waves_per_head + (active ? w : 0)) * p.wave_floats;
  const bool zero = p.fresh[seq] != 0;
  const float fade = DECAY ? p.head_decay[head] : 1.f;
  float S[NPL], nrm[NPL], bonus[NPL];
#pragma unroll
  for (int i = 0; i < NPL; ++i) {
    S[i] = (zero || !active) ? 0.f : st[i * RA_WAVE + lane];
    nrm[i] = 0.f;
    bonus[i] = (WKV && r * NPL + i < dk) ? p.u[(size_t)head * dk + r * NPL + i] : 0.f;
    if (MEMORY && !zero && active) nrm[i] = st[NPL * RA_WAVE + i * R + r];
  }
  fetch(first);
  stage(lds);
  __syncthreads();
  int which = 0;
  for (int t0 = first; t0 < last; t0 += CT) {
    const bool more = t0 + CT < last;
    if (more) fetch(t0 + CT);
    const float* buf = lds + (size_t)which * buf_floats;
    const int n = min(CT, last - t0);
    if (active) {
      const int vcol = (tid / RA_WAVE) * CPW + c;
      struct Operands { float k[NPL], q[NPL], w[WKV ? NPL : 1], v, g0, g1, g2; };
      auto read = [&](int tt, Operands& x) {         // a token's operands out of LDS
        const float* kp = buf + (size_t)tt * NV * R * PITCH + r * PITCH;
        const float* qp = kp + R * PITCH;
#pragma unroll
        for (int i = 0; i < NPL; ++i) { x.k[i] = kp[i]; x.q[i] = qp[i]; }
        if (WKV) {
#pragma unroll
          for (int i = 0; i < NPL; ++i) x.w[i] = qp[R * PITCH + i];
        }
        x.v = buf[kq_floats + tt * cols + vcol];
        x.g0 = NG ? buf[kq_floats + v_floats + NG * tt] : 0.f;
        x.g1 = NG ? buf[kq_floats + v_floats + NG * tt + 1] : 0.f;
        x.g2 = MEMORY ? buf[kq_floats + v_floats + NG * tt + 2] : 0.f;
      };
      auto step = [&](int tt, const Operands& x) {   // one token: the state moves on, the read-out is stored
        float o;
        if (MEMORY) {
          const float keep = x.g0, take = x.g1;
          float ps[2] = {0.f, 0.f}, pn[2] = {0.f, 0.f};
#pragma unroll
          for (int i = 0; i < NPL; ++i) {
            const float tk = take * x.k[i];
            nrm[i] = keep * nrm[i] + tk;
            S[i] = keep * S[i] + tk * x.v;
            ps[i & 1] += S[i] * x.q[i];
            pn[i & 1] += nrm[i] * x.q[i];
          }
          const float s1 = group_sum<R>(ps[0] + ps[1]);
          const float s2 = group_sum<R>(pn[0] + pn[1]);
          o = __fdividef(s1, fmaxf(fabsf(s2), x.g2) + p.denom_eps);      // a reciprocal and a product: within an ulp or two
        } else if (WKV) {
          // o = (S + diag(u) k v^T)^T q with the bonus for this token alone; then S <- diag(w) S + k v^T
          float po[2] = {0.f, 0.f};
#pragma unroll
          for (int i = 0; i < NPL; ++i) {
            const float kv = x.k[i] * x.v;
            po[i & 1] += x.q[i] * (S[i] + bonus[i] * kv);
            S[i] = x.w[i] * S[i] + kv;
          }
          o = group_sum<R>(po[0] + po[1]);
        } else if (DECAY) {
          float po[2] = {0.f, 0.f};
#pragma unroll
          for (int i = 0; i < NPL; ++i) {
            S[i] = fade * S[i] + x.k[i] * x.v;
            po[i & 1] += S[i] * x.q[i];
          }
          o = group_sum<R>(po[0] + po[1]);
        } else {
          float pa[2] = {0.f, 0.f}, pb[2] = {0.f, 0.f}, pkq[2] = {0.f, 0.f};
#pragma unroll
          for (int i = 0; i < NPL; ++i) {
            pa[i & 1] += S[i] * x.k[i];
            pb[i & 1] += S[i] * x.q[i];
            pkq[i & 1] += x.k[i] * x.q[i];
          }
          const float sa = group_sum<R>(pa[0] + pa[1]);
          const float sb = group_sum<R>(pb[0] + pb[1]);
          const float skq = group_sum<R>(pkq[0] + pkq[1]);
          const float u = x.g0 * (x.v - x.g1 * sa);
#pragma unroll
          for (int i = 0; i < NPL; ++i) S[i] = x.g1 * S[i] + x.k[i] * u;
          o = x.g1 * sb + u * skq;
        }
        if (col_ok && r == 0) p.out[(size_t)(t0 + tt) * ow + head * dv + col] = o;
      };
      // two sets of operand registers take turns: a token's operands are asked for before the arithmetic of the
      // token before it, and nothing is copied
      Operands xa, xb;
      read(0, xa);
      for (int tt = 0; tt < n; tt += 2) {
        if (tt + 1 < n) read(tt + 1, xb);
        step(tt, xa);
        if (tt + 1 < n) {
          if (tt + 2 < n) read(tt + 2, xa);
          step(tt + 1, xb);
        }
      }
    }
    if (more) stage(lds + (size_t)(which ^ 1) * buf_floats);
    __syncthreads();
    which ^= 1;
  }
  if (!active) return;
#pragma unroll
  for (int i = 0; i < NPL; ++i) {
    st[i * RA_WAVE + lane] = S[i];
    if (MEMORY && c == 0) st[NPL * RA_WAVE + i * R + r] = nrm[i];
  }
}

// The matrix memory's gates. z [T, 2 H] holds the pre-activations (input | forget); with a = cap tanh((z_i + bias) / cap)
// and b = log sigmoid(cap tanh((z_f + bias) / cap)) the running maximum is m_t = max(b_t + m_{t-1}, a_t), a chain over
// the request's tokens. The map m -> max(b + m, a) is the pair (a, b), and two such maps compose to
// (max(a1 + b2, a2), b1 + b2), so a workgroup a (request, head) takes 256 tokens at a time through a prefix scan
// in LDS. g3 [T, 3 H] gets keep = exp(b + m_{t-1} - m_t), take = exp(a - m_t) and exp(-m_t). The maximum itself
// is kept in the request's state at `m_off` floats behind the head's first float (0 at a request's start).
__global__ __launch_bounds__(256) void matrix_memory_gate_scan_kernel(
    const float* __restrict__ z, const float* __restrict__ bias, float cap, float* __restrict__ g3,
    float* __restrict__ state, long slot_stride, long head_floats, long m_off, const int* __restrict__ cu_tokens,
    const int* __restrict__ state_slots, const int* __restrict__ fresh, int H) {
  __shared__ float sA[256], sB[256];
  const int seq = blockIdx.x, head = blockIdx.y, tid = threadIdx.x;
  const int first = cu_tokens[seq], last = cu_tokens[seq + 1];
  const int slot = state_slots[seq];
  if (slot < 0 || first >= last) return;       // the scan writes zeros for a padding row without reading its gates
  float* mp = state + (size_t)slot * slot_stride + (size_t)head * head_floats + m_off;
  float m_run = fresh[seq] != 0 ? 0.f : *mp;
  for (int t0 = first; t0 < last; t0 += 256) {
    const int t = t0 + tid;
    const bool valid = t < last;
    float a = -INFINITY, b = 0.f;              // the identity map for rows past the end
    if (valid) {
      float zi = z[(size_t)t * 2 * H + head] + bias[head];
      float zf = z[(size_t)t * 2 * H + H + head] + bias[H + head];
      if (cap > 0.f) { zi = cap * tanhf(zi / cap); zf = cap * tanhf(zf / cap); }
      a = zi;
      b = logsigmoid_f(zf);
    }
    float A = a, B = b;
    sA[tid] = A;
    sB[tid] = B;
    __syncthreads();
    for (int off = 1; off < 256; off <<= 1) {
      float A1 = -INFINITY, B1 = 0.f;
      const bool has = tid >= off;
      if (has) { A1 = sA[tid - off]; B1 = sB[tid - off]; }
      __syncthreads();
      if (has) {                               // the earlier map first, then this one
        A = fmaxf(A1 + B, A);
        B = B1 + B;
        sA[tid] = A;
        sB[tid] = B;
      }
      __syncthreads();
    }
    const float m_t = fmaxf(B + m_run, A);
    const float m_prev = tid == 0 ? m_run : fmaxf(sB[tid - 1] + m_run, sA[tid - 1]);
    if (valid) {
      float* o = g3 + (size_t)t * 3 * H + head;
      o[0] = expf(b + m_prev - m_t);
      o[H] = expf(a - m_t);
      o[2 * H] = expf(-m_t);
    }
    const int end = min(255, last - 1 - t0);
    const float m_end = fmaxf(sB[end] + m_run, sA[end]);
    __syncthreads();                           // before the next round overwrites the maps
    m_run = m_end;
  }
  if (tid == 0) *mp = m_run;
}

// gb[t, h] <- sigmoid(b);  gb[t, H + h] <- exp(-exp(A_log[h]) softplus(a + dt_bias[h])), in place
__global__ void delta_rule_gates_kernel(float* __restrict__ gb, const float* __restrict__ a_log,
                                        const float* __restrict__ dt_bias, int H, long n) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const int j = (int)(i % (2 * H));
  const float z = gb[i];
  if (j < H) gb[i] = 1.f / (1.f + expf(-z));
  else gb[i] = expf(-expf(a_log[j - H]) * softplus_f(z + dt_bias[j - H]));
}

// ---------------------------------------------------------------------------
// The delta rule's inputs: per channel a causal filter over time (taps weights, the last one the current
// token's; rows before the step's portion come from the request's tail of taps - 1 rows, zeros at a request's
// start), silu, and for the heads of q and k the unit norm x / sqrt(sum x^2 + eps) (q also times q_scale).
// One wave a (token, head of q, k or v); float results [T, C].
// ---------------------------------------------------------------------------
#define PREP_WAVES 4
#define PREP_HOLD 8          // values a lane keeps: heads up to 512 wide
template <typename TA>
__global__ void delta_rule_prepare_kernel(const TA* __restrict__ proj, int ld, const float* __restrict__ filt,
                                          const float* __restrict__ state, long slot_stride, long tail_off,
                                          const int* __restrict__ seq_of_token, const int* __restrict__ cu_tokens,
                                          const int* __restrict__ state_slots, const int* __restrict__ fresh, int G,
                                          int dk, int H, int dv, int taps, float unit_eps, float q_scale,
                                          float* __restrict__ qkv, int T) {
  const int lane = threadIdx.x & (RA_WAVE - 1);
  const int units = 2 * G + H;
  const long idx = (long)blockIdx.x * PREP_WAVES + threadIdx.x / RA_WAVE;
  if (idx >= (long)T * units) return;
  const int t = (int)(idx / units), unit = (int)(idx % units);
  const int C = 2 * G * dk + H * dv;
  const bool is_v = unit >= 2 * G;
  const int width = is_v ? dv : dk;
  const int base = is_v ? 2 * G * dk + (unit - 2 * G) * dv : unit * dk;
  const int seq = seq_of_token[t];
  const int first = cu_tokens[seq];
  const int slot = state_slots[seq];
  float* o = qkv + (size_t)t * C + base;
  if (slot < 0) {
    for (int e = lane; e < width; e += RA_WAVE) o[e] = 0.f;
    return;
  }
  const bool zero = fresh[seq] != 0;
  const float* tail = state + (size_t)slot * slot_stride + tail_off;      // [taps - 1, C], oldest first
  float y[PREP_HOLD];
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < PREP_HOLD; ++j) {
    const int e = lane + j * RA_WAVE;
    y[j] = 0.f;
    if (e < width) {
      const int ch = base + e;
      float acc = 0.f;
      for (int p = 0; p < taps; ++p) {
        const int rel = t - first - (taps - 1) + p;        // row of the portion, negative: a row of the tail
        float x;
        if (rel >= 0) x = to_f32(proj[(size_t)(first + rel) * ld + ch]);
        else x = zero ? 0.f : tail[(size_t)(taps - 1 + rel) * C + ch];
        acc += filt[(size_t)ch * taps + p] * x;
      }
      acc = acc / (1.f + expf(-acc));
      y[j] = acc;
      ss += acc * acc;
    }
  }
  float f = 1.f;
  if (!is_v) {
    ss = wave_sum(ss);
    f = 1.f / sqrtf(ss + unit_eps);
    if (unit < G) f *= q_scale;
  }
#pragma unroll
  for (int j = 0; j < PREP_HOLD; ++j) {
    const int e = lane + j * RA_WAVE;
    if (e < width) o[e] = y[j] * f;
  }
}

// The tail moves on: after a portion of n rows it holds the last taps - 1 rows of (old tail, portion).
// One thread a (request, channel) reads what it needs before it writes.
#define MAX_TAPS 16
template <typename TA>
__global__ void delta_rule_tail_kernel(const TA* __restrict__ proj, int ld, float* __restrict__ state,
                                       long slot_stride, long tail_off, const int* __restrict__ cu_tokens,
                                       const int* __restrict__ state_slots, const int* __restrict__ fresh, int C,
                                       int taps) {
  const int seq = blockIdx.y;
  const int ch = blockIdx.x * blockDim.x + threadIdx.x;
  if (ch >= C) return;
  const int slot = state_slots[seq];
  if (slot < 0) return;
  const int first = cu_tokens[seq], n = cu_tokens[seq + 1] - first;
  const bool zero = fresh[seq] != 0;
  float* tail = state + (size_t)slot * slot_stride + tail_off;
  float keep[MAX_TAPS];
  for (int j = 0; j < taps - 1; ++j) {
    const int rel = n - (taps - 1) + j;
    if (rel >= 0) keep[j] = to_f32(proj[(size_t)(first + rel) * ld + ch]);
    else keep[j] = zero ? 0.f : tail[(size_t)(j + n) * C + ch];
  }
  for (int j = 0; j < taps - 1; ++j) tail[(size_t)j * C + ch] = keep[j];
}

// ---------------------------------------------------------------------------
// out[t, h, :] = read[t, h, :] / rms(read[t, h, :]) * weight * act(gate[t, h, :]); act = sigmoid or silu;
// weight is [heads * dv] (w_head_stride = dv) or one [dv] for all heads (0). One wave a (token, head).
// ---------------------------------------------------------------------------
template <typename TA>
__global__ void head_norm_gate_kernel(const float* __restrict__ read, const float* __restrict__ weight,
                                      int w_head_stride, const TA* __restrict__ gate, int ldg, int silu, float eps,
                                      int H, int dv, TA* __restrict__ out, long n_units) {
  const int lane = threadIdx.x & (RA_WAVE - 1);
  const long idx = (long)blockIdx.x * (blockDim.x / RA_WAVE) + threadIdx.x / RA_WAVE;
  if (idx >= n_units) return;
  const long t = idx / H;
  const int h = (int)(idx % H);
  const float* x = read + (size_t)t * H * dv + (size_t)h * dv;
  float ss = 0.f;
  for (int e = lane; e < dv; e += RA_WAVE) ss += x[e] * x[e];
  ss = wave_sum(ss);
  const float rstd = 1.f / sqrtf(ss / (float)dv + eps);
  const TA* g = gate + (size_t)t * ldg + (size_t)h * dv;
  const float* wt = weight + (size_t)h * w_head_stride;
  TA* o = out + (size_t)t * H * dv + (size_t)h * dv;
  for (int e = lane; e < dv; e += RA_WAVE) {
    const float z = to_f32(g[e]);
    const float s = 1.f / (1.f + expf(-z));
    o[e] = from_f32<TA>(x[e] * rstd * wt[e] * (silu ? z * s : s));
  }
}

// The same for heads wider than a wave can walk quickly (one "head" as wide as all read-outs together): a workgroup a
// (token, head), every thread up to HNG_CHUNKS runs of eight neighbouring elements in registers, 16-byte accesses.
#define HNG_CHUNKS 4
template <typename TA>
__global__ void head_norm_gate_wide_kernel(const float* __restrict__ read, const float* __restrict__ weight,
                                           int w_head_stride, const TA* __restrict__ gate, int ldg, int silu, float eps,
                                           int H, int dv, TA* __restrict__ out) {
  __shared__ float red[17];
  const long t = blockIdx.x / H;
  const int h = blockIdx.x % H;
  const float* x = read + (size_t)t * H * dv + (size_t)h * dv;
  const TA* g = gate + (size_t)t * ldg + (size_t)h * dv;
  const float* wt = weight + (size_t)h * w_head_stride;
  TA* o = out + (size_t)t * H * dv + (size_t)h * dv;
  float a[HNG_CHUNKS][8], w[HNG_CHUNKS][8], z[HNG_CHUNKS][8];
  float ss = 0.f;
#pragma unroll
  for (int r = 0; r < HNG_CHUNKS; ++r) {
    const int c = (threadIdx.x + r * blockDim.x) * 8;
#pragma unroll
    for (int e = 0; e < 8; ++e) a[r][e] = 0.f;
    if (c >= dv) continue;
    Vec8<float>::load(x + c, a[r]);
    Vec8<float>::load(wt + c, w[r]);
    Vec8<TA>::load(g + c, z[r]);
#pragma unroll
    for (int e = 0; e < 8; ++e) ss += a[r][e] * a[r][e];
  }
  const float total = block_sum(ss, red);
  const float rstd = 1.f / sqrtf(total / (float)dv + eps);
#pragma unroll
  for (int r = 0; r < HNG_CHUNKS; ++r) {
    const int c = (threadIdx.x + r * blockDim.x) * 8;
    if (c >= dv) continue;
    float v[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float s = 1.f / (1.f + expf(-z[r][e]));
      v[e] = a[r][e] * rstd * w[r][e] * (silu ? z[r][e] * s : s);
    }
    Vec8<TA>::store(o + c, v);
  }
}

// ---------------------------------------------------------------------------
// y[t, :] = (1 / n) sum_i x_i[t, :] / rms(x_i[t, :]) * w_i;  out = y, or resid += scale * y. One workgroup a row.
// ---------------------------------------------------------------------------
#define MEAN_MAX 4
struct MeanInputs {
  const void* x[MEAN_MAX];
  const float* w[MEAN_MAX];
};
template <typename TA, int N>
__global__ void normed_mean_kernel(MeanInputs in, float eps, int h, TA* __restrict__ out, float* __restrict__ resid,
                                   float scale) {
  __shared__ float red[N][17];
  const size_t row = (size_t)blockIdx.x * h;
  const int lane = threadIdx.x & (RA_WAVE - 1), wave = threadIdx.x / RA_WAVE, nwave = blockDim.x / RA_WAVE;
  float ss[N];
#pragma unroll
  for (int i = 0; i < N; ++i) ss[i] = 0.f;
  for (int e = threadIdx.x; e < h; e += blockDim.x) {
#pragma unroll
    for (int i = 0; i < N; ++i) {
      const float v = to_f32(((const TA*)in.x[i])[row + e]);
      ss[i] += v * v;
    }
  }
#pragma unroll
  for (int i = 0; i < N; ++i) {
    ss[i] = wave_sum(ss[i]);
    if (lane == 0) red[i][wave] = ss[i];
  }
  __syncthreads();
  float rstd[N];
#pragma unroll
  for (int i = 0; i < N; ++i) {
    float t = 0.f;
    for (int w = 0; w < nwave; ++w) t += red[i][w];          // fixed order
    rstd[i] = 1.f / sqrtf(t / (float)h + eps) * (1.f / (float)N);
  }
  for (int e = threadIdx.x; e < h; e += blockDim.x) {
    float y = 0.f;
#pragma unroll
    for (int i = 0; i < N; ++i) y += to_f32(((const TA*)in.x[i])[row + e]) * rstd[i] * in.w[i][e];
    if (resid) resid[row + e] += scale * y;
    else out[row + e] = from_f32<TA>(y);
  }
}

}  // namespace

// ---------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------
extern "C" long ra_scan_state_floats(int kind, int heads, int key_dim, int value_dim) {
  ScanGeom g;
  if (heads <= 0 || !scan_geom(kind, key_dim, value_dim, &g)) return -1;
  return (long)heads * g.waves * g.wave_floats;
}

namespace {
struct ScanLaunch {
  dim3 grid;
  int threads, chunk;
  size_t lds;
};
ScanLaunch scan_launch(const ScanGeom& g, int n_seqs, int heads, int max_q_len, int vectors = 2) {
  const int wpb = g.waves < 4 ? g.waves : 4;           // waves a workgroup
  ScanLaunch L;
  L.threads = wpb * RA_WAVE;
  L.grid = dim3(n_seqs, heads, (g.waves + wpb - 1) / wpb);
  const int cols = wpb * g.CPW;
  const int per_token = vectors * g.R * (g.NPL + 4) + cols + 3;      // k and q (and decay) runs, the columns of v, up to 3 gate numbers
  int ct = SCAN_CHUNK_MAX;
  if (ct > SCAN_KQ_REGS * L.threads / (g.R * g.NPL)) ct = SCAN_KQ_REGS * L.threads / (g.R * g.NPL);
  if (max_q_len > 0 && ct > max_q_len) ct = max_q_len;      // a step of single tokens stages one token
  if (ct > SCAN_V_REGS * L.threads / cols) ct = SCAN_V_REGS * L.threads / cols;
  if (ct > SCAN_LDS_FLOATS / per_token) ct = SCAN_LDS_FLOATS / per_token;
  if (ct > L.threads / 3) ct = L.threads / 3;
  if (ct < 1) ct = 1;
  L.chunk = ct;
  L.lds = (size_t)2 * ((size_t)ct * per_token) * sizeof(float);
  return L;
}

template <typename TA, int MEMORY>
int scan_dispatch(const ScanGeom& g, const ScanLaunch& L, const ScanArgs& a, hipStream_t stream) {
#define RA_SCAN(R, NPL) scan_kernel<TA, R, NPL, MEMORY><<<L.grid, L.threads, L.lds, stream>>>(a)
#define RA_SCAN_N(R)                               \
  do {                                             \
    if (g.NPL == 2) RA_SCAN(R, 2);                 \
    else if (g.NPL == 4) RA_SCAN(R, 4);            \
    else RA_SCAN(R, 8);                            \
  } while (0)
  if (g.R == 8) RA_SCAN_N(8);
  else if (g.R == 16) RA_SCAN_N(16);
  else if (g.R == 32) RA_SCAN_N(32);
  else RA_SCAN_N(64);
#undef RA_SCAN_N
#undef RA_SCAN
  return 0;
}
}  // namespace

extern "C" int ra_matrix_memory_scan(const void* proj, int act_dtype, int ld, int q_off, int k_off, int v_off,
                                     const float* gates, float* gates3, const float* gate_bias, float* state,
                                     long slot_stride,
                                     const int* cu_tokens, const int* state_slots, const int* fresh, int n_seqs,
                                     int n_tokens, int max_q_len, int heads, int key_dim, int value_dim,
                                     float gate_cap, float q_scale, float denom_eps, float* out, hipStream_t stream) {
  RA_CHECK(n_seqs > 0 && n_tokens > 0 && heads > 0, "matrix_memory_scan: %d requests, %d tokens, %d heads", n_seqs,
           n_tokens, heads);
  ScanGeom g;
  RA_CHECK(scan_geom(0, key_dim, value_dim, &g), "matrix_memory_scan: heads of %d x %d (keys up to 512)", key_dim,
           value_dim);
  RA_CHECK(slot_stride >= (long)heads * g.waves * g.wave_floats, "matrix_memory_scan: a state slot of %ld floats, need %ld",
           slot_stride, (long)heads * g.waves * g.wave_floats);
  RA_CHECK(heads <= 65535, "matrix_memory_scan: %d heads in one launch", heads);
  RA_CHECK(act_dtype == RA_F32 || act_dtype == RA_BF16, "matrix_memory_scan: unknown dtype tag %d", act_dtype);
  // the running maximum lives where the first wave of each head has its spare floats
  matrix_memory_gate_scan_kernel<<<dim3(n_seqs, heads), 256, 0, stream>>>(
      gates, gate_bias, gate_cap, gates3, state, slot_stride, (long)g.waves * g.wave_floats,
      (long)g.NPL * RA_WAVE + (long)g.NPL * g.R, cu_tokens, state_slots, fresh, heads);
  RA_LAUNCH_CHECK("matrix_memory_gates");
  const ScanLaunch L = scan_launch(g, n_seqs, heads, max_q_len);
  const size_t es = act_dtype == RA_F32 ? 4 : 2;
  ScanArgs a = {};
  a.q = (const char*)proj + (size_t)q_off * es;
  a.k = (const char*)proj + (size_t)k_off * es;
  a.v = (const char*)proj + (size_t)v_off * es;
  a.ld = ld; a.q_heads = heads; a.gates = gates3; a.state = state; a.slot_stride = slot_stride;
  a.cu_tokens = cu_tokens; a.state_slots = state_slots; a.fresh = fresh;
  a.H = heads; a.dk = key_dim; a.dv = value_dim; a.waves_per_head = g.waves; a.wave_floats = g.wave_floats;
  a.chunk = L.chunk; a.q_scale = q_scale; a.denom_eps = denom_eps; a.out = out;
  if (act_dtype == RA_F32) scan_dispatch<float, SCAN_MEMORY>(g, L, a, stream);
  else scan_dispatch<bf16_t, SCAN_MEMORY>(g, L, a, stream);
  RA_LAUNCH_CHECK("matrix_memory_scan");
  return 0;
}

extern "C" int ra_delta_rule_prepare(const void* proj, int act_dtype, int ld, const float* filt, float* state,
                                     long slot_stride, long tail_off, const int* seq_of_token, const int* cu_tokens,
                                     const int* state_slots, const int* fresh, int n_seqs, int n_tokens,
                                     int key_heads, int key_dim, int heads, int value_dim, int taps, float unit_eps,
                                     float q_scale, float* qkv, hipStream_t stream) {
  RA_CHECK(n_seqs > 0 && n_tokens > 0 && heads > 0 && key_heads > 0, "delta_rule_prepare: %d requests, %d tokens",
           n_seqs, n_tokens);
  RA_CHECK(taps >= 1 && taps <= MAX_TAPS, "delta_rule_prepare: a filter of %d taps (1 to %d)", taps, MAX_TAPS);
  RA_CHECK(key_dim <= PREP_HOLD * RA_WAVE && value_dim <= PREP_HOLD * RA_WAVE,
           "delta_rule_prepare: heads of %d / %d (up to %d)", key_dim, value_dim, PREP_HOLD * RA_WAVE);
  const int C = 2 * key_heads * key_dim + heads * value_dim;
  RA_CHECK(slot_stride >= tail_off + (long)(taps - 1) * C, "delta_rule_prepare: a state slot of %ld floats", slot_stride);
  RA_CHECK(n_seqs <= 65535, "delta_rule_prepare: %d requests in one launch", n_seqs);
  const long units = (long)n_tokens * (2 * key_heads + heads);
  const unsigned blocks = (unsigned)((units + PREP_WAVES - 1) / PREP_WAVES);
  dim3 tail_grid((C + 255) / 256, n_seqs);
#define RA_DP(TA)                                                                                                   \
  do {                                                                                                              \
    delta_rule_prepare_kernel<TA><<<blocks, PREP_WAVES * RA_WAVE, 0, stream>>>(                                     \
        (const TA*)proj, ld, filt, state, slot_stride, tail_off, seq_of_token, cu_tokens, state_slots, fresh,       \
        key_heads, key_dim, heads, value_dim, taps, unit_eps, q_scale, qkv, n_tokens);                              \
    if (taps > 1)                                                                                                   \
      delta_rule_tail_kernel<TA><<<tail_grid, 256, 0, stream>>>((const TA*)proj, ld, state, slot_stride, tail_off,  \
                                                                cu_tokens, state_slots, fresh, C, taps);            \
  } while (0)
  if (act_dtype == RA_F32) RA_DP(float);
  else if (act_dtype == RA_BF16) RA_DP(bf16_t);
  else return ra_fail("delta_rule_prepare: unknown dtype tag %d", act_dtype);
#undef RA_DP
  RA_LAUNCH_CHECK("delta_rule_prepare");
  return 0;
}

extern "C" int ra_delta_rule_scan(const float* qkv, int ld, float* gates, const float* a_log, const float* dt_bias,
                                  float* state, long slot_stride, const int* cu_tokens, const int* state_slots,
                                  const int* fresh, int n_seqs, int n_tokens, int max_q_len, int heads, int key_heads,
                                  int key_dim, int value_dim, float* out, hipStream_t stream) {
  RA_CHECK(n_seqs > 0 && n_tokens > 0 && heads > 0 && key_heads > 0 && heads % key_heads == 0,
           "delta_rule_scan: %d requests, %d tokens, %d heads on %d key heads", n_seqs, n_tokens, heads, key_heads);
  ScanGeom g;
  RA_CHECK(scan_geom(1, key_dim, value_dim, &g), "delta_rule_scan: heads of %d x %d (keys up to 512)", key_dim, value_dim);
  RA_CHECK(slot_stride >= (long)heads * g.waves * g.wave_floats, "delta_rule_scan: a state slot of %ld floats, need %ld",
           slot_stride, (long)heads * g.waves * g.wave_floats);
  RA_CHECK(heads <= 65535, "delta_rule_scan: %d heads in one launch", heads);
  const long n = (long)n_tokens * 2 * heads;
  delta_rule_gates_kernel<<<(unsigned)((n + 255) / 256), 256, 0, stream>>>(gates, a_log, dt_bias, heads, n);
  RA_LAUNCH_CHECK("delta_rule_gates");
  const ScanLaunch L = scan_launch(g, n_seqs, heads, max_q_len);
  ScanArgs a = {};
  a.q = qkv;
  a.k = qkv + (size_t)key_heads * key_dim;
  a.v = qkv + (size_t)2 * key_heads * key_dim;
  a.ld = ld; a.q_heads = key_heads; a.gates = gates; a.state = state; a.slot_stride = slot_stride;
  a.cu_tokens = cu_tokens; a.state_slots = state_slots; a.fresh = fresh;
  a.H = heads; a.dk = key_dim; a.dv = value_dim; a.waves_per_head = g.waves; a.wave_floats = g.wave_floats;
  a.chunk = L.chunk; a.q_scale = 1.f; a.denom_eps = 0.f; a.out = out;
  scan_dispatch<float, SCAN_DELTA>(g, L, a, stream);
  RA_LAUNCH_CHECK("delta_rule_scan");
  return 0;
}

extern "C" int ra_wkv_scan(const void* proj, int act_dtype, int ld, int r_off, int k_off, int v_off, const float* decay,
                           int ldw, const float* w0, const float* u, float* state, long slot_stride,
                           const int* cu_tokens, const int* state_slots, const int* fresh, int n_seqs, int n_tokens,
                           int max_q_len, int heads, int dim, float* out, hipStream_t stream) {
  RA_CHECK(n_seqs > 0 && n_tokens > 0 && heads > 0, "wkv_scan: %d requests, %d tokens, %d heads", n_seqs, n_tokens, heads);
  ScanGeom g;
  RA_CHECK(scan_geom(2, dim, dim, &g), "wkv_scan: heads of %d x %d (keys up to 512)", dim, dim);
  RA_CHECK(slot_stride >= (long)heads * g.waves * g.wave_floats, "wkv_scan: a state slot of %ld floats, need %ld",
           slot_stride, (long)heads * g.waves * g.wave_floats);
  RA_CHECK(heads <= 65535, "wkv_scan: %d heads in one launch", heads);
  RA_CHECK(ldw >= heads * dim, "wkv_scan: decay rows of %d for %d heads of %d", ldw, heads, dim);
  RA_CHECK(act_dtype == RA_F32 || act_dtype == RA_BF16, "wkv_scan: unknown dtype tag %d", act_dtype);
  const ScanLaunch L = scan_launch(g, n_seqs, heads, max_q_len, 3);
  const size_t es = act_dtype == RA_F32 ? 4 : 2;
  ScanArgs a = {};
  a.q = (const char*)proj + (size_t)r_off * es;
  a.k = (const char*)proj + (size_t)k_off * es;
  a.v = (const char*)proj + (size_t)v_off * es;
  a.ld = ld; a.q_heads = heads; a.gates = nullptr; a.state = state; a.slot_stride = slot_stride;
  a.cu_tokens = cu_tokens; a.state_slots = state_slots; a.fresh = fresh;
  a.H = heads; a.dk = dim; a.dv = dim; a.waves_per_head = g.waves; a.wave_floats = g.wave_floats;
  a.chunk = L.chunk; a.q_scale = 1.f; a.denom_eps = 0.f; a.out = out;
  a.w = decay; a.ldw = ldw; a.w0 = w0; a.u = u;
  if (act_dtype == RA_F32) scan_dispatch<float, SCAN_WKV>(g, L, a, stream);
  else scan_dispatch<bf16_t, SCAN_WKV>(g, L, a, stream);
  RA_LAUNCH_CHECK("wkv_scan");
  return 0;
}

// kind 3 of ra_scan_state_floats: S <- decays[h] S + k v^T, o = S^T q, with silu on q, k and v as they are read.
extern "C" int ra_decay_scan(const void* proj, int act_dtype, int ld, int q_off, int k_off, int v_off,
                             const float* decays, float* state, long slot_stride, const int* cu_tokens,
                             const int* state_slots, const int* fresh, int n_seqs, int n_tokens, int max_q_len,
                             int heads, int key_dim, int value_dim, float* out, hipStream_t stream) {
  RA_CHECK(n_seqs > 0 && n_tokens > 0 && heads > 0, "decay_scan: %d requests, %d tokens, %d heads", n_seqs, n_tokens, heads);
  RA_CHECK(decays != nullptr, "decay_scan: one factor a head is needed");
  ScanGeom g;
  RA_CHECK(scan_geom(3, key_dim, value_dim, &g), "decay_scan: heads of %d x %d (keys up to 512)", key_dim, value_dim);
  RA_CHECK(slot_stride >= (long)heads * g.waves * g.wave_floats, "decay_scan: a state slot of %ld floats, need %ld",
           slot_stride, (long)heads * g.waves * g.wave_floats);
  RA_CHECK(heads <= 65535, "decay_scan: %d heads in one launch", heads);
  RA_CHECK(act_dtype == RA_F32 || act_dtype == RA_BF16, "decay_scan: unknown dtype tag %d", act_dtype);
  const ScanLaunch L = scan_launch(g, n_seqs, heads, max_q_len);
  const size_t es = act_dtype == RA_F32 ? 4 : 2;
  ScanArgs a = {};
  a.q = (const char*)proj + (size_t)q_off * es;
  a.k = (const char*)proj + (size_t)k_off * es;
  a.v = (const char*)proj + (size_t)v_off * es;
  a.ld = ld; a.q_heads = heads; a.gates = nullptr; a.state = state; a.slot_stride = slot_stride;
  a.cu_tokens = cu_tokens; a.state_slots = state_slots; a.fresh = fresh;
  a.H = heads; a.dk = key_dim; a.dv = value_dim; a.waves_per_head = g.waves; a.wave_floats = g.wave_floats;
  a.chunk = L.chunk; a.q_scale = 1.f; a.denom_eps = 0.f; a.out = out;
  a.head_decay = decays;
  if (act_dtype == RA_F32) scan_dispatch<float, SCAN_DECAY>(g, L, a, stream);
  else scan_dispatch<bf16_t, SCAN_DECAY>(g, L, a, stream);
  RA_LAUNCH_CHECK("decay_scan");
  return 0;
}

extern "C" int ra_head_norm_gate(const float* read, const float* weight, int per_head_weight, const void* gate,
                                 int ldg, int act_dtype, int silu, float eps, int n_tokens, int heads, int value_dim,
                                 void* out, hipStream_t stream) {
  RA_CHECK(n_tokens > 0 && heads > 0 && value_dim > 0, "head_norm_gate: %d tokens, %d heads of %d", n_tokens, heads,
           value_dim);
  const long units = (long)n_tokens * heads;
  const unsigned blocks = (unsigned)((units + 3) / 4);
  const int ws = per_head_weight ? value_dim : 0;
  const int es = act_dtype == RA_F32 ? 4 : 2;
  if (value_dim >= 512 && value_dim % 8 == 0 && value_dim <= 8 * HNG_CHUNKS * 1024 && units <= 0x7fffffffL &&
      ((uintptr_t)read % 16) == 0 && ((uintptr_t)weight % 16) == 0 && ((uintptr_t)gate % 16) == 0 &&
      ((long)ldg * es) % 16 == 0 && ((uintptr_t)out % 16) == 0 && (act_dtype == RA_F32 || act_dtype == RA_BF16)) {
    int threads = (value_dim / 8 + RA_WAVE - 1) / RA_WAVE * RA_WAVE;
    if (threads > 1024) threads = 1024;
    if (act_dtype == RA_F32)
      head_norm_gate_wide_kernel<float><<<(unsigned)units, threads, 0, stream>>>(read, weight, ws, (const float*)gate, ldg,
                                                                                 silu, eps, heads, value_dim, (float*)out);
    else
      head_norm_gate_wide_kernel<bf16_t><<<(unsigned)units, threads, 0, stream>>>(read, weight, ws, (const bf16_t*)gate,
                                                                                  ldg, silu, eps, heads, value_dim,
                                                                                  (bf16_t*)out);
    RA_LAUNCH_CHECK("head_norm_gate");
    return 0;
  }
  if (act_dtype == RA_F32)
    head_norm_gate_kernel<float><<<blocks, 4 * RA_WAVE, 0, stream>>>(read, weight, ws, (const float*)gate, ldg, silu,
                                                                     eps, heads, value_dim, (float*)out, units);
  else if (act_dtype == RA_BF16)
    head_norm_gate_kernel<bf16_t><<<blocks, 4 * RA_WAVE, 0, stream>>>(read, weight, ws, (const bf16_t*)gate, ldg, silu,
                                                                      eps, heads, value_dim, (bf16_t*)out, units);
  else
    return ra_fail("head_norm_gate: unknown dtype tag %d", act_dtype);
  RA_LAUNCH_CHECK("head_norm_gate");
  return 0;
}

extern "C" int ra_normed_mean(const void* const* xs, const float* const* ws, int n, int act_dtype, float eps,
                              int n_tokens, int hidden, void* out, float* resid, float scale, hipStream_t stream) {
  RA_CHECK(n >= 1 && n <= MEAN_MAX, "normed_mean: %d inputs (1 to %d)", n, MEAN_MAX);
  RA_CHECK(n_tokens > 0 && hidden > 0, "normed_mean: %d tokens, width %d", n_tokens, hidden);
  RA_CHECK((out == nullptr) != (resid == nullptr), "normed_mean: the result goes into the stream or into out");
  MeanInputs in;
  for (int i = 0; i < MEAN_MAX; ++i) {
    in.x[i] = i < n ? xs[i] : nullptr;
    in.w[i] = i < n ? ws[i] : nullptr;
  }
  const int threads = hidden >= 2048 ? 512 : 256;
#define RA_NM(TA, N) normed_mean_kernel<TA, N><<<n_tokens, threads, 0, stream>>>(in, eps, hidden, (TA*)out, resid, scale)
#define RA_NM_N(TA)                 \
  do {                              \
    if (n == 1) RA_NM(TA, 1);       \
    else if (n == 2) RA_NM(TA, 2);  \
    else if (n == 3) RA_NM(TA, 3);  \
    else RA_NM(TA, 4);              \
  } while (0)
  if (act_dtype == RA_F32) RA_NM_N(float);
  else if (act_dtype == RA_BF16) RA_NM_N(bf16_t);
  else return ra_fail("normed_mean: unknown dtype tag %d", act_dtype);
#undef RA_NM_N
#undef RA_NM
  RA_LAUNCH_CHECK("normed_mean");
  return 0;
}
