// Matrix-state recurrences: gated delta rule, RWKV-style time mixing with
// per-channel decay, and the mLSTM matrix memory. One workgroup owns a run
// of value columns of one (sequence, head) state S [dk, dv] and walks the
// sequence's rows of this step in order; a decoded token is a run of one.
//
// All three recurrences are independent per value column j: column j of S
// is only ever combined with the token's key-side vectors. A thread keeps
// RT rows (16 or 32, a template constant) of one column in registers; KP
// threads (adjacent at lane distance JW = 64 / KP) share a column and
// reduce their partial dot products with lane shuffles. KP is a power of
// two, so dk <= 32 * 64. Rows past dk are zero padding: they are staged as
// zeros and stay zero, which keeps the per-token loops free of bounds
// tests (fixed trip counts, 16-byte LDS reads issued back to back).
// State is fp32 in HBM, loaded once per step and stored once.
//
// The walk over a portion is latency bound (one token depends on the one
// before, and every token's inputs lie in another page of the projection
// buffers), so each token's inputs are fetched into a ring of registers
// DEPTH tokens ahead, and the key-side vectors go through a double-buffered
// LDS stage: one barrier per token, global latency spread over DEPTH
// tokens' arithmetic. PE is the number of staged elements a thread carries
// per key-side vector (1 when the workgroup is at least dk threads).
#include "seq_common.h"

namespace {

constexpr int PEMAX = 4;  // staged elements per thread and vector
constexpr int DEPTH = 4;  // tokens fetched ahead

struct SeqArgs {
  const int* seq_start;
  const int* seq_len;
  const int* seq_slot;
  const int* seq_pos0;
};

struct Geometry {
  int KP, RT, DKP, JW, NW, tiles;
};

inline Geometry geometry(int dk, int dv) {
  Geometry g;
  g.KP = 1;
  // 16 rows per thread measured slightly faster than 32 for both the
  // prompt walk and decode; 32 only when the key size needs it
  while (g.KP * 16 < dk && g.KP < 64) g.KP <<= 1;
  while (g.KP * 32 < dk) g.KP <<= 1;
  TORCH_CHECK(g.KP <= 64, "seqmix: key size too large for the recurrence");
  g.RT = (dk + g.KP - 1) / g.KP <= 16 ? 16 : 32;
  g.DKP = g.KP * g.RT;  // padded key size
  g.JW = 64 / g.KP;
  const int waves = (dv + g.JW - 1) / g.JW;
  g.NW = waves < 4 ? waves : 4;
  // enough threads to stage a key-side vector with PEMAX elements each
  const int need = (g.DKP + 64 * PEMAX - 1) / (64 * PEMAX);
  if (g.NW < need) g.NW = need;
  g.tiles = (waves + g.NW - 1) / g.NW;
  return g;
}

// reduce over the KP lanes that share a column
DEVINL float part_sum(float x, int JW) {
  for (int off = JW; off < 64; off <<= 1) x += __shfl_xor(x, off, 64);
  return x;
}

#define LOAD_STATE(S, base, fresh)                                    \
  _Pragma("unroll") for (int r = 0; r < RT; r++) {                     \
    const int row = part * RT + r;                                     \
    S[r] = (!fresh && row < dk && valid) ? base[(int64_t)row * dv + j] \
                                         : 0.f;                        \
  }
#define STORE_STATE(S, base)                                          \
  _Pragma("unroll") for (int r = 0; r < RT; r++) {                     \
    const int row = part * RT + r;                                     \
    if (row < dk && valid) base[(int64_t)row * dv + j] = S[r];         \
  }
// RT staged values of this thread's rows, as 16-byte LDS reads
#define READ_ROWS(dst, vec)                                           \
  _Pragma("unroll") for (int r4 = 0; r4 < RT / 4; r4++) {              \
    const float4 x = reinterpret_cast<const float4*>(vec + part * RT)[r4]; \
    dst[4 * r4] = x.x; dst[4 * r4 + 1] = x.y;                          \
    dst[4 * r4 + 2] = x.z; dst[4 * r4 + 3] = x.w;                      \
  }

// ---------------------------------------------------------------------------
// Gate pre-passes. The nonlinearities of the gates do not depend on the
// state, so they run here, parallel over tokens, and the serial walks below
// only load their results: out[t, h] and out[t, H + h] in fp32.
//   delta: beta = sigmoid(b); g = exp(-exp(A_log) softplus(a + dt_bias))
//   mlstm: i = cap tanh((i + ib) / cap); f = logsigmoid(cap tanh((f + fb) / cap))
template <typename T, bool MLSTM>
__global__ void gates_kernel(float* __restrict__ out,
                             const T* __restrict__ proj, int proj_stride,
                             int off_0, int off_1,
                             const float* __restrict__ p0,
                             const float* __restrict__ p1, int H, int total,
                             float cap) {
  const int idx = blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const int t = idx / H, hh = idx - t * H;
  const float x0 = to_f(proj[(int64_t)t * proj_stride + off_0 + hh]);
  const float x1 = to_f(proj[(int64_t)t * proj_stride + off_1 + hh]);
  float y0, y1;
  if (MLSTM) {
    y0 = cap * tanhf((x0 + p0[hh]) / cap);
    y1 = logsigmoid_f(cap * tanhf((x1 + p1[hh]) / cap));
  } else {
    y0 = sigmoid_f(x0);
    y1 = expf(-expf(p0[hh]) * softplus_f(x1 + p1[hh]));
  }
  out[(int64_t)t * 2 * H + hh] = y0;
  out[(int64_t)t * 2 * H + H + hh] = y1;
}

// RWKV decay w = exp(-exp(wraw + w0)), fp32 [T, H*d]
template <typename T>
__global__ void rwkv_decay_kernel(float* __restrict__ out,
                                  const T* __restrict__ wraw,
                                  const float* __restrict__ w0, int HD,
                                  int64_t total) {
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  out[idx] = expf(-expf(to_f(wraw[idx]) + w0[idx % HD]));
}

// ---------------------------------------------------------------------------
// Gated delta rule. Per token: S <- g S; u = beta (v - S^T k);
// S <- S + k u^T; o = S^T q. q and k arrive after the short convolution and
// are made unit vectors here (q also scaled by qscale).
template <int PE, int RT>
__global__ __launch_bounds__(512) void gated_delta_kernel(
    float* __restrict__ out,          // [T, H, dv]
    const float* __restrict__ qkv,    // [T, Cq + Ck + Cv]: unit k, scaled
                                      // unit q, v (after conv + silu)
    const float* __restrict__ gates,  // [T, 2H]: beta | g
    float* __restrict__ state,        // [slots, H, dk, dv]
    SeqArgs sa, int H, int G, int dk, int dv, int KP) {
  extern __shared__ __attribute__((aligned(16))) float lds[];
  // [2 buffers][k | q][DKP]
  const int DKP = KP * RT;
  const int s = blockIdx.x, hh = blockIdx.y;
  const int len = sa.seq_len[s];
  if (len == 0) return;
  const int start = sa.seq_start[s];
  const bool fresh = sa.seq_pos0[s] == 0;
  const int JW = 64 / KP;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int part = lane / JW;
  const int nw = blockDim.x >> 6;
  const int j = (blockIdx.z * nw + wave) * JW + (lane % JW);
  const bool valid = j < dv;
  const int kvh = hh / (H / G);
  const int Cq = G * dk, Cc = 2 * G * dk + H * dv;
  float* sbase = state + ((int64_t)sa.seq_slot[s] * H + hh) * dk * dv;
  float S[RT];
  LOAD_STATE(S, sbase, fresh)

  struct In { float k[PE], q[PE], beta, g, vj; };
  In pre[DEPTH];
  const int end = start + len;
  auto fetch = [&](In& in, int t) {
    const float* row = qkv + (int64_t)t * Cc;
#pragma unroll
    for (int e = 0; e < PE; e++) {
      const int i = threadIdx.x + e * blockDim.x;
      in.k[e] = i < dk ? row[Cq + kvh * dk + i] : 0.f;
      in.q[e] = i < dk ? row[kvh * dk + i] : 0.f;
    }
    in.beta = gates[(int64_t)t * 2 * H + hh];
    in.g = gates[(int64_t)t * 2 * H + H + hh];
    in.vj = valid ? row[2 * Cq + hh * dv + j] : 0.f;
  };
#pragma unroll
  for (int u = 0; u < DEPTH; u++)
    if (start + u < end) fetch(pre[u], start + u);
  for (int t0 = start; t0 < end; t0 += DEPTH) {
#pragma unroll
    for (int u = 0; u < DEPTH; u++) {
      const int t = t0 + u;
      if (t >= end) break;
      float* kl = lds + (u & 1) * 2 * DKP;
      float* ql = kl + DKP;
#pragma unroll
      for (int e = 0; e < PE; e++) {
        const int i = threadIdx.x + e * blockDim.x;
        if (i < DKP) {
          kl[i] = pre[u].k[e];
          ql[i] = pre[u].q[e];
        }
      }
      const float beta = pre[u].beta;
      const float g = pre[u].g;
      const float v_cur = pre[u].vj;
      __syncthreads();
      if (t + DEPTH < end) fetch(pre[u], t + DEPTH);
      float kr[RT], qr[RT];
      READ_ROWS(kr, kl)
      READ_ROWS(qr, ql)
      // four partial sums: the add chain is the token's critical path
      float d4[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int r = 0; r < RT; r++) {
        S[r] *= g;
        d4[r & 3] += S[r] * kr[r];
      }
      const float dot = part_sum((d4[0] + d4[1]) + (d4[2] + d4[3]), JW);
      const float uu = beta * (v_cur - dot);
      float o4[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int r = 0; r < RT; r++) {
        S[r] += kr[r] * uu;
        o4[r & 3] += S[r] * qr[r];
      }
      const float o = part_sum((o4[0] + o4[1]) + (o4[2] + o4[3]), JW);
      if (valid && part == 0) out[((int64_t)t * H + hh) * dv + j] = o;
    }
  }
  STORE_STATE(S, sbase)
}

// q and k of the delta rule become unit vectors per head, in place:
// x / sqrt(sum(x^2) + unit_eps), q also times qscale. One wave per
// (token, q-or-k head).
__global__ void unit_heads_kernel(float* __restrict__ qkv, int Cc, int G,
                                  int dk, float qscale, float unit_eps) {
  const int t = blockIdx.x, v = blockIdx.y, lane = threadIdx.x;
  float* x = qkv + (int64_t)t * Cc + v * dk;  // q heads, then k heads
  float ss = 0.f;
  for (int i = lane; i < dk; i += 64) ss += x[i] * x[i];
  ss = wave_sum(ss);
  const float mul = (v < G ? qscale : 1.f) / sqrtf(ss + unit_eps);
  for (int i = lane; i < dk; i += 64) x[i] *= mul;
}

// ---------------------------------------------------------------------------
// RWKV-style time mixing. Per token, with w = exp(-exp(wraw + w0)):
// o = (S + diag(u) k v^T)^T r; S <- diag(w) S + k v^T.
template <typename T, int PE, int RT>
__global__ __launch_bounds__(512) void rwkv_kernel(
    float* __restrict__ out,       // [T, H, d]
    const T* __restrict__ r_, const T* __restrict__ k_,
    const T* __restrict__ v_,      // [T, H*d] each
    const float* __restrict__ wdec,  // [T, H*d] decay in (0, 1)
    const float* __restrict__ u,     // [H, d]
    float* __restrict__ state,     // [slots, H, d, d]
    SeqArgs sa, int H, int dk, int dv, int KP) {
  extern __shared__ __attribute__((aligned(16))) float lds[];
  // [2 buffers][r | k | w][DKP]
  const int DKP = KP * RT;
  const int s = blockIdx.x, hh = blockIdx.y;
  const int len = sa.seq_len[s];
  if (len == 0) return;
  const int start = sa.seq_start[s];
  const bool fresh = sa.seq_pos0[s] == 0;
  const int JW = 64 / KP;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int part = lane / JW;
  const int nw = blockDim.x >> 6;
  const int j = (blockIdx.z * nw + wave) * JW + (lane % JW);
  const bool valid = j < dv;
  float* sbase = state + ((int64_t)sa.seq_slot[s] * H + hh) * dk * dv;
  float S[RT], U[RT];
  LOAD_STATE(S, sbase, fresh)
#pragma unroll
  for (int r = 0; r < RT; r++) {
    const int rowi = part * RT + r;
    U[r] = rowi < dk ? u[hh * dk + rowi] : 0.f;
  }
  const int HD = H * dk;
  struct In { float r[PE], k[PE], w[PE], vj; };
  In pre[DEPTH];
  const int end = start + len;
  auto fetch = [&](In& in, int t) {
    const int64_t base = (int64_t)t * HD + hh * dk;
#pragma unroll
    for (int e = 0; e < PE; e++) {
      const int i = threadIdx.x + e * blockDim.x;
      in.r[e] = i < dk ? to_f(r_[base + i]) : 0.f;
      in.k[e] = i < dk ? to_f(k_[base + i]) : 0.f;
      in.w[e] = i < dk ? wdec[base + i] : 0.f;
    }
    in.vj = valid ? to_f(v_[(int64_t)t * H * dv + hh * dv + j]) : 0.f;
  };
#pragma unroll
  for (int u = 0; u < DEPTH; u++)
    if (start + u < end) fetch(pre[u], start + u);
  for (int t0 = start; t0 < end; t0 += DEPTH) {
#pragma unroll
    for (int u = 0; u < DEPTH; u++) {
      const int t = t0 + u;
      if (t >= end) break;
      float* rl = lds + (u & 1) * 3 * DKP;
      float* kl = rl + DKP;
      float* wl = rl + 2 * DKP;
#pragma unroll
      for (int e = 0; e < PE; e++) {
        const int i = threadIdx.x + e * blockDim.x;
        if (i < DKP) {
          rl[i] = pre[u].r[e];
          kl[i] = pre[u].k[e];
          wl[i] = pre[u].w[e];
        }
      }
      const float v_cur = pre[u].vj;
      __syncthreads();
      if (t + DEPTH < end) fetch(pre[u], t + DEPTH);
      float rr[RT], kr[RT], wr[RT];
      READ_ROWS(rr, rl)
      READ_ROWS(kr, kl)
      READ_ROWS(wr, wl)
      float o4[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int r = 0; r < RT; r++) {
        const float kv = kr[r] * v_cur;
        o4[r & 3] += rr[r] * (S[r] + U[r] * kv);
        S[r] = wr[r] * S[r] + kv;
      }
      const float o = part_sum((o4[0] + o4[1]) + (o4[2] + o4[3]), JW);
      if (valid && part == 0) out[((int64_t)t * H + hh) * dv + j] = o;
    }
  }
  STORE_STATE(S, sbase)
}

// ---------------------------------------------------------------------------
// mLSTM matrix memory with a stabiliser m that starts at 0.
// i = cap tanh((iraw + ib) / cap); f = logsigmoid(cap tanh((fraw + fb) / cap))
// m' = max(f + m, i); S <- e^(f+m-m') S + e^(i-m') k v^T; n likewise with k;
// o = S^T q / (max(|n . q|, e^(-m')) + den_eps).
template <typename T, int PE, int RT>
__global__ __launch_bounds__(512) void mlstm_kernel(
    float* __restrict__ out,  // [T, H, dv]
    const T* __restrict__ proj, int proj_stride, int off_q, int off_k,
    int off_v, const float* __restrict__ gates,  // [T, 2H]: i | f (log)
    float* __restrict__ state_S,        // [slots, H, dk, dv]
    const float* __restrict__ state_n,  // [slots, H, dk]
    const float* __restrict__ state_m,  // [slots, H]
    SeqArgs sa, int H, int dk, int dv, int KP, float qscale, float den_eps) {
  extern __shared__ __attribute__((aligned(16))) float lds[];
  // [2 buffers][k | q][DKP]
  const int DKP = KP * RT;
  const int s = blockIdx.x, hh = blockIdx.y;
  const int len = sa.seq_len[s];
  if (len == 0) return;
  const int start = sa.seq_start[s];
  const bool fresh = sa.seq_pos0[s] == 0;
  const int JW = 64 / KP;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int part = lane / JW;
  const int nw = blockDim.x >> 6;
  const int j = (blockIdx.z * nw + wave) * JW + (lane % JW);
  const bool valid = j < dv;
  const int slot = sa.seq_slot[s];
  float* sbase = state_S + ((int64_t)slot * H + hh) * dk * dv;
  const float* nbase = state_n + ((int64_t)slot * H + hh) * dk;
  float S[RT], N[RT];
  LOAD_STATE(S, sbase, fresh)
#pragma unroll
  for (int r = 0; r < RT; r++) {
    const int rowi = part * RT + r;
    N[r] = (!fresh && rowi < dk) ? nbase[rowi] : 0.f;
  }
  float m = fresh ? 0.f : state_m[slot * H + hh];

  struct In { float k[PE], q[PE], ig, fg, vj; };
  In pre[DEPTH];
  const int end = start + len;
  auto fetch = [&](In& in, int t) {
    const T* row = proj + (int64_t)t * proj_stride;
#pragma unroll
    for (int e = 0; e < PE; e++) {
      const int i = threadIdx.x + e * blockDim.x;
      in.k[e] = i < dk ? to_f(row[off_k + hh * dk + i]) : 0.f;
      in.q[e] = i < dk ? to_f(row[off_q + hh * dk + i]) * qscale : 0.f;
    }
    in.ig = gates[(int64_t)t * 2 * H + hh];
    in.fg = gates[(int64_t)t * 2 * H + H + hh];
    in.vj = valid ? to_f(row[off_v + hh * dv + j]) : 0.f;
  };
#pragma unroll
  for (int u = 0; u < DEPTH; u++)
    if (start + u < end) fetch(pre[u], start + u);
  for (int t0 = start; t0 < end; t0 += DEPTH) {
#pragma unroll
    for (int u = 0; u < DEPTH; u++) {
      const int t = t0 + u;
      if (t >= end) break;
      float* kl = lds + (u & 1) * 2 * DKP;
      float* ql = kl + DKP;
#pragma unroll
      for (int e = 0; e < PE; e++) {
        const int i = threadIdx.x + e * blockDim.x;
        if (i < DKP) {
          kl[i] = pre[u].k[e];
          ql[i] = pre[u].q[e];
        }
      }
      const float ig = pre[u].ig;
      const float fg = pre[u].fg;
      const float v_cur = pre[u].vj;
      __syncthreads();
      if (t + DEPTH < end) fetch(pre[u], t + DEPTH);
      const float mn = fmaxf(fg + m, ig);
      const float a = expf(fg + m - mn), b = expf(ig - mn);
      m = mn;
      float kr[RT], qr[RT];
      READ_ROWS(kr, kl)
      READ_ROWS(qr, ql)
      float n4[4] = {0.f, 0.f, 0.f, 0.f}, q4[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int r = 0; r < RT; r++) {
        const float bk = b * kr[r];
        S[r] = a * S[r] + bk * v_cur;
        N[r] = a * N[r] + bk;
        n4[r & 3] += S[r] * qr[r];
        q4[r & 3] += N[r] * qr[r];
      }
      const float num = part_sum((n4[0] + n4[1]) + (n4[2] + n4[3]), JW);
      const float nq = part_sum((q4[0] + q4[1]) + (q4[2] + q4[3]), JW);
      const float den = fmaxf(fabsf(nq), expf(-m)) + den_eps;
      if (valid && part == 0) out[((int64_t)t * H + hh) * dv + j] = num / den;
    }
  }
  STORE_STATE(S, sbase)
}

// The normaliser n and stabiliser m are shared by every column tile of a
// head, so the tiles above only read them; this pass, launched after, walks
// the same gates once per (sequence, head) and stores the new n and m.
template <typename T>
__global__ void mlstm_nm_kernel(
    const T* __restrict__ proj, int proj_stride, int off_k,
    const float* __restrict__ gates, float* __restrict__ state_n,
    float* __restrict__ state_m, SeqArgs sa, int H, int dk) {
  const int s = blockIdx.x, hh = blockIdx.y;
  const int len = sa.seq_len[s];
  if (len == 0) return;
  const int start = sa.seq_start[s];
  const bool fresh = sa.seq_pos0[s] == 0;
  const int slot = sa.seq_slot[s];
  float* nbase = state_n + ((int64_t)slot * H + hh) * dk;
  float m0 = fresh ? 0.f : state_m[slot * H + hh];
  float m_end = m0;  // same on every thread; thread 0 owns row 0
  for (int i = threadIdx.x; i < dk; i += blockDim.x) {
    float n = fresh ? 0.f : nbase[i];
    float m = m0;
    for (int t = start; t < start + len; t++) {
      const T* row = proj + (int64_t)t * proj_stride;
      const float ig = gates[(int64_t)t * 2 * H + hh];
      const float fg = gates[(int64_t)t * 2 * H + H + hh];
      const float mn = fmaxf(fg + m, ig);
      n = expf(fg + m - mn) * n + expf(ig - mn) * to_f(row[off_k + hh * dk + i]);
      m = mn;
    }
    nbase[i] = n;
    m_end = m;
  }
  __syncthreads();
  if (threadIdx.x == 0) state_m[slot * H + hh] = m_end;
}

// kernel<T, PE, RT> for a geometry: PE = 1 when one pass of the workgroup
// stages a whole padded key vector
#define PICK_KERNEL(K, g)                                                    \
  ((g).DKP <= (g).NW * 64                                                    \
       ? ((g).RT == 16 ? K<T, 1, 16> : K<T, 1, 32>)                          \
       : ((g).RT == 16 ? K<T, PEMAX, 16> : K<T, PEMAX, 32>))

// ---------------------------------------------------------------------------
// State-space recurrence with a scalar decay per head. Per token, with
// dt = softplus(dt_raw + dt_bias) and a = exp(-exp(A_log) dt) from the
// pre-pass: S <- a S + (dt B) x^T; o = S^T C + D x. B and C (state size dk)
// are shared by the heads of a group; x is the head's dv value channels.
template <typename T>
__global__ void ssd_gates_kernel(float* __restrict__ out,  // [T, 2H]: dt | a
                                 const T* __restrict__ dt_raw, int stride,
                                 const float* __restrict__ dt_bias,
                                 const float* __restrict__ A_log, int H,
                                 int total) {
  const int idx = blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const int t = idx / H, hh = idx - t * H;
  const float dt = softplus_f(to_f(dt_raw[(int64_t)t * stride + hh]) + dt_bias[hh]);
  out[(int64_t)t * 2 * H + hh] = dt;
  out[(int64_t)t * 2 * H + H + hh] = expf(-expf(A_log[hh]) * dt);
}

template <int PE, int RT>
__global__ __launch_bounds__(512) void ssd_kernel(
    float* __restrict__ out,          // [T, H, dv]
    const float* __restrict__ xbc,    // [T, H*dv + 2*G*dk]: x | B | C
    const float* __restrict__ gates,  // [T, 2H]: dt | decay
    const float* __restrict__ Dskip,  // [H]
    float* __restrict__ state,        // [slots, H, dk, dv]
    SeqArgs sa, int H, int G, int dk, int dv, int KP) {
  extern __shared__ __attribute__((aligned(16))) float lds[];
  // [2 buffers][B | C][DKP]
  const int DKP = KP * RT;
  // heads vary fastest over the workgroup index: workgroups go to the
  // chip's eight dies in turn, and in a batch of decoded tokens beside a
  // few prompt portions the long walks would otherwise all land on the
  // dies that the portions' sequence numbers select
  const int s = blockIdx.y, hh = blockIdx.x;
  const int len = sa.seq_len[s];
  if (len == 0) return;
  const int start = sa.seq_start[s];
  const bool fresh = sa.seq_pos0[s] == 0;
  const int JW = 64 / KP;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int part = lane / JW;
  const int nw = blockDim.x >> 6;
  const int j = (blockIdx.z * nw + wave) * JW + (lane % JW);
  const bool valid = j < dv;
  float* sbase = state + ((int64_t)sa.seq_slot[s] * H + hh) * dk * dv;
  float S[RT];
  LOAD_STATE(S, sbase, fresh)
  const int inner = H * dv, row = inner + 2 * G * dk;
  const int grp = hh / (H / G);
  const float dskip = Dskip[hh];
  struct In { float b[PE], c[PE], xj, dt, a; };
  In pre[DEPTH];
  const int end = start + len;
  auto fetch = [&](In& in, int t) {
    const int64_t base = (int64_t)t * row + inner + grp * dk;
#pragma unroll
    for (int e = 0; e < PE; e++) {
      const int i = threadIdx.x + e * blockDim.x;
      in.b[e] = i < dk ? xbc[base + i] : 0.f;
      in.c[e] = i < dk ? xbc[base + G * dk + i] : 0.f;
    }
    in.xj = valid ? xbc[(int64_t)t * row + hh * dv + j] : 0.f;
    in.dt = gates[(int64_t)t * 2 * H + hh];
    in.a = gates[(int64_t)t * 2 * H + H + hh];
  };
#pragma unroll
  for (int u = 0; u < DEPTH; u++)
    if (start + u < end) fetch(pre[u], start + u);
  for (int t0 = start; t0 < end; t0 += DEPTH) {
#pragma unroll
    for (int u = 0; u < DEPTH; u++) {
      const int t = t0 + u;
      if (t >= end) break;
      float* bl = lds + (u & 1) * 2 * DKP;
      float* cl = bl + DKP;
#pragma unroll
      for (int e = 0; e < PE; e++) {
        const int i = threadIdx.x + e * blockDim.x;
        if (i < DKP) {
          bl[i] = pre[u].b[e];
          cl[i] = pre[u].c[e];
        }
      }
      const float x_cur = pre[u].xj, a = pre[u].a;
      const float dx = pre[u].dt * x_cur;
      __syncthreads();
      if (t + DEPTH < end) fetch(pre[u], t + DEPTH);
      float br[RT], cr[RT];
      READ_ROWS(br, bl)
      READ_ROWS(cr, cl)
      float o4[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int r = 0; r < RT; r++) {
        S[r] = a * S[r] + br[r] * dx;
        o4[r & 3] += cr[r] * S[r];
      }
      const float o = part_sum((o4[0] + o4[1]) + (o4[2] + o4[3]), JW);
      if (valid && part == 0)
        out[((int64_t)t * H + hh) * dv + j] = o + dskip * x_cur;
    }
  }
  STORE_STATE(S, sbase)
}

#define PICK_KERNEL_F32(K, g)                                                \
  ((g).DKP <= (g).NW * 64                                                    \
       ? ((g).RT == 16 ? K<1, 16> : K<1, 32>)                                \
       : ((g).RT == 16 ? K<PEMAX, 16> : K<PEMAX, 32>))

SeqArgs seq_args(const torch::Tensor& seq_start, const torch::Tensor& seq_len,
                 const torch::Tensor& seq_slot, const torch::Tensor& seq_pos0,
                 int64_t slots) {
  const int64_t B = seq_start.size(0);
  for (const torch::Tensor* t : {&seq_start, &seq_len, &seq_slot, &seq_pos0})
    TORCH_CHECK(t->scalar_type() == torch::kInt && t->is_contiguous() &&
                    t->numel() >= B && t->is_cuda(),
                "seqmix: sequence descriptors must be int32 device tensors");
  (void)slots;
  return SeqArgs{cptr<int>(seq_start), cptr<int>(seq_len), cptr<int>(seq_slot),
                 cptr<int>(seq_pos0)};
}

}  // namespace

// qkv holds q | k | v after the convolution; q and k are normalised in place
void gated_delta_rule(torch::Tensor out, torch::Tensor qkv, torch::Tensor proj,
                      int64_t off_b, int64_t off_a, torch::Tensor A_log,
                      torch::Tensor dt_bias, torch::Tensor state,
                      torch::Tensor seq_start, torch::Tensor seq_len,
                      torch::Tensor seq_slot, torch::Tensor seq_pos0,
                      int64_t G, double qscale, double unit_eps) {
  const int T_ = out.size(0), H = out.size(1), dv = out.size(2);
  const int dk = state.size(2);
  SEQ_CHECK(out.scalar_type() == torch::kFloat && out.is_contiguous(), "out");
  SEQ_CHECK(state.scalar_type() == torch::kFloat && state.is_contiguous() &&
                state.size(1) == H && state.size(3) == dv, "delta state");
  SEQ_CHECK(G >= 1 && H % G == 0, "delta head grouping");
  SEQ_CHECK(qkv.scalar_type() == torch::kFloat && qkv.is_contiguous() &&
                qkv.size(0) == T_ && qkv.size(1) == 2 * G * dk + H * dv,
            "delta qkv");
  SEQ_CHECK(proj.stride(1) == 1 && proj.size(0) == T_ &&
                off_b + H <= proj.size(1) && off_a + H <= proj.size(1),
            "delta gates");
  SEQ_CHECK(A_log.scalar_type() == torch::kFloat && A_log.numel() == H &&
                dt_bias.scalar_type() == torch::kFloat && dt_bias.numel() == H,
            "delta decay parameters");
  const int B = seq_start.size(0);
  if (T_ == 0 || B == 0) return;
  SeqArgs sa = seq_args(seq_start, seq_len, seq_slot, seq_pos0, state.size(0));
  Geometry g = geometry(dk, dv);
  hipLaunchKernelGGL(unit_heads_kernel, dim3(T_, 2 * (int)G), dim3(64), 0,
                     cur_stream(), ptr<float>(qkv), (int)qkv.size(1), (int)G,
                     dk, (float)qscale, (float)unit_eps);
  torch::Tensor gates = torch::empty({T_, 2 * H}, out.options());
  DISPATCH_ACT(proj, hipLaunchKernelGGL(
      (gates_kernel<T, false>), dim3((T_ * H + 255) / 256), dim3(256), 0,
      cur_stream(), ptr<float>(gates), cptr<T>(proj), (int)proj.stride(0),
      (int)off_b, (int)off_a, cptr<float>(A_log), cptr<float>(dt_bias), H,
      T_ * H, 0.f););
  hipLaunchKernelGGL(PICK_KERNEL_F32(gated_delta_kernel, g),
                     dim3(B, H, g.tiles), dim3(g.NW * 64),
                     4 * g.DKP * sizeof(float), cur_stream(), ptr<float>(out),
                     cptr<float>(qkv), cptr<float>(gates), ptr<float>(state),
                     sa, H, (int)G, dk, dv, g.KP);
}

void rwkv_time_mix(torch::Tensor out, torch::Tensor r, torch::Tensor k,
                   torch::Tensor v, torch::Tensor wraw, torch::Tensor w0,
                   torch::Tensor u, torch::Tensor state,
                   torch::Tensor seq_start, torch::Tensor seq_len,
                   torch::Tensor seq_slot, torch::Tensor seq_pos0) {
  const int T_ = out.size(0), H = out.size(1), dv = out.size(2);
  const int dk = state.size(2);
  SEQ_CHECK(out.scalar_type() == torch::kFloat && out.is_contiguous(), "out");
  SEQ_CHECK(state.scalar_type() == torch::kFloat && state.is_contiguous() &&
                state.size(1) == H && state.size(3) == dv, "rwkv state");
  for (const torch::Tensor* t : {&r, &k, &wraw})
    SEQ_CHECK(t->is_contiguous() && t->size(0) == T_ && t->size(1) == H * dk &&
                  t->scalar_type() == r.scalar_type(), "rwkv r/k/w");
  SEQ_CHECK(v.is_contiguous() && v.size(0) == T_ && v.size(1) == H * dv &&
                v.scalar_type() == r.scalar_type(), "rwkv v");
  SEQ_CHECK(w0.scalar_type() == torch::kFloat && w0.numel() == H * dk &&
                u.scalar_type() == torch::kFloat && u.numel() == H * dk &&
                w0.is_contiguous() && u.is_contiguous(), "rwkv w0/u");
  const int B = seq_start.size(0);
  if (T_ == 0 || B == 0) return;
  SeqArgs sa = seq_args(seq_start, seq_len, seq_slot, seq_pos0, state.size(0));
  Geometry g = geometry(dk, dv);
  torch::Tensor wdec = torch::empty({T_, H * dk}, out.options());
  const int64_t nw = (int64_t)T_ * H * dk;
  DISPATCH_ACT(r, {
    hipLaunchKernelGGL(rwkv_decay_kernel<T>, dim3((nw + 255) / 256), dim3(256),
                       0, cur_stream(), ptr<float>(wdec), cptr<T>(wraw),
                       cptr<float>(w0), H * dk, nw);
    hipLaunchKernelGGL(
        PICK_KERNEL(rwkv_kernel, g), dim3(B, H, g.tiles), dim3(g.NW * 64),
        6 * g.DKP * sizeof(float), cur_stream(), ptr<float>(out), cptr<T>(r),
        cptr<T>(k), cptr<T>(v), cptr<float>(wdec), cptr<float>(u),
        ptr<float>(state), sa, H, dk, dv, g.KP);
  });
}

void mlstm_memory(torch::Tensor out, torch::Tensor proj, int64_t off_q,
                  int64_t off_k, int64_t off_v, int64_t off_i, int64_t off_f,
                  torch::Tensor i_bias, torch::Tensor f_bias,
                  torch::Tensor state_S, torch::Tensor state_n,
                  torch::Tensor state_m, torch::Tensor seq_start,
                  torch::Tensor seq_len, torch::Tensor seq_slot,
                  torch::Tensor seq_pos0, double qscale, double cap,
                  double den_eps) {
  const int T_ = out.size(0), H = out.size(1), dv = out.size(2);
  const int dk = state_S.size(2);
  SEQ_CHECK(out.scalar_type() == torch::kFloat && out.is_contiguous(), "out");
  SEQ_CHECK(state_S.scalar_type() == torch::kFloat && state_S.is_contiguous() &&
                state_S.size(1) == H && state_S.size(3) == dv, "mlstm S");
  SEQ_CHECK(state_n.scalar_type() == torch::kFloat && state_n.is_contiguous() &&
                state_n.size(0) == state_S.size(0) && state_n.size(1) == H &&
                state_n.size(2) == dk, "mlstm n");
  SEQ_CHECK(state_m.scalar_type() == torch::kFloat && state_m.is_contiguous() &&
                state_m.size(0) == state_S.size(0) && state_m.size(1) == H,
            "mlstm m");
  const int64_t P = proj.size(1);
  SEQ_CHECK(proj.stride(1) == 1 && proj.size(0) == T_ && off_q + H * dk <= P &&
                off_k + H * dk <= P && off_v + H * dv <= P && off_i + H <= P &&
                off_f + H <= P, "mlstm projections");
  SEQ_CHECK(i_bias.scalar_type() == torch::kFloat && i_bias.numel() == H &&
                f_bias.scalar_type() == torch::kFloat && f_bias.numel() == H,
            "mlstm biases");
  const int B = seq_start.size(0);
  if (T_ == 0 || B == 0) return;
  SeqArgs sa = seq_args(seq_start, seq_len, seq_slot, seq_pos0, state_S.size(0));
  Geometry g = geometry(dk, dv);
  torch::Tensor gates = torch::empty({T_, 2 * H}, out.options());
  DISPATCH_ACT(proj, {
    hipLaunchKernelGGL((gates_kernel<T, true>), dim3((T_ * H + 255) / 256),
                       dim3(256), 0, cur_stream(), ptr<float>(gates),
                       cptr<T>(proj), (int)proj.stride(0), (int)off_i,
                       (int)off_f, cptr<float>(i_bias), cptr<float>(f_bias), H,
                       T_ * H, (float)cap);
    hipLaunchKernelGGL(
        PICK_KERNEL(mlstm_kernel, g), dim3(B, H, g.tiles), dim3(g.NW * 64),
        4 * g.DKP * sizeof(float), cur_stream(), ptr<float>(out),
        cptr<T>(proj), (int)proj.stride(0), (int)off_q, (int)off_k,
        (int)off_v, cptr<float>(gates), ptr<float>(state_S),
        ptr<float>(state_n), ptr<float>(state_m), sa, H, dk, dv, g.KP,
        (float)qscale, (float)den_eps);
    hipLaunchKernelGGL(
        mlstm_nm_kernel<T>, dim3(B, H),
        dim3(dk < 64 ? 64 : (dk > 256 ? 256 : (dk + 63) / 64 * 64)), 0,
        cur_stream(), cptr<T>(proj), (int)proj.stride(0), (int)off_k,
        cptr<float>(gates), ptr<float>(state_n), ptr<float>(state_m), sa, H,
        dk);
  });
}

// xbc fp32 [T, H*dv + 2*G*dk] (x | B | C after convolution and activation),
// dt_raw [T, >= H] in the activation type (any row stride), state
// [slots, H, dk, dv]; out fp32 [T, H*dv].
void ssd_scan(torch::Tensor out, torch::Tensor xbc, torch::Tensor dt_raw,
              torch::Tensor dt_bias, torch::Tensor A_log, torch::Tensor D,
              torch::Tensor state, torch::Tensor seq_start,
              torch::Tensor seq_len, torch::Tensor seq_slot,
              torch::Tensor seq_pos0, int64_t G) {
  const int T_ = out.size(0);
  SEQ_CHECK(state.dim() == 4 && state.scalar_type() == torch::kFloat &&
                state.is_contiguous(), "ssd state [slots, H, N, P]");
  const int H = state.size(1), dk = state.size(2), dv = state.size(3);
  SEQ_CHECK(out.scalar_type() == torch::kFloat && out.is_contiguous() &&
                out.dim() == 2 && out.size(1) == H * dv, "ssd out");
  SEQ_CHECK(G >= 1 && H % G == 0, "ssd head grouping");
  SEQ_CHECK(xbc.scalar_type() == torch::kFloat && xbc.is_contiguous() &&
                xbc.size(0) == T_ && xbc.size(1) == H * dv + 2 * G * dk,
            "ssd x | B | C");
  SEQ_CHECK(is_act(dt_raw) && dt_raw.dim() == 2 && dt_raw.stride(1) == 1 &&
                dt_raw.size(0) == T_ && dt_raw.size(1) >= H, "ssd dt");
  for (const torch::Tensor* t : {&dt_bias, &A_log, &D})
    SEQ_CHECK(t->scalar_type() == torch::kFloat && t->is_contiguous() &&
                  t->numel() == H, "ssd head parameters");
  const int B = seq_start.size(0);
  if (T_ == 0 || B == 0) return;
  SeqArgs sa = seq_args(seq_start, seq_len, seq_slot, seq_pos0, state.size(0));
  Geometry g = geometry(dk, dv);
  torch::Tensor gates = torch::empty({T_, 2 * H}, out.options());
  DISPATCH_ACT(dt_raw, hipLaunchKernelGGL(
      ssd_gates_kernel<T>, dim3((T_ * H + 255) / 256), dim3(256), 0,
      cur_stream(), ptr<float>(gates), cptr<T>(dt_raw), (int)dt_raw.stride(0),
      cptr<float>(dt_bias), cptr<float>(A_log), H, T_ * H););
  hipLaunchKernelGGL(PICK_KERNEL_F32(ssd_kernel, g), dim3(H, B, g.tiles),
                     dim3(g.NW * 64), 4 * g.DKP * sizeof(float), cur_stream(),
                     ptr<float>(out), cptr<float>(xbc), cptr<float>(gates),
                     cptr<float>(D), ptr<float>(state), sa, H, (int)G, dk, dv,
                     g.KP);
}
