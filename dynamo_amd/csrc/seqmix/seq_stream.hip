// Row-wise kernels around parallel residual streams and their mixers:
// token embedding plus a row chosen by a hash of the previous and current
// token; the step between two sublayers on S residual streams (write of the
// waiting sublayer output, mixing of the streams, read and RMS norm for the
// next sublayer in one pass); RMS norms over whole column runs of a
// projection, also straight into the paged cache; head-major repacking and
// element-wise output gates around per-head batched products; the gated
// grouped norm after a state-space scan; exact GELU and SiLU-gated linear
// units; and a router that keeps the largest logits.
//
// Norms, gates and the streams are fp32; T is the activation type.
#include "seq_common.h"

namespace {

inline int row_threads(int W) {
  int b = 64;
  while (b < W && b < 1024) b <<= 1;
  return b;
}

// ---------------------------------------------------------------------------
// out[t] = embed[id] + table[(prev * mul_prev + id * mul_cur) mod n], n =
// table rows - 1; the first token of a sequence takes row n. prev of a
// portion's first row comes from the slot's state (the id as a float).
template <typename T>
__global__ void embed_pair_hash_kernel(
    float* __restrict__ out, const int* __restrict__ ids,
    const T* __restrict__ embed, const T* __restrict__ table,
    const float* __restrict__ prev_state, const int* __restrict__ tok_seq,
    const int* __restrict__ seq_start, const int* __restrict__ seq_len,
    const int* __restrict__ seq_slot, const int* __restrict__ seq_pos0, int W,
    int n, long long mul_prev, long long mul_cur) {
  const int t = blockIdx.x;
  const int s = tok_seq[t];
  const int id = ids[t];
  const T* e = embed + (int64_t)id * W;
  if (seq_len[s] == 0) {  // padding row
    for (int c = threadIdx.x; c < W; c += blockDim.x)
      out[(int64_t)t * W + c] = to_f(e[c]);
    return;
  }
  long long row;
  if (t == seq_start[s]) {
    row = seq_pos0[s] == 0
              ? n
              : (((long long)prev_state[seq_slot[s]] * mul_prev +
                  (long long)id * mul_cur) % n);
  } else {
    row = ((long long)ids[t - 1] * mul_prev + (long long)id * mul_cur) % n;
  }
  const T* b = table + row * W;
  for (int c = threadIdx.x; c < W; c += blockDim.x)
    out[(int64_t)t * W + c] = to_f(e[c]) + to_f(b[c]);
}

// second launch: nobody reads the slot's previous token any more
__global__ void pair_state_update_kernel(
    float* __restrict__ prev_state, const int* __restrict__ ids,
    const int* __restrict__ seq_start, const int* __restrict__ seq_len,
    const int* __restrict__ seq_slot, int B) {
  const int s = blockIdx.x * blockDim.x + threadIdx.x;
  if (s >= B) return;
  const int len = seq_len[s];
  if (len == 0) return;
  prev_state[seq_slot[s]] = (float)ids[seq_start[s] + len - 1];
}

// ---------------------------------------------------------------------------
// One workgroup per token row on S streams xs [T, S, W] (fp32, in place):
// new[t] = sum_s mix[s, t] old[s] + mult * out_w[t] * delta  (with delta)
// u = sum_s in_w[s] new[s]; out = u / rms(u) * (1 + norm_w)   (with in_w)
// A thread owns its channels of every stream, so the write needs no second
// launch; u is formed again from the thread's own writes after the
// reduction.
constexpr int MAXS = 8;
template <typename T, typename TO, int S_>
__global__ void stream_step_kernel(
    TO* __restrict__ out, float* __restrict__ xs, const T* __restrict__ delta,
    const float* __restrict__ mix, const float* __restrict__ out_w, float mult,
    const float* __restrict__ in_w, const float* __restrict__ norm_w, int S,
    int W, float eps) {
  __shared__ float red[16];
  __shared__ float cm[MAXS * MAXS + 2 * MAXS];
  const int t = blockIdx.x;
  const int NS = S_ > 0 ? S_ : S;
  float* cmix = cm;
  float* cout = cm + MAXS * MAXS;
  float* cin = cout + MAXS;
  for (int i = threadIdx.x; i < NS * NS; i += blockDim.x)
    cmix[i] = delta ? mix[i] : 0.f;
  for (int i = threadIdx.x; i < NS; i += blockDim.x) {
    cout[i] = delta ? mult * out_w[i] : 0.f;
    cin[i] = in_w ? in_w[i] : 0.f;
  }
  __syncthreads();
  float* row = xs + (int64_t)t * NS * W;
  float ss = 0.f;
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    float x[S_ > 0 ? S_ : MAXS];
#pragma unroll
    for (int s = 0; s < (S_ > 0 ? S_ : MAXS); s++)
      if (s < NS) x[s] = row[s * W + c];
    float u = 0.f;
    if (delta) {
      const float d = to_f(delta[(int64_t)t * W + c]);
#pragma unroll
      for (int to = 0; to < (S_ > 0 ? S_ : MAXS); to++) {
        if (to >= NS) break;
        float y = cout[to] * d;
#pragma unroll
        for (int s = 0; s < (S_ > 0 ? S_ : MAXS); s++)
          if (s < NS) y += cmix[s * NS + to] * x[s];
        row[to * W + c] = y;
        u += cin[to] * y;
      }
    } else {
#pragma unroll
      for (int s = 0; s < (S_ > 0 ? S_ : MAXS); s++)
        if (s < NS) u += cin[s] * x[s];
    }
    ss += u * u;
  }
  if (!in_w) return;
  float inv = 1.f;
  if (norm_w) inv = 1.f / sqrtf(block_sum(ss, red) / (float)W + eps);
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    float u = 0.f;
#pragma unroll
    for (int s = 0; s < (S_ > 0 ? S_ : MAXS); s++)
      if (s < NS) u += cin[s] * row[s * W + c];
    out[(int64_t)t * W + c] =
        from_f<TO>(norm_w ? u * inv * (1.f + norm_w[c]) : u);
  }
}

// ---------------------------------------------------------------------------
// dst[i] = x[i] / rms(x[0..n)) * w[i]; one workgroup per run of n entries
template <typename T>
DEVINL float run_inv_rms(const T* __restrict__ x, int n, float eps,
                         float* red) {
  float ss = 0.f;
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    const float v = to_f(x[i]);
    ss += v * v;
  }
  return 1.f / sqrtf(block_sum(ss, red) / (float)n + eps);
}

template <typename T>
__global__ void rms_norm_cols_kernel(T* __restrict__ out,
                                     const T* __restrict__ x, int stride,
                                     int col, const float* __restrict__ w,
                                     int n, float eps) {
  __shared__ float red[16];
  const int t = blockIdx.x;
  const T* src = x + (int64_t)t * stride + col;
  const float inv = run_inv_rms(src, n, eps, red);
  for (int i = threadIdx.x; i < n; i += blockDim.x)
    out[(int64_t)t * n + i] = from_f<T>(to_f(src[i]) * inv * w[i]);
}

// blockIdx.y 0: the query run in place. blockIdx.y 1: the key run, normed,
// and the raw values into the token's cache slot [pages, G, ps, d].
template <typename T>
__global__ void rownorm_append_kernel(
    T* __restrict__ proj, int stride, int nq, int off_k, int nk, int off_v,
    int nv, const float* __restrict__ qw, const float* __restrict__ kw,
    float eps, T* __restrict__ kcache, T* __restrict__ vcache,
    const int64_t* __restrict__ slot_mapping, int G, int ps) {
  __shared__ float red[16];
  const int t = blockIdx.x;
  T* rowp = proj + (int64_t)t * stride;
  if (blockIdx.y == 0) {
    const float inv = run_inv_rms(rowp, nq, eps, red);
    for (int i = threadIdx.x; i < nq; i += blockDim.x)
      rowp[i] = from_f<T>(to_f(rowp[i]) * inv * qw[i]);
    return;
  }
  const int64_t slot = slot_mapping[t];
  if (slot < 0) return;
  const int64_t page = slot / ps, inpage = slot % ps;
  const int dk = nk / G, dv = nv / G;
  const float inv = run_inv_rms(rowp + off_k, nk, eps, red);
  for (int i = threadIdx.x; i < nk; i += blockDim.x) {
    const int g = i / dk, e = i - g * dk;
    kcache[((page * G + g) * ps + inpage) * dk + e] =
        from_f<T>(to_f(rowp[off_k + i]) * inv * kw[i]);
  }
  for (int i = threadIdx.x; i < nv; i += blockDim.x) {
    const int g = i / dv, e = i - g * dv;
    vcache[((page * G + g) * ps + inpage) * dv + e] = rowp[off_v + i];
  }
}

// ---------------------------------------------------------------------------
// x fp32 [T, H, R] -> out [H, T, R]
template <typename T>
__global__ void heads_major_kernel(T* __restrict__ out,
                                   const float* __restrict__ x, int T_, int H,
                                   int R) {
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (int64_t)T_ * H * R) return;
  const int r = idx % R;
  const int64_t th = idx / R;
  const int h = th % H;
  const int64_t t = th / H;
  out[((int64_t)h * T_ + t) * R + r] = from_f<T>(x[idx]);
}

// o [H, T, dv], gate rows of stride gs -> out [T, H * dv] = o sigmoid(gate)
template <typename T>
__global__ void heads_gate_kernel(T* __restrict__ out, const T* __restrict__ o,
                                  const T* __restrict__ gate, int gs, int T_,
                                  int H, int dv) {
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (int64_t)T_ * H * dv) return;
  const int e = idx % dv;
  const int64_t th = idx / dv;
  const int h = th % H;
  const int64_t t = th / H;
  const float g = sigmoid_f(to_f(gate[t * gs + h * dv + e]));
  out[idx] = from_f<T>(to_f(o[((int64_t)h * T_ + t) * dv + e]) * g);
}

// (y * silu(z)) / rms over the group * w; one workgroup per (row, group)
template <typename T>
__global__ void gated_group_norm_kernel(
    T* __restrict__ out, const float* __restrict__ y, const T* __restrict__ z,
    int zs, const float* __restrict__ w, int C, int gw, float eps) {
  __shared__ float red[16];
  const int t = blockIdx.x, c0 = blockIdx.y * gw;
  const float* yr = y + (int64_t)t * C + c0;
  const T* zr = z + (int64_t)t * zs + c0;
  float ss = 0.f;
  for (int i = threadIdx.x; i < gw; i += blockDim.x) {
    const float v = yr[i] * silu_f(to_f(zr[i]));
    ss += v * v;
  }
  const float inv = 1.f / sqrtf(block_sum(ss, red) / (float)gw + eps);
  for (int i = threadIdx.x; i < gw; i += blockDim.x) {
    const float v = yr[i] * silu_f(to_f(zr[i]));
    out[(int64_t)t * C + c0 + i] = from_f<T>(v * inv * w[c0 + i]);
  }
}

// ---------------------------------------------------------------------------
// 16-byte pieces of activations: 4 floats or 8 bf16
template <typename T> struct Piece;
template <> struct Piece<float> {
  static constexpr int N = 4;
  float4 v;
  DEVINL float get(int i) const { return (&v.x)[i]; }
  DEVINL void set(int i, float f) { (&v.x)[i] = f; }
};
template <> struct Piece<bf16_t> {
  static constexpr int N = 8;
  uint4 v;
  DEVINL float get(int i) const {
    const uint32_t w = (&v.x)[i >> 1];
    union { float f; uint32_t u; } c;
    c.u = (i & 1) ? (w & 0xffff0000u) : (w << 16);
    return c.f;
  }
  DEVINL void set(int i, float f) {
    uint32_t& w = (&v.x)[i >> 1];
    const uint32_t b = from_f<bf16_t>(f);
    w = (i & 1) ? ((w & 0x0000ffffu) | (b << 16)) : ((w & 0xffff0000u) | b);
  }
};

DEVINL float gelu_erf_f(float v) {
  return 0.5f * v * (1.f + erff(v * 0.70710678118654752440f));
}

// VEC: every thread one 16-byte piece (n counts pieces), else one element
template <typename T, bool VEC>
__global__ void gelu_erf_kernel(T* __restrict__ out, const T* __restrict__ x,
                                int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  if (VEC) {
    Piece<T> a, o;
    a.v = reinterpret_cast<const decltype(a.v)*>(x)[i];
#pragma unroll
    for (int e = 0; e < Piece<T>::N; e++) o.set(e, gelu_erf_f(a.get(e)));
    reinterpret_cast<decltype(o.v)*>(out)[i] = o.v;
  } else {
    out[i] = from_f<T>(gelu_erf_f(to_f(x[i])));
  }
}

// gate_up [rows, 2F] -> out [rows, F] = silu(gate) * up
template <typename T, bool VEC>
__global__ void silu_glu_kernel(T* __restrict__ out,
                                const T* __restrict__ gate_up, int F,
                                int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  if (VEC) {
    constexpr int N = Piece<T>::N;
    const int fp = F / N;  // pieces per output row
    const int64_t r = i / fp;
    const int c = (i - r * fp) * N;
    Piece<T> g, u, o;
    g.v = *reinterpret_cast<const decltype(g.v)*>(gate_up + r * 2 * F + c);
    u.v = *reinterpret_cast<const decltype(u.v)*>(gate_up + r * 2 * F + F + c);
#pragma unroll
    for (int e = 0; e < N; e++) o.set(e, silu_f(g.get(e)) * u.get(e));
    *reinterpret_cast<decltype(o.v)*>(out + r * F + c) = o.v;
  } else {
    const int64_t r = i / F;
    const int c = i - r * F;
    const float g = to_f(gate_up[r * 2 * F + c]);
    const float u = to_f(gate_up[r * 2 * F + F + c]);
    out[i] = from_f<T>(silu_f(g) * u);
  }
}

// ---------------------------------------------------------------------------
// One wave per token: `top` rounds of arg-max over logits + bias (the lower
// index wins a tie), then the softmax over the chosen values.
constexpr int ROUTE_PER_LANE = 16;  // n <= 1024
__global__ void moe_route_topk_kernel(int* __restrict__ idx,
                                      float* __restrict__ wgt,
                                      const float* __restrict__ logits,
                                      int stride, const float* __restrict__ bias,
                                      int n, int top, int T_) {
  const int t = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (t >= T_) return;
  const int lane = threadIdx.x & 63;
  float v[ROUTE_PER_LANE];
#pragma unroll
  for (int e = 0; e < ROUTE_PER_LANE; e++) {
    const int i = lane + 64 * e;
    v[e] = i < n ? logits[(int64_t)t * stride + i] + (bias ? bias[i] : 0.f)
                 : -INFINITY;
  }
  float first = 0.f, sum = 0.f;
  for (int r = 0; r < top; r++) {
    float best = -INFINITY;
    int bi = 0x7fffffff;
#pragma unroll
    for (int e = 0; e < ROUTE_PER_LANE; e++) {
      const int i = lane + 64 * e;
      if (i < n && (v[e] > best || (v[e] == best && i < bi)) &&
          v[e] != -INFINITY) {
        best = v[e];
        bi = i;
      }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      const float ob = __shfl_xor(best, off, 64);
      const int oi = __shfl_xor(bi, off, 64);
      if (ob > best || (ob == best && oi < bi)) {
        best = ob;
        bi = oi;
      }
    }
    if (r == 0) first = best;
    const float p = expf(best - first);  // the first is the largest
    sum += p;
    if (lane == 0) {
      idx[(int64_t)t * top + r] = bi == 0x7fffffff ? 0 : bi;
      wgt[(int64_t)t * top + r] = p;
    }
#pragma unroll
    for (int e = 0; e < ROUTE_PER_LANE; e++)
      if (lane + 64 * e == bi) v[e] = -INFINITY;
  }
  if (lane == 0) {
    const float inv = 1.f / sum;
    for (int r = 0; r < top; r++) wgt[(int64_t)t * top + r] *= inv;
  }
}

void check_ints(const torch::Tensor& a, int64_t n, const char* what) {
  TORCH_CHECK(a.scalar_type() == torch::kInt && a.is_contiguous() &&
                  a.numel() >= n && a.is_cuda(),
              "seqmix: ", what, " must be an int32 device tensor");
}
void check_f32(const torch::Tensor& a, int64_t n, const char* what) {
  TORCH_CHECK(a.scalar_type() == torch::kFloat && a.is_contiguous() &&
                  a.numel() == n && a.is_cuda(),
              "seqmix: ", what, " must be fp32 with ", n, " entries");
}

}  // namespace

void embed_pair_hash(torch::Tensor out, torch::Tensor ids, torch::Tensor embed,
                     torch::Tensor table, int64_t mul_prev, int64_t mul_cur,
                     torch::Tensor prev_state, torch::Tensor tok_seq,
                     torch::Tensor seq_start, torch::Tensor seq_len,
                     torch::Tensor seq_slot, torch::Tensor seq_pos0) {
  const int T_ = ids.size(0), W = embed.size(1), B = seq_start.size(0);
  SEQ_CHECK(is_act(embed) && embed.is_contiguous() && table.is_contiguous() &&
                table.scalar_type() == embed.scalar_type() &&
                table.dim() == 2 && table.size(1) == W && table.size(0) >= 2,
            "embedding tables");
  SEQ_CHECK(out.scalar_type() == torch::kFloat && out.is_contiguous() &&
                out.size(0) == T_ && out.size(1) == W, "embedding out");
  SEQ_CHECK(prev_state.scalar_type() == torch::kFloat &&
                prev_state.is_contiguous() && prev_state.dim() == 2 &&
                prev_state.size(1) == 1, "previous-token state [slots, 1]");
  SEQ_CHECK(mul_prev >= 0 && mul_cur >= 0, "hash multipliers");
  check_ints(ids, T_, "ids");
  check_ints(tok_seq, T_, "tok_seq");
  check_ints(seq_start, B, "seq_start");
  check_ints(seq_len, B, "seq_len");
  check_ints(seq_slot, B, "seq_slot");
  check_ints(seq_pos0, B, "seq_pos0");
  if (T_ == 0) return;
  DISPATCH_ACT(embed, hipLaunchKernelGGL(
      embed_pair_hash_kernel<T>, dim3(T_), dim3(std::min(256, row_threads(W))),
      0, cur_stream(), ptr<float>(out), cptr<int>(ids), cptr<T>(embed),
      cptr<T>(table), cptr<float>(prev_state), cptr<int>(tok_seq),
      cptr<int>(seq_start), cptr<int>(seq_len), cptr<int>(seq_slot),
      cptr<int>(seq_pos0), W, (int)table.size(0) - 1, (long long)mul_prev,
      (long long)mul_cur););
  hipLaunchKernelGGL(pair_state_update_kernel, dim3((B + 63) / 64), dim3(64),
                     0, cur_stream(), ptr<float>(prev_state), cptr<int>(ids),
                     cptr<int>(seq_start), cptr<int>(seq_len),
                     cptr<int>(seq_slot), B);
}

void stream_step(c10::optional<torch::Tensor> out, torch::Tensor xs,
                 c10::optional<torch::Tensor> delta,
                 c10::optional<torch::Tensor> mix,
                 c10::optional<torch::Tensor> out_w, double mult,
                 c10::optional<torch::Tensor> in_w,
                 c10::optional<torch::Tensor> norm_w, double eps) {
  SEQ_CHECK(xs.dim() == 3 && xs.scalar_type() == torch::kFloat &&
                xs.is_contiguous(), "streams fp32 [T, S, W]");
  const int T_ = xs.size(0), S = xs.size(1), W = xs.size(2);
  SEQ_CHECK(S >= 1 && S <= MAXS, "number of streams");
  if (delta) {
    SEQ_CHECK(is_act(*delta) && delta->is_contiguous() && delta->dim() == 2 &&
                  delta->size(0) == T_ && delta->size(1) == W, "stream delta");
    SEQ_CHECK(mix.has_value() && out_w.has_value(), "stream write weights");
    check_f32(*mix, S * S, "stream mix");
    check_f32(*out_w, S, "stream write weights");
  }
  SEQ_CHECK(in_w.has_value() == out.has_value(), "stream read");
  bool f32out = true;
  if (in_w) {
    check_f32(*in_w, S, "stream read weights");
    if (norm_w) check_f32(*norm_w, W, "stream norm weight");
    SEQ_CHECK(out->is_contiguous() && out->dim() == 2 && out->size(0) == T_ &&
                  out->size(1) == W && is_act(*out), "stream read out");
    f32out = out->scalar_type() == torch::kFloat;
    SEQ_CHECK(norm_w.has_value() || f32out, "an unnormed read is fp32");
  } else {
    SEQ_CHECK(!norm_w.has_value(), "a norm needs a read");
  }
  if (T_ == 0) return;
  if (!delta && !in_w) return;
#define LAUNCH_SS(T, TO, S_)                                                 \
  hipLaunchKernelGGL((stream_step_kernel<T, TO, S_>), dim3(T_),              \
      dim3(std::min(512, row_threads(W))), 0, cur_stream(),                  \
      out ? reinterpret_cast<TO*>(out->data_ptr()) : (TO*)nullptr,           \
      ptr<float>(xs), delta ? cptr<T>(*delta) : (const T*)nullptr,           \
      mix ? cptr<float>(*mix) : (const float*)nullptr,                       \
      out_w ? cptr<float>(*out_w) : (const float*)nullptr, (float)mult,      \
      in_w ? cptr<float>(*in_w) : (const float*)nullptr,                     \
      norm_w ? cptr<float>(*norm_w) : (const float*)nullptr, S, W, (float)eps)
#define LAUNCH_S(T, TO)                                                      \
  do {                                                                       \
    if (S == 1) LAUNCH_SS(T, TO, 1);                                         \
    else if (S == 2) LAUNCH_SS(T, TO, 2);                                    \
    else if (S == 4) LAUNCH_SS(T, TO, 4);                                    \
    else LAUNCH_SS(T, TO, 0);                                                \
  } while (0)
  const bool dbf = delta && delta->scalar_type() == torch::kBFloat16;
  if (dbf) {
    if (f32out) LAUNCH_S(bf16_t, float);
    else LAUNCH_S(bf16_t, bf16_t);
  } else {
    if (f32out) LAUNCH_S(float, float);
    else LAUNCH_S(float, bf16_t);
  }
#undef LAUNCH_S
#undef LAUNCH_SS
}

void rms_norm_cols(torch::Tensor out, torch::Tensor x, int64_t col,
                   torch::Tensor w, double eps) {
  const int T_ = x.size(0), n = out.size(1);
  SEQ_CHECK(is_act(x) && x.dim() == 2 && x.stride(1) == 1 && col >= 0 &&
                col + n <= x.size(1) && n >= 1, "norm columns");
  SEQ_CHECK(out.is_contiguous() && out.dim() == 2 && out.size(0) == T_ &&
                out.scalar_type() == x.scalar_type(), "norm out");
  check_f32(w, n, "norm weight");
  if (T_ == 0) return;
  DISPATCH_ACT(x, hipLaunchKernelGGL(
      rms_norm_cols_kernel<T>, dim3(T_), dim3(std::min(512, row_threads(n))), 0,
      cur_stream(), ptr<T>(out), cptr<T>(x), (int)x.stride(0), (int)col,
      cptr<float>(w), n, (float)eps););
}

void rownorm_append(torch::Tensor proj, int64_t nq, int64_t off_k, int64_t nk,
                    int64_t off_v, int64_t nv, torch::Tensor qw,
                    c10::optional<torch::Tensor> kw, double eps,
                    c10::optional<torch::Tensor> kcache,
                    c10::optional<torch::Tensor> vcache,
                    torch::Tensor slot_mapping) {
  const int T_ = proj.size(0);
  SEQ_CHECK(is_act(proj) && proj.dim() == 2 && proj.stride(1) == 1 &&
                nq >= 1 && nq <= proj.size(1), "query run");
  check_f32(qw, nq, "query norm weight");
  const bool own = kcache.has_value();
  int G = 1, ps = 1;
  if (own) {
    SEQ_CHECK(vcache.has_value() && kw.has_value(), "key/value cache");
    G = kcache->size(1);
    ps = kcache->size(2);
    SEQ_CHECK(kcache->is_contiguous() && vcache->is_contiguous() &&
                  kcache->dim() == 4 && vcache->dim() == 4 &&
                  vcache->size(0) == kcache->size(0) && vcache->size(1) == G &&
                  vcache->size(2) == ps && nk == G * kcache->size(3) &&
                  nv == G * vcache->size(3) &&
                  kcache->scalar_type() == proj.scalar_type() &&
                  vcache->scalar_type() == proj.scalar_type(), "kv cache");
    SEQ_CHECK(off_k >= nq && off_k + nk <= proj.size(1) && off_v >= 0 &&
                  off_v + nv <= proj.size(1) && nk >= 1 && nv >= 1,
              "key and value runs");
    check_f32(*kw, nk, "key norm weight");
    SEQ_CHECK(slot_mapping.scalar_type() == torch::kLong &&
                  slot_mapping.is_contiguous() && slot_mapping.numel() >= T_,
              "slot mapping");
  }
  if (T_ == 0) return;
  DISPATCH_ACT(proj, hipLaunchKernelGGL(
      rownorm_append_kernel<T>, dim3(T_, own ? 2 : 1),
      dim3(std::min(512, row_threads((int)std::max(nq, nk)))), 0, cur_stream(),
      ptr<T>(proj), (int)proj.stride(0), (int)nq, (int)off_k, (int)nk,
      (int)off_v, (int)nv, cptr<float>(qw),
      own ? cptr<float>(*kw) : (const float*)nullptr, (float)eps,
      own ? ptr<T>(*kcache) : (T*)nullptr, own ? ptr<T>(*vcache) : (T*)nullptr,
      cptr<int64_t>(slot_mapping), G, ps););
}

void heads_major(torch::Tensor out, torch::Tensor x) {
  SEQ_CHECK(x.dim() == 3 && x.scalar_type() == torch::kFloat &&
                x.is_contiguous(), "heads fp32 [T, H, R]");
  const int T_ = x.size(0), H = x.size(1), R = x.size(2);
  SEQ_CHECK(is_act(out) && out.is_contiguous() && out.dim() == 3 &&
                out.size(0) == H && out.size(1) == T_ && out.size(2) == R,
            "head-major out");
  const int64_t n = (int64_t)T_ * H * R;
  if (n == 0) return;
  DISPATCH_ACT(out, hipLaunchKernelGGL(
      heads_major_kernel<T>, dim3((n + 255) / 256), dim3(256), 0, cur_stream(),
      ptr<T>(out), cptr<float>(x), T_, H, R););
}

void heads_gate(torch::Tensor out, torch::Tensor o, torch::Tensor gate) {
  SEQ_CHECK(is_act(o) && o.dim() == 3 && o.is_contiguous(),
            "head-major rows [H, T, dv]");
  const int H = o.size(0), T_ = o.size(1), dv = o.size(2);
  SEQ_CHECK(out.is_contiguous() && out.dim() == 2 && out.size(0) == T_ &&
                out.size(1) == H * dv && out.scalar_type() == o.scalar_type(),
            "gated out");
  SEQ_CHECK(gate.dim() == 2 && gate.stride(1) == 1 && gate.size(0) == T_ &&
                gate.size(1) >= H * dv && gate.scalar_type() == o.scalar_type(),
            "gate rows");
  const int64_t n = (int64_t)T_ * H * dv;
  if (n == 0) return;
  DISPATCH_ACT(o, hipLaunchKernelGGL(
      heads_gate_kernel<T>, dim3((n + 255) / 256), dim3(256), 0, cur_stream(),
      ptr<T>(out), cptr<T>(o), cptr<T>(gate), (int)gate.stride(0), T_, H, dv););
}

void gated_group_norm(torch::Tensor out, torch::Tensor y, torch::Tensor z,
                      torch::Tensor w, int64_t groups, double eps) {
  SEQ_CHECK(y.dim() == 2 && y.scalar_type() == torch::kFloat &&
                y.is_contiguous(), "scan out fp32 [T, C]");
  const int T_ = y.size(0), C = y.size(1);
  SEQ_CHECK(groups >= 1 && C % groups == 0, "norm groups");
  SEQ_CHECK(is_act(z) && z.dim() == 2 && z.stride(1) == 1 && z.size(0) == T_ &&
                z.size(1) >= C, "gate rows");
  SEQ_CHECK(out.is_contiguous() && out.dim() == 2 && out.size(0) == T_ &&
                out.size(1) == C && out.scalar_type() == z.scalar_type(),
            "norm out");
  check_f32(w, C, "norm weight");
  if (T_ == 0) return;
  const int gw = C / (int)groups;
  DISPATCH_ACT(z, hipLaunchKernelGGL(
      gated_group_norm_kernel<T>, dim3(T_, (int)groups),
      dim3(std::min(512, row_threads(gw))), 0, cur_stream(), ptr<T>(out),
      cptr<float>(y), cptr<T>(z), (int)z.stride(0), cptr<float>(w), C, gw,
      (float)eps););
}

void gelu_erf(torch::Tensor out, torch::Tensor x) {
  SEQ_CHECK(is_act(x) && x.is_contiguous() && out.is_contiguous() &&
                out.scalar_type() == x.scalar_type() &&
                out.numel() == x.numel(), "gelu rows");
  const int64_t n = x.numel();
  if (n == 0) return;
  const bool al = reinterpret_cast<uintptr_t>(x.data_ptr()) % 16 == 0 &&
                  reinterpret_cast<uintptr_t>(out.data_ptr()) % 16 == 0;
  DISPATCH_ACT(x, {
    constexpr int N = Piece<T>::N;
    if (al && n % N == 0) {
      const int64_t np = n / N;
      hipLaunchKernelGGL((gelu_erf_kernel<T, true>), dim3((np + 255) / 256),
                         dim3(256), 0, cur_stream(), ptr<T>(out), cptr<T>(x),
                         np);
    } else {
      hipLaunchKernelGGL((gelu_erf_kernel<T, false>), dim3((n + 255) / 256),
                         dim3(256), 0, cur_stream(), ptr<T>(out), cptr<T>(x),
                         n);
    }
  });
}

void silu_glu(torch::Tensor out, torch::Tensor gate_up) {
  SEQ_CHECK(is_act(gate_up) && gate_up.dim() == 2 && gate_up.is_contiguous() &&
                gate_up.size(1) % 2 == 0, "gate | up rows");
  const int F = gate_up.size(1) / 2;
  SEQ_CHECK(out.is_contiguous() && out.dim() == 2 &&
                out.size(0) == gate_up.size(0) && out.size(1) == F &&
                out.scalar_type() == gate_up.scalar_type(), "glu out");
  const int64_t n = out.numel();
  if (n == 0) return;
  const bool al = reinterpret_cast<uintptr_t>(gate_up.data_ptr()) % 16 == 0 &&
                  reinterpret_cast<uintptr_t>(out.data_ptr()) % 16 == 0;
  DISPATCH_ACT(gate_up, {
    constexpr int N = Piece<T>::N;
    if (al && F % N == 0) {
      const int64_t np = n / N;
      hipLaunchKernelGGL((silu_glu_kernel<T, true>), dim3((np + 255) / 256),
                         dim3(256), 0, cur_stream(), ptr<T>(out),
                         cptr<T>(gate_up), F, np);
    } else {
      hipLaunchKernelGGL((silu_glu_kernel<T, false>), dim3((n + 255) / 256),
                         dim3(256), 0, cur_stream(), ptr<T>(out),
                         cptr<T>(gate_up), F, n);
    }
  });
}

void moe_route_topk(torch::Tensor idx, torch::Tensor wgt, torch::Tensor logits,
                    int64_t n, c10::optional<torch::Tensor> bias) {
  SEQ_CHECK(logits.dim() == 2 && logits.scalar_type() == torch::kFloat &&
                logits.stride(1) == 1 && n >= 1 && n <= logits.size(1) &&
                n <= 64 * ROUTE_PER_LANE, "router logits");
  const int T_ = logits.size(0), top = idx.size(1);
  SEQ_CHECK(idx.scalar_type() == torch::kInt && idx.is_contiguous() &&
                idx.dim() == 2 && idx.size(0) == T_ && top >= 1 && top <= n &&
                wgt.scalar_type() == torch::kFloat && wgt.is_contiguous() &&
                wgt.numel() == idx.numel(), "router choices");
  if (bias) check_f32(*bias, n, "router bias");
  if (T_ == 0) return;
  hipLaunchKernelGGL(moe_route_topk_kernel, dim3((T_ + 3) / 4), dim3(256), 0,
                     cur_stream(), ptr<int>(idx), ptr<float>(wgt),
                     cptr<float>(logits), (int)logits.stride(0),
                     bias ? cptr<float>(*bias) : (const float*)nullptr, (int)n,
                     top, T_);
}
