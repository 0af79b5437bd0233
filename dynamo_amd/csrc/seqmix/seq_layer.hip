// Kernels for layer-list models whose sublayers are normed on both sides
// (weight-only layer norm before, and again on the sublayer's output before
// it joins the fp32 residual stream), with partially rotated queries/keys,
// differential and latent attention heads, an xIELU feed-forward and a
// real-gated linear recurrent unit. All arithmetic is fp32; activations
// that feed a matrix product are T (float or bf16).
#include "seq_common.h"

namespace {

inline int row_block(int W) {
  int b = 64;
  while (b < W && b < 1024) b <<= 1;
  return b;
}

// One workgroup per token row.
//   delta given:  res += mult * LN(delta) * post_w   (post_w absent: += delta)
//   out given:    out = LN(res) * w
// LN(x) = (x - mean) / sqrt(var + eps), var = mean of squared deviations
// (two passes, so a large mean does not cancel). A thread keeps its NI
// entries of the row in registers, so delta and res are read once and res
// and out written once; rows wider than NI * blockDim take the looping
// kernel below.
template <typename T, int NI>
__global__ void residual_layernorm_reg_kernel(
    T* __restrict__ out, float* __restrict__ res, const T* __restrict__ delta,
    const float* __restrict__ post_w, float mult, const float* __restrict__ w,
    float eps, int W) {
  __shared__ float scratch[16];
  const int t = blockIdx.x;
  float* r = res + (int64_t)t * W;
  float x[NI];
#pragma unroll
  for (int k = 0; k < NI; k++) {
    const int i = threadIdx.x + k * blockDim.x;
    x[k] = i < W ? r[i] : 0.f;
  }
  if (delta) {
    const T* dl = delta + (int64_t)t * W;
    float d[NI];
    float s = 0.f;
#pragma unroll
    for (int k = 0; k < NI; k++) {
      const int i = threadIdx.x + k * blockDim.x;
      d[k] = i < W ? to_f(dl[i]) : 0.f;
      s += d[k];
    }
    if (post_w) {
      const float mean = block_sum(s, scratch) / (float)W;
      float ss = 0.f;
#pragma unroll
      for (int k = 0; k < NI; k++) {
        const int i = threadIdx.x + k * blockDim.x;
        const float c = i < W ? d[k] - mean : 0.f;
        ss += c * c;
      }
      const float inv = 1.f / sqrtf(block_sum(ss, scratch) / (float)W + eps);
#pragma unroll
      for (int k = 0; k < NI; k++) {
        const int i = threadIdx.x + k * blockDim.x;
        if (i < W) x[k] += mult * ((d[k] - mean) * inv * post_w[i]);
      }
    } else {
#pragma unroll
      for (int k = 0; k < NI; k++) x[k] += d[k];
    }
#pragma unroll
    for (int k = 0; k < NI; k++) {
      const int i = threadIdx.x + k * blockDim.x;
      if (i < W) r[i] = x[k];
    }
  }
  if (!out) return;
  float s = 0.f;
#pragma unroll
  for (int k = 0; k < NI; k++) s += x[k];  // entries past W are 0
  const float mean = block_sum(s, scratch) / (float)W;
  float ss = 0.f;
#pragma unroll
  for (int k = 0; k < NI; k++) {
    const int i = threadIdx.x + k * blockDim.x;
    const float c = i < W ? x[k] - mean : 0.f;
    ss += c * c;
  }
  const float inv = 1.f / sqrtf(block_sum(ss, scratch) / (float)W + eps);
#pragma unroll
  for (int k = 0; k < NI; k++) {
    const int i = threadIdx.x + k * blockDim.x;
    if (i < W) out[(int64_t)t * W + i] = from_f<T>((x[k] - mean) * inv * w[i]);
  }
}

template <typename T>
__global__ void residual_layernorm_kernel(
    T* __restrict__ out, float* __restrict__ res, const T* __restrict__ delta,
    const float* __restrict__ post_w, float mult, const float* __restrict__ w,
    float eps, int W) {
  __shared__ float scratch[16];
  const int t = blockIdx.x;
  float* r = res + (int64_t)t * W;
  if (delta) {
    const T* dl = delta + (int64_t)t * W;
    if (post_w) {
      float s = 0.f;
      for (int i = threadIdx.x; i < W; i += blockDim.x) s += to_f(dl[i]);
      const float mean = block_sum(s, scratch) / (float)W;
      float ss = 0.f;
      for (int i = threadIdx.x; i < W; i += blockDim.x) {
        const float c = to_f(dl[i]) - mean;
        ss += c * c;
      }
      const float inv = 1.f / sqrtf(block_sum(ss, scratch) / (float)W + eps);
      for (int i = threadIdx.x; i < W; i += blockDim.x)
        r[i] += mult * ((to_f(dl[i]) - mean) * inv * post_w[i]);
    } else {
      for (int i = threadIdx.x; i < W; i += blockDim.x) r[i] += to_f(dl[i]);
    }
  }
  if (!out) return;
  // each thread re-reads only what it wrote itself
  float s = 0.f;
  for (int i = threadIdx.x; i < W; i += blockDim.x) s += r[i];
  const float mean = block_sum(s, scratch) / (float)W;
  float ss = 0.f;
  for (int i = threadIdx.x; i < W; i += blockDim.x) {
    const float c = r[i] - mean;
    ss += c * c;
  }
  const float inv = 1.f / sqrtf(block_sum(ss, scratch) / (float)W + eps);
  for (int i = threadIdx.x; i < W; i += blockDim.x)
    out[(int64_t)t * W + i] = from_f<T>((r[i] - mean) * inv * w[i]);
}

// xIELU: z > 0: softplus(p) z^2 + z/2;  z <= 0: (1/2 + softplus(q)) (e^z - 1 - z) + z/2
DEVINL float xielu_f(float z, float ap, float aq) {
  return z > 0.f ? ap * z * z + 0.5f * z : aq * (expm1f(z) - z) + 0.5f * z;
}

// 16 bytes per thread and step; n is a multiple of 16 / sizeof(T)
template <typename T>
__global__ void xielu_vec_kernel(T* __restrict__ out, const T* __restrict__ x,
                                 const float* __restrict__ pq, int64_t nvec) {
  constexpr int N = 16 / sizeof(T);
  const float ap = softplus_f(pq[0]), aq = 0.5f + softplus_f(pq[1]);
  union V { uint4 raw; T e[N]; };
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < nvec;
       i += (int64_t)gridDim.x * blockDim.x) {
    V v, o;
    v.raw = reinterpret_cast<const uint4*>(x)[i];
#pragma unroll
    for (int k = 0; k < N; k++) o.e[k] = from_f<T>(xielu_f(to_f(v.e[k]), ap, aq));
    reinterpret_cast<uint4*>(out)[i] = o.raw;
  }
}

template <typename T>
__global__ void xielu_kernel(T* __restrict__ out, const T* __restrict__ x,
                             const float* __restrict__ pq, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const float ap = softplus_f(pq[0]), aq = 0.5f + softplus_f(pq[1]);
  out[i] = from_f<T>(xielu_f(to_f(x[i]), ap, aq));
}

// Partial rotary over `nvec` vectors of `len` entries per token row: the
// first `dims` entries of each vector are rotated (pairs (2i, 2i+1) when
// interleaved, else (i, i + dims/2)), the rest copied. src and dst may be
// the same buffer (then nothing but the rotated pairs is touched).
template <typename T>
__global__ void rope_rows_kernel(
    T* __restrict__ dst, int dst_stride, int dst_col, int dst_vec,
    const T* __restrict__ src, int src_stride, int src_col, int src_vec,
    const int* __restrict__ positions, const float* __restrict__ freqs,
    int nvec, int len, int dims, int interleaved, int inplace) {
  const int t = blockIdx.x;
  const float pos = (float)positions[t];
  const T* s = src + (int64_t)t * src_stride + src_col;
  T* d = dst + (int64_t)t * dst_stride + dst_col;
  const int half = dims >> 1;
  for (int idx = threadIdx.x; idx < nvec * half; idx += blockDim.x) {
    const int v = idx / half, i = idx - v * half;
    const int ia = interleaved ? 2 * i : i;
    const int ib = interleaved ? 2 * i + 1 : i + half;
    float ra, rb;
    rot_pair(to_f(s[v * src_vec + ia]), to_f(s[v * src_vec + ib]), pos,
             freqs[i], freqs[half + i], ra, rb);
    d[v * dst_vec + ia] = from_f<T>(ra);
    d[v * dst_vec + ib] = from_f<T>(rb);
  }
  if (inplace) return;
  const int rest = len - dims;
  for (int idx = threadIdx.x; idx < nvec * rest; idx += blockDim.x) {
    const int v = idx / rest, i = dims + idx - v * rest;
    d[v * dst_vec + i] = s[v * src_vec + i];
  }
}

// Latent cache row of a token: [ RMS-normed latent * weight | rotated shared
// key part ], written at the token's cache slot. One workgroup per token.
template <typename T>
__global__ void latent_append_kernel(
    T* __restrict__ cache, const T* __restrict__ z, int z_stride, int z_col,
    const float* __restrict__ norm_w, const int64_t* __restrict__ slot_mapping,
    const int* __restrict__ positions, const float* __restrict__ freqs,
    int rank, int rd, int dims, int interleaved, float eps) {
  __shared__ float scratch[16];
  const int t = blockIdx.x;
  const int64_t slot = slot_mapping[t];
  if (slot < 0) return;
  const T* src = z + (int64_t)t * z_stride + z_col;
  T* dst = cache + slot * (rank + rd);
  float ss = 0.f;
  for (int i = threadIdx.x; i < rank; i += blockDim.x) {
    const float x = to_f(src[i]);
    ss += x * x;
  }
  const float inv = 1.f / sqrtf(block_sum(ss, scratch) / (float)rank + eps);
  for (int i = threadIdx.x; i < rank; i += blockDim.x)
    dst[i] = from_f<T>(to_f(src[i]) * inv * norm_w[i]);
  const float pos = (float)positions[t];
  const int half = dims >> 1;
  for (int i = threadIdx.x; i < half; i += blockDim.x) {
    const int ia = interleaved ? 2 * i : i;
    const int ib = interleaved ? 2 * i + 1 : i + half;
    float ra, rb;
    rot_pair(to_f(src[rank + ia]), to_f(src[rank + ib]), pos, freqs[i],
             freqs[half + i], ra, rb);
    dst[rank + ia] = from_f<T>(ra);
    dst[rank + ib] = from_f<T>(rb);
  }
  for (int i = dims + threadIdx.x; i < rd; i += blockDim.x)
    dst[rank + i] = src[rank + i];
}

// Differential heads: o = a1 - lambda a2; y = o / rms(o) * post * sigmoid(gate).
// a is [T, H, 2, dv] fp32. One wave per (token, head).
template <typename T>
__global__ void diff_norm_gate_kernel(T* __restrict__ out,
                                      const float* __restrict__ a,
                                      const float* __restrict__ lambda,
                                      float post, const T* __restrict__ gate,
                                      int gate_stride, float eps, int H,
                                      int dv) {
  const int t = blockIdx.x, hh = blockIdx.y, lane = threadIdx.x;
  const float* a1 = a + ((int64_t)t * H + hh) * 2 * dv;
  const float* a2 = a1 + dv;
  const float lam = lambda[0];
  float ss = 0.f;
  for (int i = lane; i < dv; i += 64) {
    const float o = a1[i] - lam * a2[i];
    ss += o * o;
  }
  ss = wave_sum(ss);
  const float inv = post / sqrtf(ss / (float)dv + eps);
  for (int i = lane; i < dv; i += 64) {
    float v = (a1[i] - lam * a2[i]) * inv;
    if (gate) v *= sigmoid_f(to_f(gate[(int64_t)t * gate_stride + hh * dv + i]));
    out[((int64_t)t * H + hh) * dv + i] = from_f<T>(v);
  }
}

// y[h, t, :] = x[t, h, :] * sigmoid(gate[t, h]); x fp32 [T, H, R], the
// output head-major so that a batched product over heads can follow.
template <typename T>
__global__ void head_sigmoid_scale_kernel(T* __restrict__ out,
                                          const float* __restrict__ x,
                                          const T* __restrict__ gate,
                                          int gate_stride, int Ttot, int H,
                                          int R) {
  const int t = blockIdx.x, hh = blockIdx.y;
  const float g = sigmoid_f(to_f(gate[(int64_t)t * gate_stride + hh]));
  const float* src = x + ((int64_t)t * H + hh) * R;
  T* dst = out + ((int64_t)hh * Ttot + t) * R;
  for (int i = threadIdx.x; i < R; i += blockDim.x)
    dst[i] = from_f<T>(src[i] * g);
}

DEVINL float gelu_tanh_f(float z) {
  return 0.5f * z * (1.f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}

// Real-gated linear recurrent unit. Per channel c of block b = c / bw:
//   r = sigmoid(gr + br), i = sigmoid(gi + bi), a = exp(-decay * r * softplus(lam))
//   S <- a S + sqrt(1 - a^2) * i * u ;   out = S * gelu_tanh(y)
// gates [nb, T, 2 bw] fp32 hold gr (first bw) and gi of each block's
// channels. The slot's state continues earlier steps and a sequence at
// position 0 starts from S = 0.
//
// The recurrence is linear in S, so a long portion is cut into chunks of
// `chunk` tokens that run in parallel: a first kernel reduces every chunk
// but the last to (A, B) with S_end = A S_begin + B, and the scan kernel
// of chunk k first folds the summaries of chunks 0..k-1 onto the slot's
// state. A thread owns one channel of one chunk of one sequence. Decoded
// tokens and short portions are a single chunk and skip the first kernel.
struct RglruCoef {
  float a, b;
};
DEVINL RglruCoef rglru_coef(float gr, float gi, float cbr, float cbi,
                            float rate, float u) {
  const float r = sigmoid_f(gr + cbr);
  const float ig = sigmoid_f(gi + cbi);
  const float la = rate * r;
  RglruCoef c;
  c.a = expf(la);
  // 1 - a^2 = -expm1(2 log a): exact also where a is close to 1
  c.b = sqrtf(-expm1f(2.f * la)) * (ig * u);
  return c;
}

__global__ void rglru_chunk_summary_kernel(
    float* __restrict__ sumA, float* __restrict__ sumB,  // [B, nch, C]
    const float* __restrict__ u, const float* __restrict__ gates,
    const float* __restrict__ br, const float* __restrict__ bi,
    const float* __restrict__ lam, const int* __restrict__ seq_start,
    const int* __restrict__ seq_len, int Ttot, int C, int bw, float decay,
    int chunk, int nch) {
  const int s = blockIdx.z, k = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  const int len = seq_len[s];
  // the last chunk of a sequence carries into nothing
  if (c >= C || (k + 1) * chunk >= len) return;
  const int start = seq_start[s] + k * chunk;
  const int b = c / bw, o = c - b * bw;
  const float* gr = gates + ((int64_t)b * Ttot + start) * 2 * bw + o;
  const float rate = -decay * softplus_f(lam[c]);
  const float cbr = br[c], cbi = bi[c];
  float A = 1.f, S = 0.f;
#pragma unroll 4
  for (int j = 0; j < chunk; j++) {
    const RglruCoef q = rglru_coef(gr[(int64_t)j * 2 * bw],
                                   gr[(int64_t)j * 2 * bw + bw], cbr, cbi, rate,
                                   u[(int64_t)(start + j) * C + c]);
    A *= q.a;
    S = q.a * S + q.b;
  }
  sumA[((int64_t)s * nch + k) * C + c] = A;
  sumB[((int64_t)s * nch + k) * C + c] = S;
}

template <typename T>
__global__ void rglru_scan_kernel(
    T* __restrict__ out, const float* __restrict__ u,
    const float* __restrict__ gates, const float* __restrict__ br,
    const float* __restrict__ bi, const float* __restrict__ lam,
    const T* __restrict__ y, int y_stride, float* __restrict__ state,
    const float* __restrict__ sumA, const float* __restrict__ sumB,
    const int* __restrict__ seq_start, const int* __restrict__ seq_len,
    const int* __restrict__ seq_slot, const int* __restrict__ seq_pos0,
    int Ttot, int C, int bw, float decay, int chunk, int nch) {
  const int s = blockIdx.z, k = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  const int len = seq_len[s];
  if (c >= C || k * chunk >= len) return;
  const int n = min(chunk, len - k * chunk);
  const int start = seq_start[s] + k * chunk;
  float* st = state + (int64_t)seq_slot[s] * C + c;
  float S = seq_pos0[s] > 0 ? *st : 0.f;
  for (int kk = 0; kk < k; kk++)
    S = sumA[((int64_t)s * nch + kk) * C + c] * S +
        sumB[((int64_t)s * nch + kk) * C + c];
  const int b = c / bw, o = c - b * bw;
  const float* gr = gates + ((int64_t)b * Ttot + start) * 2 * bw + o;
  const float rate = -decay * softplus_f(lam[c]);
  const float cbr = br[c], cbi = bi[c];
#pragma unroll 4
  for (int j = 0; j < n; j++) {
    const int64_t t = start + j;
    const RglruCoef q = rglru_coef(gr[(int64_t)j * 2 * bw],
                                   gr[(int64_t)j * 2 * bw + bw], cbr, cbi, rate,
                                   u[t * C + c]);
    S = q.a * S + q.b;
    out[t * C + c] = from_f<T>(S * gelu_tanh_f(to_f(y[t * y_stride + c])));
  }
  // the state is read by every chunk of the sequence before any write can
  // land only if the last chunk is alone; otherwise the earlier chunks read
  // the slot in this same launch, so the last chunk writes it in a second
  // launch (see rglru_state_kernel)
  if (nch == 1) *st = S;
}

// The state after the last token of each multi-chunk sequence: fold every
// chunk summary but the last onto the old state, then walk the last chunk.
__global__ void rglru_state_kernel(
    float* __restrict__ state, const float* __restrict__ u,
    const float* __restrict__ gates, const float* __restrict__ br,
    const float* __restrict__ bi, const float* __restrict__ lam,
    const float* __restrict__ sumA, const float* __restrict__ sumB,
    const int* __restrict__ seq_start, const int* __restrict__ seq_len,
    const int* __restrict__ seq_slot, const int* __restrict__ seq_pos0,
    int Ttot, int C, int bw, float decay, int chunk, int nch) {
  const int s = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  const int len = seq_len[s];
  if (c >= C || len == 0) return;
  float* st = state + (int64_t)seq_slot[s] * C + c;
  float S = seq_pos0[s] > 0 ? *st : 0.f;
  const int last = (len - 1) / chunk;
  for (int kk = 0; kk < last; kk++)
    S = sumA[((int64_t)s * nch + kk) * C + c] * S +
        sumB[((int64_t)s * nch + kk) * C + c];
  const int start = seq_start[s] + last * chunk;
  const int n = len - last * chunk;
  const int b = c / bw, o = c - b * bw;
  const float* gr = gates + ((int64_t)b * Ttot + start) * 2 * bw + o;
  const float rate = -decay * softplus_f(lam[c]);
  const float cbr = br[c], cbi = bi[c];
  for (int j = 0; j < n; j++) {
    const RglruCoef q = rglru_coef(gr[(int64_t)j * 2 * bw],
                                   gr[(int64_t)j * 2 * bw + bw], cbr, cbi, rate,
                                   u[(int64_t)(start + j) * C + c]);
    S = q.a * S + q.b;
  }
  *st = S;
}

void check_seq(const torch::Tensor& a, int64_t n, const char* what) {
  TORCH_CHECK(a.scalar_type() == torch::kInt && a.is_contiguous() &&
                  a.numel() >= n, "seqmix: ", what, " must be int32 [>=", n, "]");
}

}  // namespace

void residual_layernorm(c10::optional<torch::Tensor> out, torch::Tensor res,
                        c10::optional<torch::Tensor> delta,
                        c10::optional<torch::Tensor> post_w, double mult,
                        c10::optional<torch::Tensor> w, double eps) {
  const int T_ = res.size(0), W = res.size(1);
  SEQ_CHECK(res.dim() == 2 && res.scalar_type() == torch::kFloat &&
                res.is_contiguous(), "res");
  SEQ_CHECK(out.has_value() == w.has_value(), "norm output needs a weight");
  SEQ_CHECK(out.has_value() || delta.has_value(), "nothing to do");
  if (out)
    SEQ_CHECK(is_act(*out) && out->is_contiguous() && out->size(0) == T_ &&
                  out->size(1) == W && w->scalar_type() == torch::kFloat &&
                  w->is_contiguous() && w->numel() == W, "norm out/weight");
  if (delta)
    SEQ_CHECK(is_act(*delta) && delta->is_contiguous() &&
                  delta->size(0) == T_ && delta->size(1) == W &&
                  (!out || delta->scalar_type() == out->scalar_type()),
              "delta");
  if (post_w)
    SEQ_CHECK(delta && post_w->scalar_type() == torch::kFloat &&
                  post_w->is_contiguous() && post_w->numel() == W,
              "post-norm weight");
  if (T_ == 0) return;
  const torch::Tensor& ty = out ? *out : *delta;
  // 256 threads with up to 8 entries each in registers (many rows), or up
  // to 1024 threads with 2-4 entries each (few rows: decoding, where the
  // row's latency counts); wider rows loop
  const int threads = W <= 512 ? row_block((W + 3) / 4)
                      : T_ <= 1024 ? std::min(1024, row_block((W + 1) / 2))
                                   : 256;
  const int ni = (W + threads - 1) / threads;
#define LN_ARGS                                                               \
  out ? ptr<T>(*out) : (T*)nullptr, ptr<float>(res),                          \
      delta ? cptr<T>(*delta) : (const T*)nullptr,                            \
      post_w ? cptr<float>(*post_w) : (const float*)nullptr, (float)mult,     \
      w ? cptr<float>(*w) : (const float*)nullptr, (float)eps, W
  DISPATCH_ACT(ty, {
    if (ni <= 4)
      hipLaunchKernelGGL((residual_layernorm_reg_kernel<T, 4>), dim3(T_),
                         dim3(threads), 0, cur_stream(), LN_ARGS);
    else if (ni <= 8)
      hipLaunchKernelGGL((residual_layernorm_reg_kernel<T, 8>), dim3(T_),
                         dim3(threads), 0, cur_stream(), LN_ARGS);
    else if (ni <= 16)
      hipLaunchKernelGGL((residual_layernorm_reg_kernel<T, 16>), dim3(T_),
                         dim3(threads), 0, cur_stream(), LN_ARGS);
    else
      hipLaunchKernelGGL(residual_layernorm_kernel<T>, dim3(T_), dim3(1024), 0,
                         cur_stream(), LN_ARGS);
  });
#undef LN_ARGS
}

void xielu(torch::Tensor out, torch::Tensor x, torch::Tensor pq) {
  SEQ_CHECK(x.is_contiguous() && out.is_contiguous() &&
                out.sizes() == x.sizes() &&
                out.scalar_type() == x.scalar_type(), "xielu shapes");
  SEQ_CHECK(pq.scalar_type() == torch::kFloat && pq.is_contiguous() &&
                pq.numel() == 2, "xielu parameters");
  const int64_t n = x.numel();
  if (n == 0) return;
  const bool vec = reinterpret_cast<uintptr_t>(x.data_ptr()) % 16 == 0 &&
                   reinterpret_cast<uintptr_t>(out.data_ptr()) % 16 == 0 &&
                   (n * x.element_size()) % 16 == 0;
  DISPATCH_ACT(x, {
    if (vec) {
      const int64_t nvec = n * sizeof(T) / 16;
      const int64_t blocks = std::min<int64_t>((nvec + 255) / 256, 8192);
      hipLaunchKernelGGL(xielu_vec_kernel<T>, dim3(blocks), dim3(256), 0,
                         cur_stream(), ptr<T>(out), cptr<T>(x),
                         cptr<float>(pq), nvec);
    } else {
      hipLaunchKernelGGL(xielu_kernel<T>, dim3((n + 255) / 256), dim3(256), 0,
                         cur_stream(), ptr<T>(out), cptr<T>(x),
                         cptr<float>(pq), n);
    }
  });
}

void rope_rows(torch::Tensor dst, int64_t dst_col, int64_t dst_vec,
               torch::Tensor src, int64_t src_col, int64_t src_vec,
               torch::Tensor positions, torch::Tensor freqs, int64_t nvec,
               int64_t len, bool interleaved) {
  const int T_ = src.size(0);
  SEQ_CHECK(freqs.dim() == 2 && freqs.size(0) == 2, "frequencies [2, dims/2]");
  const int dims = 2 * freqs.size(1);
  SEQ_CHECK(src.dim() == 2 && dst.dim() == 2 && src.stride(1) == 1 &&
                dst.stride(1) == 1 && dst.size(0) == T_ &&
                dst.scalar_type() == src.scalar_type(), "rope rows");
  SEQ_CHECK(nvec >= 0 && dims <= len && len <= src_vec && len <= dst_vec &&
                src_col >= 0 && dst_col >= 0 &&
                (nvec == 0 ||
                 (src_col + (nvec - 1) * src_vec + len <= src.size(1) &&
                  dst_col + (nvec - 1) * dst_vec + len <= dst.size(1))),
            "rope vector layout");
  SEQ_CHECK(freqs.scalar_type() == torch::kFloat && freqs.is_contiguous(),
            "rope frequencies");
  check_seq(positions, T_, "positions");
  if (T_ == 0 || nvec == 0) return;
  const bool inplace = src.data_ptr() == dst.data_ptr();
  if (inplace)
    SEQ_CHECK(src_col == dst_col && src_vec == dst_vec &&
                  src.stride(0) == dst.stride(0), "in-place rope layout");
  if (inplace && dims == 0) return;
  const int work = std::max<int64_t>(nvec * (dims / 2), nvec * (len - dims));
  DISPATCH_ACT(src, hipLaunchKernelGGL(
      rope_rows_kernel<T>, dim3(T_), dim3(std::min(row_block(work), 256)), 0,
      cur_stream(), ptr<T>(dst), (int)dst.stride(0), (int)dst_col,
      (int)dst_vec, cptr<T>(src), (int)src.stride(0), (int)src_col,
      (int)src_vec, cptr<int>(positions), cptr<float>(freqs), (int)nvec,
      (int)len, dims, interleaved ? 1 : 0, inplace ? 1 : 0););
}

void latent_append(torch::Tensor cache, torch::Tensor z, int64_t z_col,
                   torch::Tensor norm_w, torch::Tensor slot_mapping,
                   torch::Tensor positions, torch::Tensor freqs,
                   bool interleaved, double eps) {
  // cache [pages, 1, page_size, rank + rd]
  const int T_ = z.size(0);
  const int rank = norm_w.numel(), rd = cache.size(3) - rank;
  SEQ_CHECK(freqs.dim() == 2 && freqs.size(0) == 2, "frequencies [2, dims/2]");
  const int dims = 2 * freqs.size(1);
  SEQ_CHECK(cache.dim() == 4 && cache.is_contiguous() && cache.size(1) == 1 &&
                cache.scalar_type() == z.scalar_type() && rd >= 0,
            "latent cache");
  SEQ_CHECK(z.dim() == 2 && z.stride(1) == 1 && z_col >= 0 &&
                z_col + rank + rd <= z.size(1), "latent rows");
  SEQ_CHECK(norm_w.scalar_type() == torch::kFloat && norm_w.is_contiguous() &&
                freqs.scalar_type() == torch::kFloat && freqs.is_contiguous() &&
                dims <= rd, "latent norm weight / frequencies");
  SEQ_CHECK(slot_mapping.scalar_type() == torch::kLong &&
                slot_mapping.is_contiguous() && slot_mapping.numel() >= T_,
            "slot mapping");
  check_seq(positions, T_, "positions");
  if (T_ == 0) return;
  DISPATCH_ACT(z, hipLaunchKernelGGL(
      latent_append_kernel<T>, dim3(T_), dim3(std::min(row_block(rank), 256)),
      0, cur_stream(), ptr<T>(cache), cptr<T>(z), (int)z.stride(0), (int)z_col,
      cptr<float>(norm_w), cptr<int64_t>(slot_mapping), cptr<int>(positions),
      cptr<float>(freqs), rank, rd, dims, interleaved ? 1 : 0, (float)eps););
}

void diff_norm_gate(torch::Tensor out, torch::Tensor a, torch::Tensor lambda,
                    double post, c10::optional<torch::Tensor> gate,
                    double eps) {
  SEQ_CHECK(a.dim() == 4 && a.size(2) == 2 &&
                a.scalar_type() == torch::kFloat && a.is_contiguous(),
            "differential maps [T, H, 2, dv] fp32");
  const int T_ = a.size(0), H = a.size(1), dv = a.size(3);
  SEQ_CHECK(is_act(out) && out.is_contiguous() &&
                out.numel() == (int64_t)T_ * H * dv, "differential out");
  SEQ_CHECK(lambda.scalar_type() == torch::kFloat && lambda.numel() == 1,
            "lambda");
  if (gate)
    SEQ_CHECK(gate->dim() == 2 && gate->stride(1) == 1 && gate->size(0) == T_ &&
                  gate->size(1) >= H * dv &&
                  gate->scalar_type() == out.scalar_type(), "head gate");
  if (T_ == 0) return;
  DISPATCH_ACT(out, hipLaunchKernelGGL(
      diff_norm_gate_kernel<T>, dim3(T_, H), dim3(64), 0, cur_stream(),
      ptr<T>(out), cptr<float>(a), cptr<float>(lambda), (float)post,
      gate ? cptr<T>(*gate) : (const T*)nullptr,
      gate ? (int)gate->stride(0) : 0, (float)eps, H, dv););
}

void head_sigmoid_scale(torch::Tensor out, torch::Tensor x, torch::Tensor gate) {
  SEQ_CHECK(x.dim() == 3 && x.scalar_type() == torch::kFloat &&
                x.is_contiguous(), "head rows [T, H, R] fp32");
  const int T_ = x.size(0), H = x.size(1), R = x.size(2);
  SEQ_CHECK(is_act(out) && out.is_contiguous() && out.dim() == 3 &&
                out.size(0) == H && out.size(1) == T_ && out.size(2) == R,
            "head-major out [H, T, R]");
  SEQ_CHECK(gate.dim() == 2 && gate.stride(1) == 1 && gate.size(0) == T_ &&
                gate.size(1) >= H && gate.scalar_type() == out.scalar_type(),
            "per-head gate");
  if (T_ == 0) return;
  DISPATCH_ACT(out, hipLaunchKernelGGL(
      head_sigmoid_scale_kernel<T>, dim3(T_, H), dim3(std::min(row_block(R), 256)),
      0, cur_stream(), ptr<T>(out), cptr<float>(x), cptr<T>(gate),
      (int)gate.stride(0), T_, H, R););
}

void rglru_scan(torch::Tensor out, torch::Tensor u, torch::Tensor gates,
                torch::Tensor br, torch::Tensor bi, torch::Tensor lam,
                torch::Tensor y, torch::Tensor state, torch::Tensor seq_start,
                torch::Tensor seq_len, torch::Tensor seq_slot,
                torch::Tensor seq_pos0, double decay, int64_t max_len) {
  // max_len: an upper bound of the longest sequence portion of this step
  const int T_ = u.size(0), C = u.size(1);
  const int B = seq_start.size(0);
  SEQ_CHECK(u.dim() == 2 && u.scalar_type() == torch::kFloat &&
                u.is_contiguous(), "recurrence input fp32 [T, C]");
  SEQ_CHECK(gates.dim() == 3 && gates.scalar_type() == torch::kFloat &&
                gates.is_contiguous() && gates.size(1) == T_ &&
                gates.size(2) % 2 == 0 &&
                gates.size(0) * (gates.size(2) / 2) == C, "gates [nb, T, 2bw]");
  const int bw = gates.size(2) / 2;
  for (const torch::Tensor* p : {&br, &bi, &lam})
    SEQ_CHECK(p->scalar_type() == torch::kFloat && p->is_contiguous() &&
                  p->numel() == C, "per-channel parameters");
  SEQ_CHECK(is_act(y) && y.dim() == 2 && y.stride(1) == 1 && y.size(0) == T_ &&
                y.size(1) >= C, "gate branch");
  SEQ_CHECK(out.is_contiguous() && out.size(0) == T_ && out.size(1) == C &&
                out.scalar_type() == y.scalar_type(), "recurrence out");
  SEQ_CHECK(state.scalar_type() == torch::kFloat && state.is_contiguous() &&
                state.dim() == 2 && state.size(1) == C, "recurrent state");
  check_seq(seq_len, B, "seq_len");
  check_seq(seq_slot, B, "seq_slot");
  check_seq(seq_pos0, B, "seq_pos0");
  SEQ_CHECK(max_len >= 1, "longest portion");
  if (T_ == 0 || B == 0) return;
  const int threads = 64;
  const int chunk = 64;
  const int nch = (int)((std::min<int64_t>(max_len, T_) + chunk - 1) / chunk);
  const int cb = (C + threads - 1) / threads;
  torch::Tensor sums;
  const float* sumA = nullptr;
  const float* sumB = nullptr;
  if (nch > 1) {
    sums = torch::empty({2, B, nch, C}, u.options());
    sumA = cptr<float>(sums);
    sumB = sumA + (int64_t)B * nch * C;
    hipLaunchKernelGGL(rglru_chunk_summary_kernel, dim3(cb, nch, B),
                       dim3(threads), 0, cur_stream(), ptr<float>(sums),
                       ptr<float>(sums) + (int64_t)B * nch * C, cptr<float>(u),
                       cptr<float>(gates), cptr<float>(br), cptr<float>(bi),
                       cptr<float>(lam), cptr<int>(seq_start),
                       cptr<int>(seq_len), T_, C, bw, (float)decay, chunk, nch);
  }
  DISPATCH_ACT(y, hipLaunchKernelGGL(
      rglru_scan_kernel<T>, dim3(cb, nch, B), dim3(threads), 0, cur_stream(),
      ptr<T>(out), cptr<float>(u), cptr<float>(gates), cptr<float>(br),
      cptr<float>(bi), cptr<float>(lam), cptr<T>(y), (int)y.stride(0),
      ptr<float>(state), sumA, sumB, cptr<int>(seq_start), cptr<int>(seq_len),
      cptr<int>(seq_slot), cptr<int>(seq_pos0), T_, C, bw, (float)decay, chunk,
      nch););
  if (nch > 1)
    hipLaunchKernelGGL(rglru_state_kernel, dim3(cb, B), dim3(threads), 0,
                       cur_stream(), ptr<float>(state), cptr<float>(u),
                       cptr<float>(gates), cptr<float>(br), cptr<float>(bi),
                       cptr<float>(lam), sumA, sumB, cptr<int>(seq_start),
                       cptr<int>(seq_len), cptr<int>(seq_slot),
                       cptr<int>(seq_pos0), T_, C, bw, (float)decay, chunk, nch);
}
