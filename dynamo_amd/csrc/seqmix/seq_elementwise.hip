// Row-wise kernels of the sequence-mixer models: embedding, scalar-gain RMS
// norm fused with the fp32 residual add, short causal convolution (with or
// without bias and SiLU), token
// shift, per-head output norm with gate, clamped GLU, two-branch merge and
// the logit soft cap. All of them are bandwidth bound; one workgroup per
// token row, fp32 arithmetic, activations in T.
#include "seq_common.h"

namespace {

// x[t] = embed[id[t]] * scale + pos[position[t]]  (fp32 residual stream)
template <typename T>
__global__ void embed_scale_pos_kernel(float* __restrict__ out,
                                       const int* __restrict__ ids,
                                       const int* __restrict__ positions,
                                       const T* __restrict__ embed,
                                       const T* __restrict__ pos, float scale,
                                       int W, int has_pos) {
  const int t = blockIdx.x;
  const T* e = embed + (int64_t)ids[t] * W;
  const T* p = pos + (int64_t)positions[t] * W;
  for (int i = threadIdx.x; i < W; i += blockDim.x) {
    float v = to_f(e[i]) * scale;
    if (has_pos) v += to_f(p[i]);
    out[(int64_t)t * W + i] = v;
  }
}

// res += delta (when given); out = res / sqrt(mean(res^2) + eps) * g[0]
template <typename T, bool ADD>
__global__ void add_scalar_rmsnorm_kernel(T* __restrict__ out,
                                          float* __restrict__ res,
                                          const T* __restrict__ delta,
                                          const float* __restrict__ g,
                                          float eps, int W) {
  __shared__ float scratch[16];
  const int t = blockIdx.x;
  float* r = res + (int64_t)t * W;
  float ss = 0.f;
  for (int i = threadIdx.x; i < W; i += blockDim.x) {
    float v = r[i];
    if (ADD) {
      v += to_f(delta[(int64_t)t * W + i]);
      r[i] = v;
    }
    ss += v * v;
  }
  ss = block_sum(ss, scratch);
  const float inv = g[0] / sqrtf(ss / (float)W + eps);
  for (int i = threadIdx.x; i < W; i += blockDim.x)
    out[(int64_t)t * W + i] = from_f<T>(r[i] * inv);
}

// y[t, c] = act(bias[c] + sum_j w[c, j] * x[t - (taps-1) + j, c]), act =
// silu or identity, bias optional; rows before the start of this step's
// portion come from the slot's saved inputs (the last taps-1 raw inputs of
// the sequence), or are zero at position 0.
template <typename T>
__global__ void causal_conv_kernel(
    float* __restrict__ out, const T* __restrict__ x, int x_stride,
    const float* __restrict__ w, const float* __restrict__ bias, int act,
    const float* __restrict__ conv_state,
    const int* __restrict__ tok_seq, const int* __restrict__ seq_start,
    const int* __restrict__ seq_slot, const int* __restrict__ seq_pos0,
    int C, int taps) {
  const int t = blockIdx.x;
  const int s = tok_seq[t];
  const int start = seq_start[s], pos0 = seq_pos0[s];
  const float* st = conv_state + (int64_t)seq_slot[s] * (taps - 1) * C;
  const int rel = t - start;  // rows of this portion before t
  // one thread per (token, channel): the loads of a row's channels issue
  // together instead of in a workgroup's loop over the row
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c < C) {
    float acc = bias ? bias[c] : 0.f;
    for (int j = 0; j < taps; j++) {
      const int back = taps - 1 - j;  // how many tokens before t
      float xv;
      if (back <= rel) {
        xv = to_f(x[(int64_t)(t - back) * x_stride + c]);
      } else {
        // state row i holds the input (taps-1-i) tokens before the portion
        const int before = back - rel;  // 1..taps-1 tokens before the start
        xv = (pos0 - before >= 0) ? st[(int64_t)(taps - 1 - before) * C + c]
                                  : 0.f;
      }
      acc += w[c * taps + j] * xv;
    }
    out[(int64_t)t * C + c] = act ? silu_f(acc) : acc;
  }
}

// What a sublayer of a conv-fed layer reads: out = x + conv(x) over the fp32
// residual rows x [T, W], a causal per-channel convolution whose last tap
// weighs the current token. Rows before the portion come from the slot's
// saved rows (zeros before position 0).
template <typename TO, int TAPS>
__global__ void residual_conv_kernel(
    TO* __restrict__ out, const float* __restrict__ x,
    const float* __restrict__ w, const float* __restrict__ conv_state,
    const int* __restrict__ tok_seq, const int* __restrict__ seq_start,
    const int* __restrict__ seq_slot, const int* __restrict__ seq_pos0,
    int C, int taps_rt) {
  // one thread per (token, channel); TAPS > 0 fixes the tap count at
  // compile time so that the loads of all taps issue together
  const int taps = TAPS > 0 ? TAPS : taps_rt;
  const int t = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int s = tok_seq[t];
  const int start = seq_start[s], pos0 = seq_pos0[s];
  const float* st = conv_state + (int64_t)seq_slot[s] * (taps - 1) * C;
  const int rel = t - start;  // rows of this portion before t
  const float cur = x[(int64_t)t * C + c];
  float acc = cur;
#pragma unroll
  for (int j = 0; j < taps; j++) {
    const int back = taps - 1 - j;  // how many tokens before t
    float xv;
    if (back == 0) {
      xv = cur;
    } else if (back <= rel) {
      xv = x[(int64_t)(t - back) * C + c];
    } else {
      // state row i holds the input (taps-1-i) tokens before the portion
      const int before = back - rel;  // 1..taps-1 tokens before the start
      xv = (pos0 - before >= 0) ? st[(int64_t)(taps - 1 - before) * C + c]
                                : 0.f;
    }
    acc += w[c * taps + j] * xv;
  }
  out[(int64_t)t * C + c] = from_f<TO>(acc);
}

// Decoded tokens (every sequence brings one row): the waiting sublayer
// output joins the residual stream and the next sublayer's input is formed
// in one pass over the row,
//   x += LN(delta) * post_w;  out = x + conv(x);  slot rows <- shifted + x,
// with LN the weight-only layer norm (two passes over registers) and the
// convolution reading the slot's saved rows. A thread owns NI channels of
// its row, so every state entry is read and written by one thread only.
// Padding rows (seq_len 0) leave the slot alone.
template <typename T, int TAPS, int NI>
__global__ void join_conv_single_kernel(
    T* __restrict__ out, float* __restrict__ res, const T* __restrict__ delta,
    const float* __restrict__ post_w, float eps, const float* __restrict__ cw,
    float* __restrict__ conv_state, const int* __restrict__ tok_seq,
    const int* __restrict__ seq_len, const int* __restrict__ seq_slot,
    const int* __restrict__ seq_pos0, int W) {
  __shared__ float scratch[16];
  constexpr int K = TAPS - 1;
  const int t = blockIdx.x;
  const int s = tok_seq[t];
  const bool live = seq_len[s] == 1;
  const int pos0 = seq_pos0[s];
  float* st = conv_state + (int64_t)seq_slot[s] * K * W;
  float* r = res + (int64_t)t * W;
  float x[NI], hist[NI][K > 0 ? K : 1], wt[NI][TAPS], pw[NI];
  // everything the row needs is requested before the first reduction
#pragma unroll
  for (int k = 0; k < NI; k++) {
    const int i = threadIdx.x + k * blockDim.x;
    const int ic = min(i, W - 1);
    x[k] = i < W ? r[i] : 0.f;
#pragma unroll
    for (int j = 0; j < K; j++)  // row j: the input K - j tokens back
      hist[k][j] = (i < W && pos0 - (K - j) >= 0) ? st[(int64_t)j * W + i] : 0.f;
#pragma unroll
    for (int j = 0; j < TAPS; j++) wt[k][j] = cw[ic * TAPS + j];
    pw[k] = post_w ? post_w[ic] : 0.f;
  }
  if (delta) {
    const T* dl = delta + (int64_t)t * W;
    float d[NI];
    float sum = 0.f;
#pragma unroll
    for (int k = 0; k < NI; k++) {
      const int i = threadIdx.x + k * blockDim.x;
      d[k] = i < W ? to_f(dl[i]) : 0.f;
      sum += d[k];
    }
    const float mean = block_sum(sum, scratch) / (float)W;
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
      if (i < W) {
        x[k] += (d[k] - mean) * inv * pw[k];
        r[i] = x[k];
      }
    }
  }
#pragma unroll
  for (int k = 0; k < NI; k++) {
    const int i = threadIdx.x + k * blockDim.x;
    if (i >= W) continue;
    float acc = x[k] + wt[k][K] * x[k];
#pragma unroll
    for (int j = 0; j < K; j++) acc += wt[k][j] * hist[k][j];
    out[(int64_t)t * W + i] = from_f<T>(acc);
    if (live) {
#pragma unroll
      for (int j = 0; j + 1 < K; j++) st[(int64_t)j * W + i] = hist[k][j + 1];
      if (K > 0) st[(int64_t)(K - 1) * W + i] = x[k];
    }
  }
}

// After a step: the slot keeps the last taps-1 raw inputs of each sequence.
template <typename T>
__global__ void conv_state_update_kernel(
    float* __restrict__ conv_state, const T* __restrict__ x, int x_stride,
    const int* __restrict__ seq_start, const int* __restrict__ seq_len,
    const int* __restrict__ seq_slot, const int* __restrict__ seq_pos0, int C,
    int taps) {
  const int s = blockIdx.x;
  const int len = seq_len[s];
  if (len == 0) return;
  const int start = seq_start[s], pos0 = seq_pos0[s];
  float* st = conv_state + (int64_t)seq_slot[s] * (taps - 1) * C;
  const int K = taps - 1;
  for (int c = threadIdx.x; c < C; c += blockDim.x) {
    // new row i holds the input (K - i) tokens before the NEXT portion;
    // rows are filled in rising order, each reading only old rows above it
    for (int i = 0; i < K; i++) {
      const int back = K - i;  // tokens before the end of this portion
      float v;
      if (back <= len) {
        v = to_f(x[(int64_t)(start + len - back) * x_stride + c]);
      } else {
        const int before = back - len;  // tokens before this portion's start
        v = (pos0 - before >= 0) ? st[(int64_t)(K - before) * C + c] : 0.f;
      }
      st[(int64_t)i * C + c] = v;
    }
  }
}

// Token shift: mix_s[t] = h[t] + (h[t-1] - h[t]) * mu_s, S mixes at once.
// The row before a portion comes from the slot (zero at position 0).
template <typename T>
__global__ void token_shift_mix_kernel(
    T* __restrict__ out,  // [S, Ttot, W]
    const T* __restrict__ h, const float* __restrict__ mu,  // [S, W]
    const float* __restrict__ prev_state,                   // [slots, W]
    const int* __restrict__ tok_seq, const int* __restrict__ seq_start,
    const int* __restrict__ seq_slot, const int* __restrict__ seq_pos0,
    int Ttot, int W, int S) {
  const int t = blockIdx.x;
  const int s = tok_seq[t];
  const bool first = (t == seq_start[s]);
  const bool zero = first && seq_pos0[s] == 0;
  const float* ps = prev_state + (int64_t)seq_slot[s] * W;
  for (int i = threadIdx.x; i < W; i += blockDim.x) {
    const float cur = to_f(h[(int64_t)t * W + i]);
    const float prev =
        zero ? 0.f : (first ? ps[i] : to_f(h[(int64_t)(t - 1) * W + i]));
    for (int k = 0; k < S; k++)
      out[((int64_t)k * Ttot + t) * W + i] =
          from_f<T>(cur + (prev - cur) * mu[k * W + i]);
  }
}

template <typename T>
__global__ void shift_state_update_kernel(
    float* __restrict__ prev_state, const T* __restrict__ h,
    const int* __restrict__ seq_start, const int* __restrict__ seq_len,
    const int* __restrict__ seq_slot, int W) {
  const int s = blockIdx.x;
  const int len = seq_len[s];
  if (len == 0) return;
  const T* last = h + (int64_t)(seq_start[s] + len - 1) * W;
  float* ps = prev_state + (int64_t)seq_slot[s] * W;
  for (int i = threadIdx.x; i < W; i += blockDim.x) ps[i] = to_f(last[i]);
}

// y[t, h, :] = o[t, h, :] / rms(o[t, h, :]) * w[h * w_stride + :] * act(gate)
// gate_act: 0 none, 1 silu, 2 sigmoid. One wave per (token, head).
template <typename T>
__global__ void head_norm_gate_kernel(T* __restrict__ out,
                                      const float* __restrict__ o,
                                      const float* __restrict__ w, int w_stride,
                                      const T* __restrict__ gate,
                                      int gate_stride, int gate_act, float eps,
                                      int H, int dv) {
  const int t = blockIdx.x, hh = blockIdx.y, lane = threadIdx.x;
  const float* src = o + ((int64_t)t * H + hh) * dv;
  float ss = 0.f;
  for (int i = lane; i < dv; i += 64) ss += src[i] * src[i];
  ss = wave_sum(ss);
  const float inv = 1.f / sqrtf(ss / (float)dv + eps);
  for (int i = lane; i < dv; i += 64) {
    float v = src[i] * inv * w[hh * w_stride + i];
    if (gate_act) {
      const float gr = to_f(gate[(int64_t)t * gate_stride + hh * dv + i]);
      v *= (gate_act == 1) ? silu_f(gr) : sigmoid_f(gr);
    }
    out[((int64_t)t * H + hh) * dv + i] = from_f<T>(v);
  }
}

// g = min(gate, L); u = clamp(up, -L, L); y = g * sigmoid(alpha g) * (u + 1)
template <typename T>
__global__ void clamped_glu_kernel(T* __restrict__ out,
                                   const T* __restrict__ gate_up, int F,
                                   float limit, float alpha, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const int64_t t = i / F;
  const int c = (int)(i - t * F);
  const float g = fminf(to_f(gate_up[t * 2 * F + c]), limit);
  const float u = fminf(fmaxf(to_f(gate_up[t * 2 * F + F + c]), -limit), limit);
  out[i] = from_f<T>(g * sigmoid_f(alpha * g) * (u + 1.f));
}

// out = 0.5 * (a / rms(a) * wa + b / rms(b) * wb)
template <typename T>
__global__ void dual_rmsnorm_mean_kernel(T* __restrict__ out,
                                         const T* __restrict__ a,
                                         const T* __restrict__ b,
                                         const float* __restrict__ wa,
                                         const float* __restrict__ wb,
                                         float eps, int W) {
  __shared__ float scratch[16];
  const int t = blockIdx.x;
  float sa = 0.f, sb = 0.f;
  for (int i = threadIdx.x; i < W; i += blockDim.x) {
    const float x = to_f(a[(int64_t)t * W + i]);
    const float y = to_f(b[(int64_t)t * W + i]);
    sa += x * x;
    sb += y * y;
  }
  sa = block_sum(sa, scratch);
  sb = block_sum(sb, scratch);
  const float ia = 1.f / sqrtf(sa / (float)W + eps);
  const float ib = 1.f / sqrtf(sb / (float)W + eps);
  for (int i = threadIdx.x; i < W; i += blockDim.x) {
    const float x = to_f(a[(int64_t)t * W + i]) * ia * wa[i];
    const float y = to_f(b[(int64_t)t * W + i]) * ib * wb[i];
    out[(int64_t)t * W + i] = from_f<T>(0.5f * (x + y));
  }
}

__global__ void softcap_kernel(float* __restrict__ x, float cap, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) x[i] = cap * tanhf(x[i] / cap);
}

inline int row_block(int W) {
  int b = 64;
  while (b < W && b < 1024) b <<= 1;
  return b;
}

}  // namespace

void embed_scale_pos(torch::Tensor out, torch::Tensor ids,
                     torch::Tensor positions, torch::Tensor embed,
                     c10::optional<torch::Tensor> pos, double scale) {
  const int T_ = ids.size(0), W = embed.size(1);
  SEQ_CHECK(out.scalar_type() == torch::kFloat && out.is_contiguous() &&
                out.size(0) == T_ && out.size(1) == W, "embed out");
  SEQ_CHECK(ids.scalar_type() == torch::kInt &&
                positions.scalar_type() == torch::kInt &&
                positions.size(0) == T_, "embed ids/positions int32");
  SEQ_CHECK(embed.is_contiguous(), "embed table");
  if (pos) SEQ_CHECK(pos->is_contiguous() && pos->size(1) == W &&
                         pos->scalar_type() == embed.scalar_type(), "pos table");
  if (T_ == 0) return;
  DISPATCH_ACT(embed, hipLaunchKernelGGL(
      embed_scale_pos_kernel<T>, dim3(T_), dim3(row_block(W)), 0, cur_stream(),
      ptr<float>(out), cptr<int>(ids), cptr<int>(positions), cptr<T>(embed),
      pos ? cptr<T>(*pos) : cptr<T>(embed), (float)scale, W, pos ? 1 : 0););
}

void add_scalar_rmsnorm(torch::Tensor out, torch::Tensor res,
                        c10::optional<torch::Tensor> delta, torch::Tensor g,
                        double eps) {
  const int T_ = res.size(0), W = res.size(1);
  SEQ_CHECK(res.scalar_type() == torch::kFloat && res.is_contiguous(), "res");
  SEQ_CHECK(out.is_contiguous() && out.size(0) == T_ && out.size(1) == W, "out");
  SEQ_CHECK(g.scalar_type() == torch::kFloat && g.numel() == 1, "gain");
  if (delta)
    SEQ_CHECK(delta->is_contiguous() && delta->size(0) == T_ &&
                  delta->size(1) == W &&
                  delta->scalar_type() == out.scalar_type(), "delta");
  if (T_ == 0) return;
  DISPATCH_ACT(out, {
    if (delta)
      hipLaunchKernelGGL((add_scalar_rmsnorm_kernel<T, true>), dim3(T_),
                         dim3(row_block(W)), 0, cur_stream(), ptr<T>(out),
                         ptr<float>(res), cptr<T>(*delta), cptr<float>(g),
                         (float)eps, W);
    else
      hipLaunchKernelGGL((add_scalar_rmsnorm_kernel<T, false>), dim3(T_),
                         dim3(row_block(W)), 0, cur_stream(), ptr<T>(out),
                         ptr<float>(res), (const T*)nullptr, cptr<float>(g),
                         (float)eps, W);
  });
}

static void check_seq(const torch::Tensor& a, int64_t n, const char* what) {
  TORCH_CHECK(a.scalar_type() == torch::kInt && a.is_contiguous() &&
                  a.numel() >= n, "seqmix: ", what, " must be int32 [>=", n, "]");
}

void causal_conv(torch::Tensor out, torch::Tensor x, torch::Tensor w,
                 c10::optional<torch::Tensor> bias, bool silu,
                 torch::Tensor conv_state, torch::Tensor tok_seq,
                 torch::Tensor seq_start, torch::Tensor seq_len,
                 torch::Tensor seq_slot, torch::Tensor seq_pos0) {
  // x: [T, >=C] rows of stride x.stride(0); the first C columns convolve
  const int T_ = x.size(0), C = w.size(0), taps = w.size(1);
  const int B = seq_start.size(0);
  SEQ_CHECK(x.stride(1) == 1 && x.size(1) >= C, "conv input");
  SEQ_CHECK(out.scalar_type() == torch::kFloat && out.is_contiguous() &&
                out.size(0) == T_ && out.size(1) == C, "conv out");
  SEQ_CHECK(w.scalar_type() == torch::kFloat && w.is_contiguous(), "conv w");
  if (bias)
    SEQ_CHECK(bias->scalar_type() == torch::kFloat && bias->is_contiguous() &&
                  bias->numel() == C, "conv bias");
  SEQ_CHECK(conv_state.scalar_type() == torch::kFloat &&
                conv_state.is_contiguous() && conv_state.size(1) == taps - 1 &&
                conv_state.size(2) == C, "conv state");
  check_seq(tok_seq, T_, "tok_seq");
  check_seq(seq_len, B, "seq_len");
  check_seq(seq_slot, B, "seq_slot");
  check_seq(seq_pos0, B, "seq_pos0");
  if (T_ == 0) return;
  DISPATCH_ACT(x, {
    hipLaunchKernelGGL(causal_conv_kernel<T>, dim3(T_, (C + 255) / 256),
                       dim3(256), 0, cur_stream(), ptr<float>(out), cptr<T>(x),
                       (int)x.stride(0), cptr<float>(w),
                       bias ? cptr<float>(*bias) : (const float*)nullptr,
                       silu ? 1 : 0, cptr<float>(conv_state),
                       cptr<int>(tok_seq),
                       cptr<int>(seq_start), cptr<int>(seq_slot),
                       cptr<int>(seq_pos0), C, taps);
    if (taps > 1)
      hipLaunchKernelGGL(conv_state_update_kernel<T>, dim3(B),
                         dim3(row_block(C)), 0, cur_stream(),
                         ptr<float>(conv_state), cptr<T>(x), (int)x.stride(0),
                         cptr<int>(seq_start), cptr<int>(seq_len),
                         cptr<int>(seq_slot), cptr<int>(seq_pos0), C, taps);
  });
}

void residual_conv(torch::Tensor out, torch::Tensor x, torch::Tensor w,
                   torch::Tensor conv_state, torch::Tensor tok_seq,
                   torch::Tensor seq_start, torch::Tensor seq_len,
                   torch::Tensor seq_slot, torch::Tensor seq_pos0) {
  // x: fp32 [T, C]; out [T, C] = x + conv(x) in the activation type
  const int T_ = x.size(0), C = w.size(0), taps = w.size(1);
  const int B = seq_start.size(0);
  SEQ_CHECK(x.dim() == 2 && x.scalar_type() == torch::kFloat &&
                x.is_contiguous() && x.size(1) == C, "conv input fp32 [T, C]");
  SEQ_CHECK(is_act(out) && out.is_contiguous() && out.size(0) == T_ &&
                out.size(1) == C, "conv out");
  SEQ_CHECK(w.scalar_type() == torch::kFloat && w.is_contiguous() && taps >= 1,
            "conv w");
  SEQ_CHECK(conv_state.scalar_type() == torch::kFloat &&
                conv_state.is_contiguous() && conv_state.dim() == 3 &&
                conv_state.size(1) == taps - 1 && conv_state.size(2) == C,
            "conv state");
  check_seq(tok_seq, T_, "tok_seq");
  check_seq(seq_len, B, "seq_len");
  check_seq(seq_slot, B, "seq_slot");
  check_seq(seq_pos0, B, "seq_pos0");
  if (T_ == 0) return;
  const int threads = std::min(256, row_block(C));
  const dim3 grid(T_, (C + threads - 1) / threads);
#define CONV_LAUNCH(TAPS_)                                                   \
  hipLaunchKernelGGL((residual_conv_kernel<T, TAPS_>), grid, dim3(threads),  \
                     0, cur_stream(), ptr<T>(out), cptr<float>(x),           \
                     cptr<float>(w), cptr<float>(conv_state),                \
                     cptr<int>(tok_seq), cptr<int>(seq_start),               \
                     cptr<int>(seq_slot), cptr<int>(seq_pos0), C, taps)
  DISPATCH_ACT(out, {
    if (taps == 4) CONV_LAUNCH(4);
    else if (taps == 2) CONV_LAUNCH(2);
    else if (taps == 3) CONV_LAUNCH(3);
    else CONV_LAUNCH(0);
  });
#undef CONV_LAUNCH
  if (taps > 1)
    hipLaunchKernelGGL(conv_state_update_kernel<float>, dim3(B),
                       dim3(row_block(C)), 0, cur_stream(),
                       ptr<float>(conv_state), cptr<float>(x), C,
                       cptr<int>(seq_start), cptr<int>(seq_len),
                       cptr<int>(seq_slot), cptr<int>(seq_pos0), C, taps);
}

// One row per sequence (decoded tokens). delta/post_w absent: the stream is
// taken as it is. Returns false (nothing done) for sizes the fused kernel
// is not built for; the caller then takes the separate kernels.
bool join_conv_single(torch::Tensor out, torch::Tensor res,
                      c10::optional<torch::Tensor> delta,
                      c10::optional<torch::Tensor> post_w, double eps,
                      torch::Tensor w, torch::Tensor conv_state,
                      torch::Tensor tok_seq, torch::Tensor seq_len,
                      torch::Tensor seq_slot, torch::Tensor seq_pos0) {
  const int T_ = res.size(0), W = res.size(1), taps = w.size(1);
  const int B = seq_len.size(0);
  if (taps < 1 || taps > 4 || W > 8192) return false;
  SEQ_CHECK(res.dim() == 2 && res.scalar_type() == torch::kFloat &&
                res.is_contiguous(), "res");
  SEQ_CHECK(is_act(out) && out.is_contiguous() && out.size(0) == T_ &&
                out.size(1) == W, "conv out");
  SEQ_CHECK(delta.has_value() == post_w.has_value(), "delta and its weight");
  if (delta)
    SEQ_CHECK(delta->is_contiguous() && delta->size(0) == T_ &&
                  delta->size(1) == W &&
                  delta->scalar_type() == out.scalar_type() &&
                  post_w->scalar_type() == torch::kFloat &&
                  post_w->is_contiguous() && post_w->numel() == W, "delta");
  SEQ_CHECK(w.scalar_type() == torch::kFloat && w.is_contiguous() &&
                w.size(0) == W, "conv w");
  SEQ_CHECK(conv_state.scalar_type() == torch::kFloat &&
                conv_state.is_contiguous() && conv_state.dim() == 3 &&
                conv_state.size(1) == taps - 1 && conv_state.size(2) == W,
            "conv state");
  check_seq(tok_seq, T_, "tok_seq");
  check_seq(seq_len, B, "seq_len");
  check_seq(seq_slot, B, "seq_slot");
  check_seq(seq_pos0, B, "seq_pos0");
  if (T_ == 0) return true;
  const int threads = std::min(1024, row_block((W + 3) / 4));
  const int ni = (W + threads - 1) / threads;
#define JC_LAUNCH(TAPS_, NI_)                                                \
  hipLaunchKernelGGL((join_conv_single_kernel<T, TAPS_, NI_>), dim3(T_),     \
                     dim3(threads), 0, cur_stream(), ptr<T>(out),            \
                     ptr<float>(res),                                        \
                     delta ? cptr<T>(*delta) : (const T*)nullptr,            \
                     post_w ? cptr<float>(*post_w) : (const float*)nullptr,  \
                     (float)eps, cptr<float>(w), ptr<float>(conv_state),     \
                     cptr<int>(tok_seq), cptr<int>(seq_len),                 \
                     cptr<int>(seq_slot), cptr<int>(seq_pos0), W)
#define JC_TAPS(NI_)                                                         \
  do {                                                                       \
    if (taps == 4) JC_LAUNCH(4, NI_);                                        \
    else if (taps == 3) JC_LAUNCH(3, NI_);                                   \
    else if (taps == 2) JC_LAUNCH(2, NI_);                                   \
    else JC_LAUNCH(1, NI_);                                                  \
  } while (0)
  DISPATCH_ACT(out, {
    if (ni <= 4) JC_TAPS(4);
    else JC_TAPS(8);
  });
#undef JC_TAPS
#undef JC_LAUNCH
  return true;
}

void causal_conv_silu(torch::Tensor out, torch::Tensor x, torch::Tensor w,
                      torch::Tensor conv_state, torch::Tensor tok_seq,
                      torch::Tensor seq_start, torch::Tensor seq_len,
                      torch::Tensor seq_slot, torch::Tensor seq_pos0) {
  causal_conv(out, x, w, c10::nullopt, true, conv_state, tok_seq, seq_start,
              seq_len, seq_slot, seq_pos0);
}

void token_shift_mix(torch::Tensor out, torch::Tensor h, torch::Tensor mu,
                     torch::Tensor prev_state, torch::Tensor tok_seq,
                     torch::Tensor seq_start, torch::Tensor seq_len,
                     torch::Tensor seq_slot, torch::Tensor seq_pos0) {
  const int T_ = h.size(0), W = h.size(1), S = mu.size(0);
  const int B = seq_start.size(0);
  SEQ_CHECK(h.is_contiguous() && out.is_contiguous() &&
                out.scalar_type() == h.scalar_type() && out.size(0) == S &&
                out.size(1) == T_ && out.size(2) == W, "shift out");
  SEQ_CHECK(mu.scalar_type() == torch::kFloat && mu.is_contiguous() &&
                mu.size(1) == W, "shift mu");
  SEQ_CHECK(prev_state.scalar_type() == torch::kFloat &&
                prev_state.is_contiguous() && prev_state.size(1) == W,
            "shift state");
  check_seq(tok_seq, T_, "tok_seq");
  check_seq(seq_len, B, "seq_len");
  check_seq(seq_slot, B, "seq_slot");
  check_seq(seq_pos0, B, "seq_pos0");
  if (T_ == 0) return;
  DISPATCH_ACT(h, {
    hipLaunchKernelGGL(token_shift_mix_kernel<T>, dim3(T_), dim3(row_block(W)),
                       0, cur_stream(), ptr<T>(out), cptr<T>(h),
                       cptr<float>(mu), cptr<float>(prev_state),
                       cptr<int>(tok_seq), cptr<int>(seq_start),
                       cptr<int>(seq_slot), cptr<int>(seq_pos0), T_, W, S);
    hipLaunchKernelGGL(shift_state_update_kernel<T>, dim3(B),
                       dim3(row_block(W)), 0, cur_stream(),
                       ptr<float>(prev_state), cptr<T>(h), cptr<int>(seq_start),
                       cptr<int>(seq_len), cptr<int>(seq_slot), W);
  });
}

void head_norm_gate(torch::Tensor out, torch::Tensor o, torch::Tensor w,
                    int64_t w_stride, c10::optional<torch::Tensor> gate,
                    int64_t gate_act, double eps) {
  // o [T, H, dv] fp32; gate [T, >=H*dv] strided rows (column 0 = head 0)
  const int T_ = o.size(0), H = o.size(1), dv = o.size(2);
  SEQ_CHECK(o.scalar_type() == torch::kFloat && o.is_contiguous(), "head o");
  SEQ_CHECK(out.is_contiguous() && out.numel() == o.numel(), "head out");
  SEQ_CHECK(w.scalar_type() == torch::kFloat && w.is_contiguous() &&
                w.numel() >= (H - 1) * w_stride + dv, "head weight");
  SEQ_CHECK(gate_act == 0 || gate.has_value(), "gate missing");
  if (gate)
    SEQ_CHECK(gate->stride(1) == 1 && gate->size(0) == T_ &&
                  gate->size(1) >= H * dv &&
                  gate->scalar_type() == out.scalar_type(), "head gate");
  if (T_ == 0) return;
  DISPATCH_ACT(out, hipLaunchKernelGGL(
      head_norm_gate_kernel<T>, dim3(T_, H), dim3(64), 0, cur_stream(),
      ptr<T>(out), cptr<float>(o), cptr<float>(w), (int)w_stride,
      gate ? cptr<T>(*gate) : (const T*)nullptr,
      gate ? (int)gate->stride(0) : 0, (int)gate_act, (float)eps, H, dv););
}

void clamped_glu(torch::Tensor out, torch::Tensor gate_up, double limit,
                 double alpha) {
  const int64_t T_ = gate_up.size(0);
  const int F = gate_up.size(1) / 2;
  SEQ_CHECK(gate_up.is_contiguous() && out.is_contiguous() &&
                out.size(0) == T_ && out.size(1) == F &&
                out.scalar_type() == gate_up.scalar_type(), "glu shapes");
  const int64_t n = T_ * F;
  if (n == 0) return;
  DISPATCH_ACT(out, hipLaunchKernelGGL(
      clamped_glu_kernel<T>, dim3((n + 255) / 256), dim3(256), 0, cur_stream(),
      ptr<T>(out), cptr<T>(gate_up), F, (float)limit, (float)alpha, n););
}

void dual_rmsnorm_mean(torch::Tensor out, torch::Tensor a, torch::Tensor b,
                       torch::Tensor wa, torch::Tensor wb, double eps) {
  const int T_ = a.size(0), W = a.size(1);
  SEQ_CHECK(a.is_contiguous() && b.is_contiguous() && out.is_contiguous() &&
                b.sizes() == a.sizes() && out.sizes() == a.sizes() &&
                a.scalar_type() == b.scalar_type() &&
                a.scalar_type() == out.scalar_type(), "merge shapes");
  SEQ_CHECK(wa.scalar_type() == torch::kFloat && wa.numel() == W &&
                wb.scalar_type() == torch::kFloat && wb.numel() == W,
            "merge weights");
  if (T_ == 0) return;
  DISPATCH_ACT(out, hipLaunchKernelGGL(
      dual_rmsnorm_mean_kernel<T>, dim3(T_), dim3(row_block(W)), 0,
      cur_stream(), ptr<T>(out), cptr<T>(a), cptr<T>(b), cptr<float>(wa),
      cptr<float>(wb), (float)eps, W););
}

void softcap_(torch::Tensor x, double cap) {
  SEQ_CHECK(x.scalar_type() == torch::kFloat && x.is_contiguous(), "softcap");
  const int64_t n = x.numel();
  if (n == 0) return;
  hipLaunchKernelGGL(softcap_kernel, dim3((n + 255) / 256), dim3(256), 0,
                     cur_stream(), ptr<float>(x), (float)cap, n);
}
