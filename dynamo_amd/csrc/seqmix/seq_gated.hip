// Kernels for layer-list models with RMS-normed, partially rotated query and
// key heads written straight into the paged cache, a minimal gated
// recurrent unit, and a routed mixture of small feed-forward experts with
// identity experts. All arithmetic is fp32; activations that feed a matrix
// product are T (float or bf16).
#include "seq_common.h"

namespace {

void check_ints(const torch::Tensor& a, int64_t n, const char* what) {
  TORCH_CHECK(a.scalar_type() == torch::kInt && a.is_contiguous() &&
                  a.numel() >= n, "seqmix: ", what, " must be int32 [>=", n, "]");
}

// ---- normed, rotated heads -------------------------------------------------
// One wave per (token, vector): vectors 0..H-1 are the query heads (normed
// and rotated in place), H..H+G-1 the key heads (normed, rotated, written to
// the token's cache slot), H+G..H+2G-1 the value heads (copied to the slot).
// Norm: x / sqrt(mean(x^2) + eps) * w with one weight vector for all heads
// of a kind. Rotation of the first `dims` entries at angle position * f_i,
// pairs (i, i + dims/2) or (2i, 2i+1).
template <typename T>
__global__ __launch_bounds__(256) void headnorm_rope_append_kernel(
    T* __restrict__ proj, int stride, int H, int G, int dk, int dv, int off_k,
    int off_v, const float* __restrict__ qw, const float* __restrict__ kw,
    const float* __restrict__ freqs, int dims, int interleaved, float eps,
    const int* __restrict__ positions, T* __restrict__ kcache,
    T* __restrict__ vcache, const int64_t* __restrict__ slot_mapping, int ps) {
  const int t = blockIdx.x, lane = threadIdx.x & 63;
  const int vi = blockIdx.y * 4 + (threadIdx.x >> 6);
  if (vi >= H + 2 * G) return;
  T* row = proj + (int64_t)t * stride;
  const int64_t slot = slot_mapping[t];
  const int64_t page = slot / ps, inpage = slot % ps;
  if (vi >= H + G) {
    if (slot < 0) return;
    const int g = vi - H - G;
    const T* v = row + off_v + g * dv;
    T* d = vcache + ((page * G + g) * ps + inpage) * dv;
    for (int i = lane; i < dv; i += 64) d[i] = v[i];
    return;
  }
  const bool isq = vi < H;
  if (!isq && slot < 0) return;
  const T* src = isq ? row + vi * dk : row + off_k + (vi - H) * dk;
  T* dst = isq ? row + vi * dk
               : kcache + ((page * G + (vi - H)) * ps + inpage) * dk;
  const float* w = isq ? qw : kw;
  float ss = 0.f;
  for (int i = lane; i < dk; i += 64) {
    const float x = to_f(src[i]);
    ss += x * x;
  }
  const float inv = 1.f / sqrtf(wave_sum(ss) / (float)dk + eps);
  const float pos = (float)positions[t];
  const int half = dims >> 1;
  for (int i = lane; i < half; i += 64) {
    const int ia = interleaved ? 2 * i : i;
    const int ib = interleaved ? 2 * i + 1 : i + half;
    float ra, rb;
    rot_pair(to_f(src[ia]) * inv * w[ia], to_f(src[ib]) * inv * w[ib], pos,
             freqs[i], freqs[half + i], ra, rb);
    dst[ia] = from_f<T>(ra);
    dst[ib] = from_f<T>(rb);
  }
  for (int i = dims + lane; i < dk; i += 64)
    dst[i] = from_f<T>(to_f(src[i]) * inv * w[i]);
}

// ---- minimal gated recurrent unit -------------------------------------------
// Per channel: z = sigmoid(zr), S <- (1 - z) S + z c(ur), c(u) = u + 1/2 for
// u >= 0 and sigmoid(u) below; out = S * silu(g). proj rows hold zr | ur | g
// (C each). The recurrence is linear in S, so a long portion is cut into
// chunks that run in parallel: a first kernel reduces every chunk but the
// last to (A, B) with S_end = A S_begin + B, the scan kernel of chunk k
// folds the summaries before it onto the slot's state, and a third launch
// writes the slot (so that no chunk reads a state another has advanced).
// Decoded tokens and short portions are one chunk and one launch.
struct Coef {
  float a, b;
};
DEVINL Coef mingru_coef(float zr, float ur) {
  Coef c;
  c.a = sigmoid_f(-zr);  // 1 - z without cancellation
  c.b = sigmoid_f(zr) * (ur >= 0.f ? ur + 0.5f : sigmoid_f(ur));
  return c;
}

template <typename T>
__global__ void mingru_chunk_summary_kernel(
    float* __restrict__ sumA, float* __restrict__ sumB,  // [B, nch, C]
    const T* __restrict__ proj, int stride, const int* __restrict__ seq_start,
    const int* __restrict__ seq_len, int C, int chunk, int nch) {
  const int s = blockIdx.z, k = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  const int len = seq_len[s];
  // the last chunk of a sequence carries into nothing
  if (c >= C || (k + 1) * chunk >= len) return;
  const T* p = proj + (int64_t)(seq_start[s] + k * chunk) * stride + c;
  float A = 1.f, S = 0.f;
#pragma unroll 4
  for (int j = 0; j < chunk; j++) {
    const Coef q = mingru_coef(to_f(p[(int64_t)j * stride]),
                               to_f(p[(int64_t)j * stride + C]));
    A *= q.a;
    S = q.a * S + q.b;
  }
  sumA[((int64_t)s * nch + k) * C + c] = A;
  sumB[((int64_t)s * nch + k) * C + c] = S;
}

template <typename T>
__global__ void mingru_scan_kernel(
    T* __restrict__ out, const T* __restrict__ proj, int stride,
    float* __restrict__ state, const float* __restrict__ sumA,
    const float* __restrict__ sumB, const int* __restrict__ seq_start,
    const int* __restrict__ seq_len, const int* __restrict__ seq_slot,
    const int* __restrict__ seq_pos0, int C, int chunk, int nch) {
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
  const T* p = proj + (int64_t)start * stride + c;
#pragma unroll 4
  for (int j = 0; j < n; j++) {
    const T* r = p + (int64_t)j * stride;
    const Coef q = mingru_coef(to_f(r[0]), to_f(r[C]));
    S = q.a * S + q.b;
    out[(int64_t)(start + j) * C + c] = from_f<T>(S * silu_f(to_f(r[2 * C])));
  }
  if (nch == 1) *st = S;
}

template <typename T>
__global__ void mingru_state_kernel(
    float* __restrict__ state, const T* __restrict__ proj, int stride,
    const float* __restrict__ sumA, const float* __restrict__ sumB,
    const int* __restrict__ seq_start, const int* __restrict__ seq_len,
    const int* __restrict__ seq_slot, const int* __restrict__ seq_pos0, int C,
    int chunk, int nch) {
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
  const T* p = proj + (int64_t)(seq_start[s] + last * chunk) * stride + c;
  const int n = len - last * chunk;
  for (int j = 0; j < n; j++) {
    const Coef q = mingru_coef(to_f(p[(int64_t)j * stride]),
                               to_f(p[(int64_t)j * stride + C]));
    S = q.a * S + q.b;
  }
  *st = S;
}

// ---- squared relu -----------------------------------------------------------
DEVINL float relu2_f(float z) {
  const float r = fmaxf(z, 0.f);
  return r * r;
}
// 16 bytes per thread and step
template <typename T>
__global__ void relu_squared_vec_kernel(T* __restrict__ out,
                                        const T* __restrict__ x, int64_t nvec) {
  constexpr int N = 16 / sizeof(T);
  union V { uint4 raw; T e[N]; };
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < nvec;
       i += (int64_t)gridDim.x * blockDim.x) {
    V v, o;
    v.raw = reinterpret_cast<const uint4*>(x)[i];
#pragma unroll
    for (int k = 0; k < N; k++) o.e[k] = from_f<T>(relu2_f(to_f(v.e[k])));
    reinterpret_cast<uint4*>(out)[i] = o.raw;
  }
}
template <typename T>
__global__ void relu_squared_kernel(T* __restrict__ out,
                                    const T* __restrict__ x, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) out[i] = from_f<T>(relu2_f(to_f(x[i])));
}

// ---- router -------------------------------------------------------------------
// LDS written by some lanes of a wave is read by others of the same wave
DEVINL void wave_sync() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// (value, index) maximum over a wave; ties go to the lower index
DEVINL void wave_argmax(float& v, int& i) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    const float ov = __shfl_xor(v, off, 64);
    const int oi = __shfl_xor(i, off, 64);
    if (ov > v || (ov == v && oi < i)) {
      v = ov;
      i = oi;
    }
  }
}

// One wave per token. s = softmax(logits) over all n outputs; choice =
// s + correction; a group's score is the largest choice score among its
// n / groups neighbouring outputs; outputs outside the `keep` best groups
// are out of the running; the `top` largest remaining choices are taken in
// falling order and weigh in with s * scale.
// LDS per wave: s [n], choice [n], group score [groups].
// The logits are given (fp32 [T, n]; a wave per token, four tokens per
// workgroup), or - FUSED, for few rows - formed here as the fp32 products of
// the token's input h [W] (activation type) with the router's fp32 rows
// [n, W]: then a workgroup owns one token, all its threads share the
// channels, eight outputs at a time, and its first wave routes.
template <typename T, bool FUSED>
__global__ __launch_bounds__(256) void moe_route_kernel(
    int* __restrict__ idx, float* __restrict__ wgt,
    const float* __restrict__ logits, const T* __restrict__ h,
    const float* __restrict__ router, int W,
    const float* __restrict__ correction,
    int T_, int n, int groups, int keep, int top, float scale) {
  extern __shared__ float lds[];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int t = FUSED ? blockIdx.x : blockIdx.x * 4 + wave;
  if (t >= T_) return;
  float* sc = lds + (FUSED ? 0 : wave) * (2 * n + groups);
  float* ch = sc + n;
  float* gs = ch + n;
  if (!FUSED) {
    for (int i = lane; i < n; i += 64) ch[i] = logits[(int64_t)t * n + i];
  } else {
    __shared__ float part[4][8];
    const T* hr = h + (int64_t)t * W;
    for (int i0 = 0; i0 < n; i0 += 8) {
      float acc[8];
#pragma unroll
      for (int u = 0; u < 8; u++) acc[u] = 0.f;
#pragma unroll 2
      for (int c = threadIdx.x; c < W; c += 256) {
        const float hv = to_f(hr[c]);
#pragma unroll
        for (int u = 0; u < 8; u++)
          acc[u] += hv * router[(int64_t)min(i0 + u, n - 1) * W + c];
      }
#pragma unroll
      for (int u = 0; u < 8; u++) {
        const float v = wave_sum(acc[u]);
        if (lane == 0) part[wave][u] = v;
      }
      __syncthreads();
      if (threadIdx.x < 8 && i0 + threadIdx.x < n)
        ch[i0 + threadIdx.x] = (part[0][threadIdx.x] + part[1][threadIdx.x]) +
                               (part[2][threadIdx.x] + part[3][threadIdx.x]);
      __syncthreads();
    }
    if (wave != 0) return;
  }
  wave_sync();
  const float* z = ch;  // raw logits, replaced by the choice scores below
  float mx = -INFINITY;
  for (int i = lane; i < n; i += 64) mx = fmaxf(mx, z[i]);
  mx = wave_max(mx);
  float sum = 0.f;
  for (int i = lane; i < n; i += 64) {
    const float e = expf(z[i] - mx);
    sc[i] = e;
    sum += e;
  }
  const float inv = 1.f / wave_sum(sum);
  for (int i = lane; i < n; i += 64) {
    const float s = sc[i] * inv;
    sc[i] = s;
    ch[i] = s + correction[i];
  }
  wave_sync();
  if (groups > 1) {
    const int gsz = n / groups;
    for (int g = lane; g < groups; g += 64) {
      float m = -INFINITY;
      for (int i = 0; i < gsz; i++) m = fmaxf(m, ch[g * gsz + i]);
      gs[g] = m;
    }
    wave_sync();
    // take the best groups out one by one (marked with +inf), then drop
    // the outputs of every group that was not taken
    for (int r = 0; r < keep; r++) {
      float bv = -INFINITY;
      int bi = 0x7fffffff;
      for (int g = lane; g < groups; g += 64) {
        const float v = gs[g];
        if (v != INFINITY && (v > bv || bi == 0x7fffffff)) {
          bv = v;
          bi = g;
        }
      }
      wave_argmax(bv, bi);
      if (lane == 0 && bi != 0x7fffffff) gs[bi] = INFINITY;
      wave_sync();
    }
    for (int i = lane; i < n; i += 64)
      if (gs[i / gsz] != INFINITY) ch[i] = -INFINITY;
    wave_sync();
  }
  for (int r = 0; r < top; r++) {
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    for (int i = lane; i < n; i += 64) {
      const float v = ch[i];
      // NaN marks an output that is already taken
      if (v == v && (v > bv || bi == 0x7fffffff)) {
        bv = v;
        bi = i;
      }
    }
    wave_argmax(bv, bi);
    if (bi == 0x7fffffff) bi = 0;  // fewer candidates than `top`: checked on the host
    if (lane == 0) {
      idx[(int64_t)t * top + r] = bi;
      wgt[(int64_t)t * top + r] = sc[bi] * scale;
      ch[bi] = __builtin_nanf("");
    }
    wave_sync();
  }
}

// Workgroup e walks all entries of idx in order: rank[i] = how many earlier
// entries chose output e, for the entries that chose it; counts[e] = total.
__global__ __launch_bounds__(256) void moe_dispatch_kernel(
    int* __restrict__ rank, int* __restrict__ counts,
    const int* __restrict__ idx, int n_entries) {
  __shared__ int wtot[4];
  const int e = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  int base = 0;
  for (int i0 = 0; i0 < n_entries; i0 += 256) {
    const int i = i0 + threadIdx.x;
    const bool mine = i < n_entries && idx[i] == e;
    const unsigned long long mask = __ballot(mine);
    const int before = __popcll(mask & ((1ull << lane) - 1ull));
    if (lane == 0) wtot[wave] = __popcll(mask);
    __syncthreads();
    int off = base;
    for (int w = 0; w < wave; w++) off += wtot[w];
    if (mine) rank[i] = off + before;
    base += wtot[0] + wtot[1] + wtot[2] + wtot[3];
    __syncthreads();
  }
  if (threadIdx.x == 0) counts[e] = base;
}

// xg[base[e] + rank[t, j]] = h[t] for every choice e = idx[t, j] < E.
template <typename T>
__global__ void moe_gather_kernel(T* __restrict__ xg, const T* __restrict__ h,
                                  const int* __restrict__ idx,
                                  const int* __restrict__ rank,
                                  const int* __restrict__ base, int E, int W,
                                  int top, int rows, int vec) {
  const int t = blockIdx.x, j = blockIdx.y;
  const int e = idx[(int64_t)t * top + j];
  if (e < 0 || e >= E) return;
  const int r = base[e] + rank[(int64_t)t * top + j];
  if (r < 0 || r >= rows) return;
  const T* src = h + (int64_t)t * W;
  T* dst = xg + (int64_t)r * W;
  if (vec) {
    constexpr int N = 16 / sizeof(T);
    for (int i = threadIdx.x; i < W / N; i += blockDim.x)
      reinterpret_cast<uint4*>(dst)[i] = reinterpret_cast<const uint4*>(src)[i];
  } else {
    for (int i = threadIdx.x; i < W; i += blockDim.x) dst[i] = src[i];
  }
}

// out[t] = sum_j wgt[t, j] * (y[base[e] + rank[t, j]] or, for an identity
// expert e >= E, h[t]) + shared[t], summed in fp32 in the order of j.
template <typename T>
__global__ void moe_combine_kernel(
    T* __restrict__ out, const T* __restrict__ y, const T* __restrict__ h,
    const int* __restrict__ idx, const float* __restrict__ wgt,
    const int* __restrict__ rank, const int* __restrict__ base,
    const T* __restrict__ shared, const float* __restrict__ shared_gate,
    int gate_stride, int E, int W, int top, int rows) {
  constexpr int MAXTOP = 64;  // checked on the host
  __shared__ const T* src[MAXTOP];
  __shared__ float wj[MAXTOP];
  const int t = blockIdx.x;
  const T* hr = h + (int64_t)t * W;
  // the rows this token sums, looked up once
  for (int j = threadIdx.x; j < top; j += blockDim.x) {
    const int e = idx[(int64_t)t * top + j];
    wj[j] = wgt[(int64_t)t * top + j];
    if (e >= E || e < 0) {
      src[j] = hr;
    } else {
      const int r = min(max(base[e] + rank[(int64_t)t * top + j], 0), rows - 1);
      src[j] = y + (int64_t)r * W;
    }
  }
  __syncthreads();
  // the shared row weighs in with sigmoid(gate value of the token)
  const float sg =
      shared_gate ? sigmoid_f(shared_gate[(int64_t)t * gate_stride]) : 1.f;
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    float acc = 0.f;
    for (int j = 0; j < top; j++) acc += wj[j] * to_f(src[j][c]);
    if (shared) acc += sg * to_f(shared[(int64_t)t * W + c]);
    out[(int64_t)t * W + c] = from_f<T>(acc);
  }
}

inline int pow2_block(int n, int cap) {
  int b = 64;
  while (b < n && b < cap) b <<= 1;
  return b;
}

}  // namespace

void headnorm_rope_append(torch::Tensor proj, int64_t H, int64_t G, int64_t dk,
                          int64_t dv, int64_t off_k, int64_t off_v,
                          torch::Tensor qw, torch::Tensor kw,
                          c10::optional<torch::Tensor> freqs, bool interleaved,
                          double eps, torch::Tensor positions,
                          torch::Tensor kcache, torch::Tensor vcache,
                          torch::Tensor slot_mapping) {
  const int T_ = proj.size(0);
  SEQ_CHECK(is_act(proj) && proj.dim() == 2 && proj.stride(1) == 1 && H >= 1 &&
                G >= 1 && dk >= 1 && dv >= 1 && H * dk <= off_k &&
                off_k + G * dk <= off_v && off_v + G * dv <= proj.size(1),
            "q | k | v projections");
  SEQ_CHECK(kcache.is_contiguous() && vcache.is_contiguous() &&
                kcache.dim() == 4 && vcache.dim() == 4 &&
                kcache.size(1) == G && kcache.size(3) == dk &&
                vcache.size(0) == kcache.size(0) && vcache.size(1) == G &&
                vcache.size(2) == kcache.size(2) && vcache.size(3) == dv &&
                kcache.scalar_type() == proj.scalar_type() &&
                vcache.scalar_type() == proj.scalar_type(), "kv cache");
  for (const torch::Tensor* w : {&qw, &kw})
    SEQ_CHECK(w->scalar_type() == torch::kFloat && w->is_contiguous() &&
                  w->numel() == dk, "head norm weights");
  int dims = 0;
  if (freqs) {
    SEQ_CHECK(freqs->scalar_type() == torch::kFloat && freqs->is_contiguous() &&
                  freqs->dim() == 2 && freqs->size(0) == 2 &&
                  2 * freqs->size(1) <= dk, "rotary frequencies [2, dims/2]");
    dims = 2 * (int)freqs->size(1);
  }
  check_ints(positions, T_, "positions");
  SEQ_CHECK(slot_mapping.scalar_type() == torch::kLong &&
                slot_mapping.is_contiguous() && slot_mapping.numel() >= T_,
            "slot mapping");
  if (T_ == 0) return;
  const int nvec = (int)(H + 2 * G);
  DISPATCH_ACT(proj, hipLaunchKernelGGL(
      headnorm_rope_append_kernel<T>, dim3(T_, (nvec + 3) / 4), dim3(256), 0,
      cur_stream(), ptr<T>(proj), (int)proj.stride(0), (int)H, (int)G, (int)dk,
      (int)dv, (int)off_k, (int)off_v, cptr<float>(qw), cptr<float>(kw),
      freqs ? cptr<float>(*freqs) : (const float*)nullptr, dims,
      interleaved ? 1 : 0, (float)eps, cptr<int>(positions), ptr<T>(kcache),
      ptr<T>(vcache), cptr<int64_t>(slot_mapping), (int)kcache.size(2)););
}

void mingru_scan(torch::Tensor out, torch::Tensor proj, torch::Tensor state,
                 torch::Tensor seq_start, torch::Tensor seq_len,
                 torch::Tensor seq_slot, torch::Tensor seq_pos0,
                 int64_t max_len) {
  // max_len: an upper bound of the longest sequence portion of this step
  const int T_ = proj.size(0), C = out.size(1);
  const int B = seq_start.size(0);
  SEQ_CHECK(is_act(proj) && proj.dim() == 2 && proj.stride(1) == 1 &&
                proj.size(1) >= 3 * C, "gate | candidate | out-gate rows");
  SEQ_CHECK(out.is_contiguous() && out.dim() == 2 && out.size(0) == T_ &&
                out.scalar_type() == proj.scalar_type(), "recurrence out");
  SEQ_CHECK(state.scalar_type() == torch::kFloat && state.is_contiguous() &&
                state.dim() == 2 && state.size(1) == C, "recurrent state");
  check_ints(seq_len, B, "seq_len");
  check_ints(seq_slot, B, "seq_slot");
  check_ints(seq_pos0, B, "seq_pos0");
  SEQ_CHECK(max_len >= 1, "longest portion");
  if (T_ == 0 || B == 0) return;
  const int threads = 64, chunk = 64;
  const int nch = (int)((std::min<int64_t>(max_len, T_) + chunk - 1) / chunk);
  const int cb = (C + threads - 1) / threads;
  const int stride = (int)proj.stride(0);
  torch::Tensor sums;
  float* sumA = nullptr;
  float* sumB = nullptr;
  if (nch > 1) {
    sums = torch::empty({2, B, nch, C},
                        proj.options().dtype(torch::kFloat));
    sumA = ptr<float>(sums);
    sumB = sumA + (int64_t)B * nch * C;
  }
  DISPATCH_ACT(proj, {
    if (nch > 1)
      hipLaunchKernelGGL(mingru_chunk_summary_kernel<T>, dim3(cb, nch, B),
                         dim3(threads), 0, cur_stream(), sumA, sumB,
                         cptr<T>(proj), stride, cptr<int>(seq_start),
                         cptr<int>(seq_len), C, chunk, nch);
    hipLaunchKernelGGL(mingru_scan_kernel<T>, dim3(cb, nch, B), dim3(threads),
                       0, cur_stream(), ptr<T>(out), cptr<T>(proj), stride,
                       ptr<float>(state), sumA, sumB, cptr<int>(seq_start),
                       cptr<int>(seq_len), cptr<int>(seq_slot),
                       cptr<int>(seq_pos0), C, chunk, nch);
    if (nch > 1)
      hipLaunchKernelGGL(mingru_state_kernel<T>, dim3(cb, B), dim3(threads), 0,
                         cur_stream(), ptr<float>(state), cptr<T>(proj), stride,
                         sumA, sumB, cptr<int>(seq_start), cptr<int>(seq_len),
                         cptr<int>(seq_slot), cptr<int>(seq_pos0), C, chunk,
                         nch);
  });
}

void relu_squared(torch::Tensor out, torch::Tensor x) {
  SEQ_CHECK(is_act(x) && x.is_contiguous() && out.is_contiguous() &&
                out.scalar_type() == x.scalar_type() &&
                out.numel() == x.numel(), "relu^2 in/out");
  const int64_t n = x.numel();
  if (n == 0) return;
  DISPATCH_ACT(x, {
    constexpr int N = 16 / sizeof(T);
    if (n % N == 0 && reinterpret_cast<uintptr_t>(x.data_ptr()) % 16 == 0 &&
        reinterpret_cast<uintptr_t>(out.data_ptr()) % 16 == 0) {
      const int64_t nvec = n / N;
      const int blocks = (int)std::min<int64_t>((nvec + 255) / 256, 8192);
      hipLaunchKernelGGL(relu_squared_vec_kernel<T>, dim3(blocks), dim3(256), 0,
                         cur_stream(), ptr<T>(out), cptr<T>(x), nvec);
    } else {
      hipLaunchKernelGGL(relu_squared_kernel<T>, dim3((n + 255) / 256),
                         dim3(256), 0, cur_stream(), ptr<T>(out), cptr<T>(x), n);
    }
  });
}

// `logits` fp32 [T, n], or - with `router` fp32 [n, W] given - the router's
// input rows h [T, W] in the activation type.
void moe_route(torch::Tensor idx, torch::Tensor wgt, torch::Tensor logits,
               c10::optional<torch::Tensor> router, torch::Tensor correction,
               int64_t groups, int64_t keep, double scale) {
  const int T_ = logits.size(0), top = idx.size(1);
  const int n = router ? router->size(0) : logits.size(1);
  if (router) {
    SEQ_CHECK(is_act(logits) && logits.dim() == 2 && logits.is_contiguous() &&
                  router->scalar_type() == torch::kFloat &&
                  router->is_contiguous() && router->dim() == 2 &&
                  router->size(1) == logits.size(1), "router input and rows");
  } else {
    SEQ_CHECK(logits.dim() == 2 && logits.scalar_type() == torch::kFloat &&
                  logits.is_contiguous(), "router logits fp32 [T, n]");
  }
  SEQ_CHECK(correction.scalar_type() == torch::kFloat &&
                correction.is_contiguous() && correction.numel() == n,
            "router correction");
  SEQ_CHECK(idx.dim() == 2 && idx.scalar_type() == torch::kInt &&
                idx.is_contiguous() && idx.size(0) == T_ &&
                wgt.scalar_type() == torch::kFloat && wgt.is_contiguous() &&
                wgt.dim() == 2 && wgt.size(0) == T_ && wgt.size(1) == top,
            "router outputs");
  SEQ_CHECK(groups >= 1 && n % groups == 0 && keep >= 1 && keep <= groups &&
                top >= 1 && top <= keep * (n / groups), "router groups");
  const size_t lds = 4 * (2 * (size_t)n + groups) * sizeof(float);
  SEQ_CHECK(lds <= 64 * 1024, "too many router outputs");
  if (T_ == 0) return;
  if (router) {
    DISPATCH_ACT(logits, hipLaunchKernelGGL(
        (moe_route_kernel<T, true>), dim3(T_), dim3(256), lds, cur_stream(),
        ptr<int>(idx), ptr<float>(wgt), (const float*)nullptr,
        cptr<T>(logits), cptr<float>(*router), (int)logits.size(1),
        cptr<float>(correction), T_, n, (int)groups, (int)keep, top,
        (float)scale););
  } else {
    hipLaunchKernelGGL((moe_route_kernel<float, false>), dim3((T_ + 3) / 4),
                       dim3(256), lds, cur_stream(), ptr<int>(idx),
                       ptr<float>(wgt),
                       cptr<float>(logits), (const float*)nullptr,
                       (const float*)nullptr, 0, cptr<float>(correction), T_,
                       n, (int)groups, (int)keep, top, (float)scale);
  }
}

void moe_dispatch(torch::Tensor rank, torch::Tensor counts, torch::Tensor idx) {
  SEQ_CHECK(idx.scalar_type() == torch::kInt && idx.is_contiguous() &&
                rank.scalar_type() == torch::kInt && rank.is_contiguous() &&
                rank.numel() == idx.numel() &&
                counts.scalar_type() == torch::kInt && counts.is_contiguous() &&
                counts.numel() >= 1, "dispatch tensors");
  hipLaunchKernelGGL(moe_dispatch_kernel, dim3((int)counts.numel()), dim3(256),
                     0, cur_stream(), ptr<int>(rank), ptr<int>(counts),
                     cptr<int>(idx), (int)idx.numel());
}

void moe_gather(torch::Tensor xg, torch::Tensor h, torch::Tensor idx,
                torch::Tensor rank, torch::Tensor base, int64_t E) {
  const int T_ = h.size(0), W = h.size(1), top = idx.size(1);
  SEQ_CHECK(is_act(h) && h.dim() == 2 && h.is_contiguous() &&
                xg.is_contiguous() && xg.dim() == 2 && xg.size(1) == W &&
                xg.scalar_type() == h.scalar_type(), "gather rows");
  SEQ_CHECK(idx.scalar_type() == torch::kInt && idx.is_contiguous() &&
                idx.dim() == 2 && idx.size(0) == T_ &&
                rank.scalar_type() == torch::kInt && rank.is_contiguous() &&
                rank.numel() == idx.numel(), "gather choices");
  check_ints(base, E, "base");
  if (T_ == 0 || xg.size(0) == 0) return;
  DISPATCH_ACT(h, {
    const int vec = (W * sizeof(T)) % 16 == 0 &&
                    reinterpret_cast<uintptr_t>(h.data_ptr()) % 16 == 0 &&
                    reinterpret_cast<uintptr_t>(xg.data_ptr()) % 16 == 0;
    hipLaunchKernelGGL(moe_gather_kernel<T>, dim3(T_, top),
                       dim3(pow2_block(W / 8, 256)), 0, cur_stream(),
                       ptr<T>(xg), cptr<T>(h), cptr<int>(idx), cptr<int>(rank),
                       cptr<int>(base), (int)E, W, top, (int)xg.size(0), vec);
  });
}

void moe_combine(torch::Tensor out, torch::Tensor y, torch::Tensor h,
                 torch::Tensor idx, torch::Tensor wgt, torch::Tensor rank,
                 torch::Tensor base, int64_t E,
                 c10::optional<torch::Tensor> shared,
                 c10::optional<torch::Tensor> shared_gate) {
  const int T_ = h.size(0), W = h.size(1), top = idx.size(1);
  if (shared_gate)
    SEQ_CHECK(shared.has_value() && shared_gate->dim() == 1 &&
                  shared_gate->size(0) == T_ &&
                  shared_gate->scalar_type() == torch::kFloat,
              "shared gate fp32 [T]");
  SEQ_CHECK(is_act(h) && h.dim() == 2 && h.is_contiguous() &&
                out.is_contiguous() && out.dim() == 2 && out.size(0) == T_ &&
                out.size(1) == W && out.scalar_type() == h.scalar_type() &&
                y.is_contiguous() && y.dim() == 2 && y.size(1) == W &&
                y.scalar_type() == h.scalar_type(), "combine rows");
  SEQ_CHECK(idx.scalar_type() == torch::kInt && idx.is_contiguous() &&
                idx.dim() == 2 && idx.size(0) == T_ &&
                rank.scalar_type() == torch::kInt && rank.is_contiguous() &&
                rank.numel() == idx.numel() &&
                wgt.scalar_type() == torch::kFloat && wgt.is_contiguous() &&
                wgt.numel() == idx.numel(), "combine choices");
  check_ints(base, E, "base");
  SEQ_CHECK(top >= 1 && top <= 64, "experts per token");
  if (shared)
    SEQ_CHECK(shared->is_contiguous() && shared->dim() == 2 &&
                  shared->size(0) == T_ && shared->size(1) == W &&
                  shared->scalar_type() == h.scalar_type(), "shared rows");
  if (T_ == 0) return;
  DISPATCH_ACT(h, hipLaunchKernelGGL(
      moe_combine_kernel<T>, dim3(T_), dim3(pow2_block(W, 256)), 0,
      cur_stream(), ptr<T>(out), cptr<T>(y), cptr<T>(h), cptr<int>(idx),
      cptr<float>(wgt), cptr<int>(rank), cptr<int>(base),
      shared ? cptr<T>(*shared) : (const T*)nullptr,
      shared_gate ? cptr<float>(*shared_gate) : (const float*)nullptr,
      shared_gate ? (int)shared_gate->stride(0) : 0, (int)E, W, top,
      (int)std::max<int64_t>(y.size(0), 1)););
}
