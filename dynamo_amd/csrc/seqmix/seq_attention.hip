// Softmax attention over the paged cache with a logarithmic distance bias
// and a position-dependent query temperature, for head sizes the MFMA
// flash kernels do not cover (any dk, dv up to 64 * EVMAX) and for fp32
// caches. One workgroup per (token row, group of query heads sharing a kv
// head); see biased_attention_kernel. Scores, softmax and the accumulator
// are fp32.
//
//   score(i, j) = temp(i) * scale * (q_i . k_j) - r1_h * log1p(r2_h * (i - j))
//   temp(i)     = 1 + coef * ln(floor((i + 1) / every) + 1)
//
// The same kernel serves prompt portions and decoded tokens: a row only
// needs its position and its sequence's page table.
//
// The kernel is general in three more ways, which paged_attention_rows
// exposes: a sliding window (row i sees keys j with 0 <= i - j < window),
// several key maps per kv head (the cached key row of a kv head holds
// `kmaps` keys of size dk back to back; query head h has one query per map,
// laid out [h][map][dk], and every map is a softmax attention of its own
// over the same values - the output is [T, H, kmaps, dv]), and a value row
// stride of its own, so values may alias a prefix of the key rows (latent
// attention, where the cached latent is both key part and value). The
// output may be fp32 whatever the cache type. With a window, the first
// `keep_first` keys of a sequence may stay visible whatever their distance;
// a per-head constant may be added to the scaled scores; and the weights
// may be plain sigmoids of the scores (not normalised over the keys)
// instead of a softmax. The softmax form further takes a soft cap
// c tanh(score / c) on the scaled scores, a bias looked up by key distance
// in a table [H, dist_max + 1] (added after the cap; distances beyond the
// table take its last entry), and a per-head sink: exp(sink_h) is added to the
// softmax denominator, with no key and no value.
#include "seq_common.h"

namespace {

constexpr int EVMAX = 16;  // value channels per lane: dv <= 1024

// Append this step's keys (raw) and values (each head divided by its root
// mean square when vnorm is set) to the paged cache. One wave per
// (token, kv head). Cache layout [pages, G, page_size, d].
template <typename T>
__global__ void kv_append_norm_kernel(
    T* __restrict__ kcache, T* __restrict__ vcache, const T* __restrict__ proj,
    int proj_stride, int off_k, int off_v,
    const int64_t* __restrict__ slot_mapping, int G, int dk, int dv, int ps,
    int vnorm, float eps) {
  const int t = blockIdx.x, g = blockIdx.y, lane = threadIdx.x;
  const int64_t slot = slot_mapping[t];
  if (slot < 0) return;
  const int64_t page = slot / ps, inpage = slot % ps;
  const T* krow = proj + (int64_t)t * proj_stride + off_k + g * dk;
  const T* vrow = proj + (int64_t)t * proj_stride + off_v + g * dv;
  T* kd = kcache + ((page * G + g) * ps + inpage) * dk;
  T* vd = vcache + ((page * G + g) * ps + inpage) * dv;
  for (int i = lane; i < dk; i += 64) kd[i] = krow[i];
  float inv = 1.f;
  if (vnorm) {
    float ss = 0.f;
    for (int i = lane; i < dv; i += 64) {
      const float x = to_f(vrow[i]);
      ss += x * x;
    }
    ss = wave_sum(ss);
    inv = 1.f / sqrtf(ss / (float)dv + eps);
  }
  for (int i = lane; i < dv; i += 64) vd[i] = from_f<T>(to_f(vrow[i]) * inv);
}

// 16-byte vector of activations
template <typename T> struct Vec16;
template <> struct Vec16<float> {
  static constexpr int N = 4;
  float4 v;
  DEVINL float get(int i) const { return (&v.x)[i]; }
};
template <> struct Vec16<bf16_t> {
  static constexpr int N = 8;
  uint4 v;
  DEVINL float get(int i) const {
    const uint32_t w = (&v.x)[i >> 1];
    union { float f; uint32_t u; } c;
    c.u = (i & 1) ? (w & 0xffff0000u) : (w << 16);
    return c.f;
  }
};

// One workgroup per (token row, group of GS query heads that share a kv
// head). Its waves (4 for large prompt batches, 16 when few rows are in
// flight, so a decoded token with a long context still fills a CU) take
// 64-key chunks in turn and are merged through LDS at the end. Within a
// chunk, 4 adjacent lanes share a key: each reads every 4th 16-byte piece
// of the key row (a quad covers 64 contiguous bytes) and the quad adds its
// partial dots, 16 keys a pass, 4 passes a chunk; no transposed staging is
// needed. For the weighted sum a lane owns pairs of adjacent value channels
// and reads value rows as they lie in the page, eight rows in flight.
// FAST needs key rows that are whole 16-byte pieces, an even value size
// and a page size that is a multiple of 16: then every load address is
// clamped into range instead of tested, so the loads of a pass issue back
// to back. Otherwise a plain scalar path runs. EVT is the number of value
// channels a lane owns.
template <typename T, typename TO, int GS, bool FAST, int EVT>
__global__ __launch_bounds__(1024) void biased_attention_kernel(
    TO* __restrict__ out,  // [T, H, kmaps, dv]
    const T* __restrict__ proj, int proj_stride, int off_q,
    const T* __restrict__ kcache, const T* __restrict__ vcache,
    const int* __restrict__ page_table, int table_stride,
    const int* __restrict__ tok_seq, const int* __restrict__ positions,
    const int* __restrict__ seq_len, const float* __restrict__ r1,
    const float* __restrict__ r2, int H, int G, int dk, int dv, int ps,
    float scale, float temp_coef, int temp_every, int has_bias, int kmaps,
    int vrow, int window, int keep_first, const float* __restrict__ head_bias,
    int sigmoid, float softcap, const float* __restrict__ dist_bias,
    int dist_max, const float* __restrict__ sink) {
  extern __shared__ __attribute__((aligned(16))) float lds[];
  // q [GS][dk]; merge [waves][GS][2 + dv]
  constexpr int VN = Vec16<T>::N;
  const int t = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int nwv = blockDim.x >> 6;
  const int s = tok_seq[t];
  if (seq_len[s] == 0) return;  // padding row
  // blockIdx.y = ((kv head * kmaps) + map) * (blocks per kv head) + block
  const int gsz = H / G, bpg = gsz / GS;
  const int g = blockIdx.y / (kmaps * bpg);
  const int map = (blockIdx.y / bpg) % kmaps;
  const int h0 = g * gsz + (blockIdx.y % bpg) * GS;  // first query head
  const int krow = kmaps * dk, koff = map * dk;
  const int pos = positions[t];
  float temp = 1.f;
  if (temp_coef != 0.f)
    temp += temp_coef * logf((float)((pos + 1) / temp_every) + 1.f);
  const float qmul = temp * scale;
  float* qs = lds;
  float* mg = lds + GS * dk;
  for (int i = threadIdx.x; i < GS * dk; i += blockDim.x) {
    const int a = i / dk, e = i - a * dk;
    qs[i] = to_f(proj[(int64_t)t * proj_stride + off_q +
                      ((h0 + a) * kmaps + map) * dk + e]) * qmul;
  }
  __syncthreads();
  const int* table = page_table + (int64_t)s * table_stride;
  float b1[GS], b2[GS], hb[GS];
#pragma unroll
  for (int a = 0; a < GS; a++) {
    b1[a] = has_bias ? r1[h0 + a] : 0.f;
    b2[a] = has_bias ? r2[h0 + a] : 0.f;
    hb[a] = head_bias ? head_bias[h0 + a] : 0.f;
  }
  const int quad = lane >> 2, qq = lane & 3;
  const int nvec = dk / VN;  // 16-byte pieces of a key row (FAST)

  // l is kept per lane (the sum over the keys this lane scored, each key
  // counted by the 4 lanes of its quad) and only reduced at the end
  float m[GS], l[GS], acc[GS][EVT];
#pragma unroll
  for (int a = 0; a < GS; a++) {
    m[a] = -INFINITY;
    l[a] = 0.f;
#pragma unroll
    for (int e = 0; e < EVT; e++) acc[a][e] = 0.f;
  }
  const int ctx = pos + 1;
  const int jmin = window > 0 ? max(0, ctx - window) : 0;  // first visible key
  const int nchunks = (ctx + 63) >> 6;
  // chunks that hold kept first keys and lie wholly before the window's
  // first chunk are walked first, then the window's chunks
  const int c_lo = jmin >> 6;
  const int nsink = (keep_first > 0 && jmin > 0)
                        ? min((min(keep_first, jmin) + 63) >> 6, c_lo) : 0;
  for (int vc = wave; vc < nsink + nchunks - c_lo; vc += nwv) {
    const int c = vc < nsink ? vc : vc - nsink + c_lo;
    const int j0 = c << 6;
    // ---- scores: pass p covers keys j0 + 16 p + quad ----
    float sc[4][GS];
#pragma unroll
    for (int p = 0; p < 4; p++) {
      const int j = j0 + 16 * p + quad;
      const int jc = min(j, ctx - 1);  // loads stay in range, masked below
      float d[GS];
#pragma unroll
      for (int a = 0; a < GS; a++) d[a] = 0.f;
      const int64_t page = table[jc / ps];
      const T* k = kcache + ((page * G + g) * ps + (jc % ps)) * krow + koff;
      if (FAST) {
        for (int v0 = qq; v0 < nvec; v0 += 16) {
          Vec16<T> kv[4];
#pragma unroll
          for (int u = 0; u < 4; u++)
            kv[u].v = *reinterpret_cast<const decltype(kv[u].v)*>(
                k + min(v0 + 4 * u, nvec - 1) * VN);
#pragma unroll
          for (int u = 0; u < 4; u++) {
            const int v = min(v0 + 4 * u, nvec - 1);
            const float on = v0 + 4 * u < nvec ? 1.f : 0.f;
#pragma unroll
            for (int a = 0; a < GS; a++) {
              const float4* q4 =
                  reinterpret_cast<const float4*>(qs + a * dk + v * VN);
              float part = 0.f;
#pragma unroll
              for (int i4 = 0; i4 < VN / 4; i4++) {
                const float4 q = q4[i4];
                part += q.x * kv[u].get(4 * i4) + q.y * kv[u].get(4 * i4 + 1) +
                        q.z * kv[u].get(4 * i4 + 2) + q.w * kv[u].get(4 * i4 + 3);
              }
              d[a] += on * part;
            }
          }
        }
      } else {
        for (int i = qq; i < dk; i += 4) {
          const float kf = to_f(k[i]);
#pragma unroll
          for (int a = 0; a < GS; a++) d[a] += qs[a * dk + i] * kf;
        }
      }
#pragma unroll
      for (int a = 0; a < GS; a++) {
        float x = d[a];
        x += __shfl_xor(x, 1, 64);
        x += __shfl_xor(x, 2, 64);
        if (softcap > 0.f) x = softcap * tanhf(x / softcap);
        if (has_bias) x -= b1[a] * log1pf(b2[a] * (float)(pos - jc));
        if (dist_bias)
          x += dist_bias[(h0 + a) * (dist_max + 1) + min(pos - jc, dist_max)];
        x += hb[a];
        sc[p][a] = (j < ctx && (j >= jmin || j < keep_first)) ? x : -INFINITY;
      }
    }
    // ---- online softmax (every lane of a quad holds the same score) ----
    float pr[4][GS];
    if (sigmoid) {
      // unnormalised weights: a masked key (score -inf) weighs exactly 0
#pragma unroll
      for (int a = 0; a < GS; a++)
#pragma unroll
        for (int p = 0; p < 4; p++) pr[p][a] = sigmoid_f(sc[p][a]);
    } else
#pragma unroll
    for (int a = 0; a < GS; a++) {
      float mx = fmaxf(fmaxf(sc[0][a], sc[1][a]), fmaxf(sc[2][a], sc[3][a]));
      mx = fmaxf(m[a], wave_max(mx));
      const float corr = expf(m[a] - mx);
      float sum = 0.f;
#pragma unroll
      for (int p = 0; p < 4; p++) {
        pr[p][a] = expf(sc[p][a] - mx);  // 0 for masked keys
        sum += pr[p][a];
      }
      l[a] = l[a] * corr + sum;
      m[a] = mx;
#pragma unroll
      for (int e = 0; e < EVT; e++) acc[a][e] *= corr;
    }
    // ---- weighted sum of values: lane owns channels
    //      (e / 2) * 128 + 2 * lane + (e & 1) ----
#pragma unroll
    for (int p = 0; p < 4; p++) {
      const int jp = j0 + 16 * p;
      const int nk = min(16, ctx - jp);
      if (nk <= 0) break;
      if (FAST) {
        // the 16 keys of a pass lie in one page; rows past the context
        // are read from the last valid row and weigh 0
        const T* vrun =
            vcache +
            (((int64_t)table[jp / ps] * G + g) * ps + (jp % ps)) * vrow;
#pragma unroll
        for (int k0 = 0; k0 < 16; k0 += 8) {
          if (k0 >= nk) break;
          float vf[8][EVT];
#pragma unroll
          for (int u = 0; u < 8; u++) {
            const T* v = vrun + (int64_t)min(k0 + u, nk - 1) * vrow;
#pragma unroll
            for (int e = 0; e < EVT; e += 2) {
              const int ch = min((e / 2) * 128 + 2 * lane, dv - 2);
              if (sizeof(T) == 2) {
                const uint32_t w = *reinterpret_cast<const uint32_t*>(v + ch);
                union { float f; uint32_t u; } c0, c1;
                c0.u = w << 16;
                c1.u = w & 0xffff0000u;
                vf[u][e] = c0.f;
                vf[u][e + 1] = c1.f;
              } else {
                const float2 w = *reinterpret_cast<const float2*>(v + ch);
                vf[u][e] = w.x;
                vf[u][e + 1] = w.y;
              }
            }
          }
#pragma unroll
          for (int u = 0; u < 8; u++) {
#pragma unroll
            for (int a = 0; a < GS; a++) {
              const float w = __shfl(pr[p][a], (k0 + u) << 2, 64);
#pragma unroll
              for (int e = 0; e < EVT; e++) acc[a][e] += w * vf[u][e];
            }
          }
        }
      } else {
        for (int kk = 0; kk < nk; kk++) {
          const int j = jp + kk;
          const T* v = vcache +
              (((int64_t)table[j / ps] * G + g) * ps + (j % ps)) * vrow;
          float w[GS];
#pragma unroll
          for (int a = 0; a < GS; a++) w[a] = __shfl(pr[p][a], kk << 2, 64);
#pragma unroll
          for (int e = 0; e < EVT; e++) {
            const int ch = (e / 2) * 128 + 2 * lane + (e & 1);
            if (ch < dv) {
              const float vf = to_f(v[ch]);
#pragma unroll
              for (int a = 0; a < GS; a++) acc[a][e] += w[a] * vf;
            }
          }
        }
      }
    }
  }
#pragma unroll
  for (int a = 0; a < GS; a++) l[a] = 0.25f * wave_sum(l[a]);
  // ---- merge the waves ----
  const int MS = 2 + dv;  // floats per (wave, head) record
#pragma unroll
  for (int a = 0; a < GS; a++) {
    float* rec = mg + (wave * GS + a) * MS;
    if (lane == 0) {
      rec[0] = m[a];
      rec[1] = l[a];
    }
#pragma unroll
    for (int e = 0; e < EVT; e++) {
      const int ch = (e / 2) * 128 + 2 * lane + (e & 1);
      if (ch < dv) rec[2 + ch] = acc[a][e];
    }
  }
  __syncthreads();
  for (int a = wave; a < GS; a += nwv) {  // wave a finishes head a
    if (sigmoid) {  // plain sum of the waves' partial results
      for (int ch = lane; ch < dv; ch += 64) {
        float o = 0.f;
        for (int w = 0; w < nwv; w++) o += mg[(w * GS + a) * MS + 2 + ch];
        out[(((int64_t)t * H + h0 + a) * kmaps + map) * dv + ch] =
            from_f<TO>(o);
      }
      continue;
    }
    float mx = sink ? sink[h0 + a] : -INFINITY;
    for (int w = 0; w < nwv; w++) mx = fmaxf(mx, mg[(w * GS + a) * MS]);
    float lt = sink ? expf(sink[h0 + a] - mx) : 0.f;
    for (int w = 0; w < nwv; w++) {
      const float mw = mg[(w * GS + a) * MS];
      if (mw != -INFINITY) lt += expf(mw - mx) * mg[(w * GS + a) * MS + 1];
    }
    const float inv = 1.f / lt;
    for (int ch = lane; ch < dv; ch += 64) {
      float o = 0.f;
      for (int w = 0; w < nwv; w++) {
        const float mw = mg[(w * GS + a) * MS];
        if (mw != -INFINITY) o += expf(mw - mx) * mg[(w * GS + a) * MS + 2 + ch];
      }
      out[(((int64_t)t * H + h0 + a) * kmaps + map) * dv + ch] =
          from_f<TO>(o * inv);
    }
  }
}

template <typename T, typename TO>
void launch_attention(torch::Tensor& out, torch::Tensor& proj, int64_t off_q,
                      torch::Tensor& kcache, const void* vptr, int dv, int vrow,
                      torch::Tensor& page_table, torch::Tensor& tok_seq,
                      torch::Tensor& positions, torch::Tensor& seq_len,
                      c10::optional<torch::Tensor>& r1,
                      c10::optional<torch::Tensor>& r2, double scale,
                      double temp_coef, int64_t temp_every, int kmaps,
                      int window, int keep_first,
                      c10::optional<torch::Tensor>& head_bias, bool sigmoid,
                      double softcap, c10::optional<torch::Tensor>& dist_bias,
                      c10::optional<torch::Tensor>& sink) {
  const int T_ = out.size(0), H = out.size(1);
  const int G = kcache.size(1), ps = kcache.size(2);
  const int dk = kcache.size(3) / kmaps;
  const int gsz = H / G;
  // heads of a group share each key/value load; with few rows in flight a
  // smaller group gives the chip more workgroups instead
  int GS = gsz % 4 == 0 ? 4 : (gsz % 2 == 0 ? 2 : 1);
  if (GS == 4 && T_ * (H * kmaps / 4) < 256) GS = 2;
  // few rows in flight (decoding): 16 waves split the keys of each row; a
  // window bounds the keys of a row, and the waves with them
  int NW = T_ * (H * kmaps / GS) <= 2048 ? 16 : 4;
  if (window > 0)
    while (NW > 1 && (NW - 1) * 64 >= window + keep_first + 126) NW >>= 1;
  auto lds_bytes = [&](int gs, int nw) {
    return (size_t)(gs * dk + nw * gs * (2 + dv)) * sizeof(float);
  };
  while (NW > 1 && lds_bytes(GS, NW) > 64 * 1024) NW >>= 1;
  while (GS > 1 && lds_bytes(GS, NW) > 64 * 1024) GS >>= 1;
  const size_t lds = lds_bytes(GS, NW);
  TORCH_CHECK(lds <= 64 * 1024,
              "seqmix: attention head sizes exceed the LDS budget");
  const bool vec = (dk * sizeof(T)) % 16 == 0 && dv % 2 == 0 && ps % 16 == 0 &&
                   vrow % 2 == 0 &&
                   reinterpret_cast<uintptr_t>(kcache.data_ptr()) % 16 == 0 &&
                   reinterpret_cast<uintptr_t>(vptr) % 8 == 0;
  const bool small = dv <= 128, mid = dv <= 512;
#define LAUNCH_ATT(GS_, VEC_, EVT_)                                         \
  hipLaunchKernelGGL((biased_attention_kernel<T, TO, GS_, VEC_, EVT_>),     \
      dim3(T_, H * kmaps / GS_), dim3(NW * 64), lds, cur_stream(),          \
      ptr<TO>(out), cptr<T>(proj), (int)proj.stride(0), (int)off_q,         \
      cptr<T>(kcache), reinterpret_cast<const T*>(vptr),                    \
      cptr<int>(page_table), (int)page_table.stride(0),                     \
      cptr<int>(tok_seq), cptr<int>(positions), cptr<int>(seq_len),         \
      r1 ? cptr<float>(*r1) : nullptr, r2 ? cptr<float>(*r2) : nullptr, H,  \
      G, dk, dv, ps, (float)scale, (float)temp_coef, (int)temp_every,       \
      r1 ? 1 : 0, kmaps, vrow, window, keep_first,                          \
      head_bias ? cptr<float>(*head_bias) : nullptr, sigmoid ? 1 : 0,       \
      (float)softcap, dist_bias ? cptr<float>(*dist_bias) : nullptr,        \
      dist_bias ? (int)dist_bias->size(1) - 1 : 0,                          \
      sink ? cptr<float>(*sink) : nullptr)
#define LAUNCH_GS(GS_)                                                      \
  do {                                                                      \
    if (vec && small) LAUNCH_ATT(GS_, true, 2);                             \
    else if (vec && mid) LAUNCH_ATT(GS_, true, 8);                          \
    else if (vec) LAUNCH_ATT(GS_, true, EVMAX);                             \
    else if (small) LAUNCH_ATT(GS_, false, 2);                              \
    else if (mid) LAUNCH_ATT(GS_, false, 8);                                \
    else LAUNCH_ATT(GS_, false, EVMAX);                                     \
  } while (0)
  if (GS == 4) LAUNCH_GS(4);
  else if (GS == 2) LAUNCH_GS(2);
  else LAUNCH_GS(1);
#undef LAUNCH_GS
#undef LAUNCH_ATT
}

}  // namespace

void kv_append_norm(torch::Tensor kcache, torch::Tensor vcache,
                    torch::Tensor proj, int64_t off_k, int64_t off_v,
                    torch::Tensor slot_mapping, bool vnorm, double eps) {
  // caches [pages, G, ps, d]
  const int T_ = proj.size(0);
  const int G = kcache.size(1), ps = kcache.size(2), dk = kcache.size(3);
  const int dv = vcache.size(3);
  SEQ_CHECK(kcache.is_contiguous() && vcache.is_contiguous() &&
                vcache.size(0) == kcache.size(0) && vcache.size(1) == G &&
                vcache.size(2) == ps &&
                kcache.scalar_type() == proj.scalar_type() &&
                vcache.scalar_type() == proj.scalar_type(), "kv cache");
  SEQ_CHECK(proj.stride(1) == 1 && off_k + G * dk <= proj.size(1) &&
                off_v + G * dv <= proj.size(1), "kv projections");
  SEQ_CHECK(slot_mapping.scalar_type() == torch::kLong &&
                slot_mapping.is_contiguous() && slot_mapping.numel() >= T_,
            "slot mapping");
  if (T_ == 0) return;
  DISPATCH_ACT(proj, hipLaunchKernelGGL(
      kv_append_norm_kernel<T>, dim3(T_, G), dim3(64), 0, cur_stream(),
      ptr<T>(kcache), ptr<T>(vcache), cptr<T>(proj), (int)proj.stride(0),
      (int)off_k, (int)off_v, cptr<int64_t>(slot_mapping), G, dk, dv, ps,
      vnorm ? 1 : 0, (float)eps););
}

// out [T, H, kmaps, dv] (fp32 or the cache type); q rows in proj at off_q,
// laid out [H][kmaps][dk]; kcache [P, G, ps, kmaps * dk]. Values come from
// vcache [P, G, ps, dv], or - when vcache is absent - from the first dv
// entries of each cached key row. window 0 = every earlier key is visible.
void paged_attention_rows(torch::Tensor out, torch::Tensor proj, int64_t off_q,
                          torch::Tensor kcache,
                          c10::optional<torch::Tensor> vcache,
                          torch::Tensor page_table, torch::Tensor tok_seq,
                          torch::Tensor positions, torch::Tensor seq_len,
                          c10::optional<torch::Tensor> r1,
                          c10::optional<torch::Tensor> r2, double scale,
                          double temp_coef, int64_t temp_every, int64_t kmaps,
                          int64_t window, int64_t keep_first,
                          c10::optional<torch::Tensor> head_bias,
                          bool sigmoid, double softcap,
                          c10::optional<torch::Tensor> dist_bias,
                          c10::optional<torch::Tensor> sink) {
  SEQ_CHECK(out.dim() == 4 && out.is_contiguous() && out.size(2) == kmaps,
            "attention out [T, H, maps, dv]");
  SEQ_CHECK(softcap >= 0.0 && !(sigmoid && (sink || softcap > 0.0)),
            "soft cap / sink belong to the softmax form");
  if (dist_bias)
    SEQ_CHECK(dist_bias->scalar_type() == torch::kFloat &&
                  dist_bias->is_contiguous() && dist_bias->dim() == 2 &&
                  dist_bias->size(1) >= 1 && dist_bias->size(0) == out.size(1),
              "distance bias fp32 [H, D + 1]");
  if (sink)
    SEQ_CHECK(sink->scalar_type() == torch::kFloat && sink->is_contiguous() &&
                  sink->numel() == out.size(1), "sink fp32 [H]");
  SEQ_CHECK(keep_first >= 0, "kept first keys");
  if (head_bias)
    SEQ_CHECK(head_bias->scalar_type() == torch::kFloat &&
                  head_bias->is_contiguous() &&
                  head_bias->numel() == out.size(1), "head bias fp32 [H]");
  const int T_ = out.size(0), H = out.size(1), dv = out.size(3);
  const int G = kcache.size(1), krow = kcache.size(3);
  SEQ_CHECK(kmaps >= 1 && krow % kmaps == 0 && window >= 0, "key maps/window");
  const int dk = krow / kmaps;
  SEQ_CHECK(out.scalar_type() == proj.scalar_type() ||
                out.scalar_type() == torch::kFloat, "attention out type");
  SEQ_CHECK(kcache.is_contiguous() &&
                kcache.scalar_type() == proj.scalar_type(), "attention cache");
  const void* vptr;
  int vrow;
  if (vcache) {
    SEQ_CHECK(vcache->is_contiguous() && vcache->size(3) == dv &&
                  vcache->size(1) == G && vcache->size(2) == kcache.size(2) &&
                  vcache->size(0) == kcache.size(0) &&
                  vcache->scalar_type() == proj.scalar_type(),
              "attention value cache");
    vptr = vcache->data_ptr();
    vrow = dv;
  } else {
    SEQ_CHECK(dv <= krow, "values inside the key rows");
    vptr = kcache.data_ptr();
    vrow = krow;
  }
  SEQ_CHECK(G >= 1 && H % G == 0 && dv >= 1 && dv <= 64 * EVMAX,
            "attention head sizes");
  SEQ_CHECK(proj.dim() == 2 && proj.stride(1) == 1 && proj.size(0) == T_ &&
                off_q >= 0 && off_q + H * kmaps * dk <= proj.size(1),
            "attention q");
  SEQ_CHECK(page_table.scalar_type() == torch::kInt && page_table.dim() == 2 &&
                page_table.stride(1) == 1, "page table");
  for (const torch::Tensor* t : {&tok_seq, &positions})
    SEQ_CHECK(t->scalar_type() == torch::kInt && t->is_contiguous() &&
                  t->numel() >= T_, "token descriptors");
  SEQ_CHECK(seq_len.scalar_type() == torch::kInt &&
                seq_len.is_contiguous() &&
                seq_len.numel() <= page_table.size(0), "seq_len");
  SEQ_CHECK(r1.has_value() == r2.has_value(), "bias parameters");
  if (r1)
    SEQ_CHECK(kmaps == 1 && r1->scalar_type() == torch::kFloat &&
                  r1->numel() == H && r2->scalar_type() == torch::kFloat &&
                  r2->numel() == H, "bias parameters");
  SEQ_CHECK(temp_every >= 1, "temperature period");
  if (T_ == 0) return;
  const bool f32out = out.scalar_type() == torch::kFloat;
  DISPATCH_ACT(proj, {
    if (f32out)
      launch_attention<T, float>(out, proj, off_q, kcache, vptr, dv, vrow,
                                 page_table, tok_seq, positions, seq_len, r1,
                                 r2, scale, temp_coef, temp_every, (int)kmaps,
                                 (int)window, (int)keep_first, head_bias,
                                 sigmoid, softcap, dist_bias, sink);
    else
      launch_attention<T, T>(out, proj, off_q, kcache, vptr, dv, vrow,
                             page_table, tok_seq, positions, seq_len, r1, r2,
                             scale, temp_coef, temp_every, (int)kmaps,
                             (int)window, (int)keep_first, head_bias, sigmoid,
                             softcap, dist_bias, sink);
  });
}

void biased_attention(torch::Tensor out, torch::Tensor proj, int64_t off_q,
                      torch::Tensor kcache, torch::Tensor vcache,
                      torch::Tensor page_table, torch::Tensor tok_seq,
                      torch::Tensor positions, torch::Tensor seq_len,
                      c10::optional<torch::Tensor> r1,
                      c10::optional<torch::Tensor> r2, double scale,
                      double temp_coef, int64_t temp_every) {
  SEQ_CHECK(out.dim() == 3 && out.is_contiguous() &&
                out.scalar_type() == proj.scalar_type(), "attention out");
  paged_attention_rows(out.unsqueeze(2), proj, off_q, kcache, vcache,
                       page_table, tok_seq, positions, seq_len, r1, r2, scale,
                       temp_coef, temp_every, 1, 0, 0, c10::nullopt, false, 0.0,
                       c10::nullopt, c10::nullopt);
}
