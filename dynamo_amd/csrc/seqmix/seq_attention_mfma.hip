// Prompt-portion softmax attention over the paged cache on the matrix cores
// (bf16 only): scores and the weighted sum are mfma_f32_16x16x32_bf16
// products, everything between them is fp32. Options: a logarithmic
// distance bias with a query temperature, a sliding window, several key
// maps per kv head, values that alias the head of the key rows (latent
// attention), fp32 output, kept first keys under a window, a per-head
// constant on the scores, and plain sigmoid weights (not normalised over
// the keys) in place of the softmax; for the softmax form also a soft cap
// on the scaled scores, a bias by key distance from a table, and a per-head
// sink in the denominator.
//
// A workgroup (4 waves) owns a tile of up to 64 consecutive rows of one
// sequence and one (query head, key map); each wave owns 16 rows. Keys and
// values of the kv head are walked in blocks of 64 keys. Key channels are
// staged in LDS in chunks of at most 128 channels as they lie in the page
// (zero padded to multiples of 32), the partial scores accumulating over
// the chunks; values are staged transposed (channel-major), again at most
// 128 channels at a time, so that the B operand of the second product is a
// 16-byte run of keys. Large rows (a 576-wide latent row with 512 value
// channels) therefore need no more LDS than small ones. The fp32 scores
// get the row's temperature and scale, the distance penalty and the mask,
// then an online softmax. Both products are formed transposed
// (S^T = K Q^T, O^T = V^T P^T): a lane then holds the scores of one query
// row, and the weights it computes are, as they lie in its registers, the
// B operand of the second product - as a bf16 hi + lo pair, i.e. two
// products - without passing through LDS. The keys of a block are staged
// for the second product in the order in which the lanes hold them.
//
// Decoded tokens use the same kernel with the roles of the tile's rows
// changed (HEADS): a tile is one token, its rows are the query heads that
// share a kv head (all 16, 64, 128 heads of a latent layer share the one
// cached row, so the products are as dense as in a prompt). The keys of a
// token are split over several workgroups; each leaves an unnormalised
// partial result (max, sum, accumulator) that a merge kernel combines.
//
// Fragment layouts of mfma_f32_16x16x32_bf16 (lane l, lr = l % 16,
// lg = l / 16):  A: A[row = lr][k = 8 lg + i], i = 0..7
//                B: B[k = 8 lg + i][col = lr]
//                D: D[row = 4 lg + r][col = lr], r = 0..3
// S^T block n: A = keys 16 n + (0..15) (rows) x channels, B = Q^T, so
// lane (lr, lg) gets the scores of query row lr with keys 16 n + 4 lg + r.
// O^T: A = V^T (16 channels x 32 keys), B = P^T: lane (lr, lg) supplies
// the weights of query row lr for 8 keys of the 32 - those it holds: of
// half kt of the block, key 32 kt + 16 a + 4 lg + r sits at position
// 32 kt + 8 lg + 4 a + r of the staged value rows. D = O^T[channel 4 lg + r
// of the 16][query row lr].
#include "seq_common.h"

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(8))) short short8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;
typedef __attribute__((ext_vector_type(8))) float f32x8_t;

// sigmoid from the hardware exponential and reciprocal (about 1 ulp each;
// the weights are used with 16 bits of mantissa)
DEVINL float sigmoid_fast(float x) {
  return __builtin_amdgcn_rcpf(1.f + __expf(-x));
}

// tanh from the hardware exponential and reciprocal: 1 - 2 / (1 + e^(2x)),
// exact at both ends (e^(2x) = 0 or inf)
DEVINL float tanh_fast(float x) {
  return 1.f - 2.f * __builtin_amdgcn_rcpf(1.f + __expf(2.f * x));
}

constexpr int BN = 64;    // keys per block
constexpr int PADE = 8;   // padding elements per LDS row (16 bytes)

template <typename TO> DEVINL TO out_cast(float f);
template <> DEVINL float out_cast<float>(float f) { return f; }
template <> DEVINL bf16_t out_cast<bf16_t>(float f) { return from_f<bf16_t>(f); }

struct MfmaArgs {
  const bf16_t* proj; int proj_stride; int off_q;
  const bf16_t* kcache; const bf16_t* vcache;
  const int* page_table; int table_stride;
  const int* tile_row0; const int* tile_rows;
  const int* tok_seq; const int* positions;
  const float* r1; const float* r2;
  int H, G, dk, dv, ps;
  float scale, temp_coef; int temp_every, has_bias;
  int kmaps, krow, vrow, window;
  int keep_first; const float* head_bias; int sigmoid;
  float softcap, inv_softcap; const float* dist_bias; int dist_max;
  const float* sink;
  // HEADS mode: rows of a tile are heads of one decoded token
  const int* seq_len; int nsplit; float* partial;
};

// KC = padded key size / 32, DN = padded value size / 16. EX compiles the
// soft cap and the distance table into the score loop; the variants for
// wide latent rows have no registers to spare and are built without.
template <int KC, int DN, typename TO, bool HEADS, bool EX>
__global__ __launch_bounds__(256) void paged_attention_mfma_kernel(
    TO* __restrict__ out,  // [T, H, kmaps, dv]
    const MfmaArgs a) {
  constexpr int KCH = KC < 4 ? KC : 4;       // key chunk: KCH * 32 channels
  constexpr int NKCH = (KC + KCH - 1) / KCH;
  constexpr int DCH = DN < 8 ? DN : 8;       // value chunk: DCH * 16 channels
  constexpr int NDCH = (DN + DCH - 1) / DCH;
  constexpr int KS = KCH * 32 + PADE;  // k_lds row stride (elements)
  constexpr int VS = BN + PADE;        // vt_lds row stride
  extern __shared__ __attribute__((aligned(16))) short smem[];
  short* k_lds = smem;                    // [BN][KS]
  short* vt_lds = k_lds + BN * KS;        // [DCH * 16][VS]

  const int H = a.H, G = a.G, dk = a.dk, dv = a.dv, ps = a.ps;
  // Workgroups go to the 8 XCDs in turn by their linear index, each XCD
  // with an L2 of its own. Prompt tiles are renumbered so that an XCD gets
  // a contiguous run of (head, tile) pairs: the tiles of a head - and of
  // the heads that share its keys and values - then meet in one L2 instead
  // of every XCD streaming every sequence's keys.
  int bx = blockIdx.x, by = blockIdx.y;
  if (!HEADS) {
    const int total = gridDim.x * gridDim.y;
    if (total % 8 == 0) {
      const int lin = bx + gridDim.x * by;
      const int w = (lin % 8) * (total / 8) + lin / 8;
      bx = w % gridDim.x;
      by = w / gridDim.x;
    }
  }
  const int tile = bx;
  const int gsz = H / G;
  // prompt tiles: blockIdx.y = head * kmaps + map, rows are tokens.
  // HEADS: blockIdx.y = ((kv head * kmaps) + map) * nhb + head block,
  // blockIdx.x is the token and rows are the heads h0 + row.
  const int nhb = (gsz + 63) / 64;
  const int map = HEADS ? (by / nhb) % a.kmaps : by % a.kmaps;
  const int g = HEADS ? by / (nhb * a.kmaps) : (by / a.kmaps) / gsz;
  const int h = HEADS ? g * gsz + (by % nhb) * 64 : by / a.kmaps;
  const int koff = map * dk;
  const int row0 = HEADS ? tile : a.tile_row0[tile];
  const int nrows = HEADS ? min(64, g * gsz + gsz - h) : a.tile_rows[tile];
  const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
  const int lr = lane & 15, lg = lane >> 4;
  const int seq = a.tok_seq[row0];
  if (HEADS && a.seq_len[seq] == 0) return;  // padding row (uniform exit)
  const int* table = a.page_table + (int64_t)seq * a.table_stride;
  const bool active = wid * 16 < nrows;  // this wave has rows (wave-uniform)

  // ---- Q fragments of row wid*16 + lr (zero beyond dk / beyond the tile)
  bf16x8_t q_frag[KC];
  {
    const int arow = wid * 16 + lr;
    const bool ok = arow < nrows;
    const bf16_t* q =
        HEADS ? a.proj + (int64_t)row0 * a.proj_stride + a.off_q +
                    ((h + (ok ? arow : 0)) * a.kmaps + map) * dk
              : a.proj + (int64_t)(row0 + (ok ? arow : 0)) * a.proj_stride +
                    a.off_q + (h * a.kmaps + map) * dk;
#pragma unroll
    for (int kc = 0; kc < KC; kc++) {
      short8_t v;
#pragma unroll
      for (int i = 0; i < 8; i++) {
        const int col = kc * 32 + lg * 8 + i;
        v[i] = (ok && col < dk) ? (short)q[col] : (short)0;
      }
      q_frag[kc] = *reinterpret_cast<bf16x8_t*>(&v);
    }
  }
  // ---- the query row whose scores this lane holds: wid*16 + lr
  const int my_row = wid * 16 + lr;
  const bool my_ok = my_row < nrows;
  const int my_pos = HEADS ? a.positions[row0]
                           : (my_ok ? a.positions[row0 + my_row] : 0);
  float my_qmul = a.scale;
  if (a.temp_coef != 0.f)
    my_qmul *= 1.f + a.temp_coef *
                         logf((float)((my_pos + 1) / a.temp_every) + 1.f);
  const float b1 = a.has_bias ? a.r1[h] : 0.f;
  const float b2 = a.has_bias ? a.r2[h] : 0.f;
  // constant added to the scaled scores of the row's head
  const float my_hb = !a.head_bias ? 0.f
                      : HEADS ? (my_ok ? a.head_bias[h + my_row] : 0.f)
                              : a.head_bias[h];
  // (the tables indexed by head are addressed where they are used, from
  // kernel arguments: nothing of them stays in registers over the key loop
  // when a layer has no such table - the widest variants have none to spare)
  // prompt rows are in order; the heads of a token share its position
  const int kv_end = a.positions[HEADS ? row0 : row0 + nrows - 1] + 1;
  // the first key any row of the tile sees
  const int window = a.window;
  const int pos_first = a.positions[row0];  // smallest position of the tile
  const int kv_begin = window > 0 ? max(0, pos_first - window + 1) : 0;

  float m = -INFINITY, l = 0.f;
  f32x4_t acc_o[DN];  // O^T: channels 16 d + 4 lg + r of query row lr
#pragma unroll
  for (int d = 0; d < DN; d++) acc_o[d] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  // ---- staging through registers: the loads of the next chunk are issued
  // before the products of the current one, so their latency hides behind
  // the matrix cores. One buffer serves key and value chunks in turn.
  constexpr int NSK = (BN * KCH * 4 + 255) / 256;  // 16-byte pieces / thread
  constexpr int NSV = (BN * DCH * 2 + 255) / 256;
  constexpr int NST = NSK > NSV ? NSK : NSV;
  short8_t stage[NST];
  // Loads are unconditional with clamped addresses (a branch around a load
  // would make each wait for the one before); what lies past the end of
  // the keys or of the row is zeroed when the piece is written to LDS.
  // slot of key j: page index and place in the page (shift and mask when
  // the page size is a power of two)
  const bool ps_pow2 = (ps & (ps - 1)) == 0;
  const int ps_shift = __ffs(ps) - 1;
  auto key_row = [&](int j) -> int64_t {
    int pg, in;
    if (ps_pow2) {
      pg = j >> ps_shift;
      in = j & (ps - 1);
    } else {
      pg = j / ps;
      in = j - pg * ps;
    }
    return ((int64_t)table[pg] * G + g) * ps + in;
  };
  // A whole block inside one page and inside the keys (all but a
  // sequence's last block when pages are at least a block long): one page
  // lookup for the workgroup, the rest of a thread's address never changes.
  const bool one_page = ps_pow2 && ps >= BN;
  auto load_k = [&](int t0, int cc) {
    constexpr int kvecs = KCH * 4;  // 16-byte pieces per staged row
    const bool fast = one_page && t0 + BN <= kv_end;
    const bf16_t* base =
        a.kcache +
        ((((int64_t)table[fast ? t0 >> ps_shift : 0] * G + g) * ps +
          (t0 & (ps - 1))) * a.krow + koff);
#pragma unroll
    for (int u = 0; u < NSK; u++) {
      const int slot = threadIdx.x + u * 256;
      const int row = slot / kvecs, v = slot - row * kvecs;
      const int ch = min((cc * KCH * 4 + v) * 8, dk - 8);
      if (fast) {
        stage[u] =
            *reinterpret_cast<const short8_t*>(base + (row * a.krow + ch));
      } else {
        const int j = min(t0 + row, kv_end - 1);
        stage[u] = *reinterpret_cast<const short8_t*>(
            a.kcache + key_row(j) * a.krow + koff + ch);
      }
    }
  };
  auto store_k = [&](int t0, int cc) {
    constexpr int kvecs = KCH * 4;
#pragma unroll
    for (int u = 0; u < NSK; u++) {
      const int slot = threadIdx.x + u * 256;
      const int row = slot / kvecs, v = slot - row * kvecs;
      const bool ok = t0 + row < kv_end && (cc * KCH * 4 + v) * 8 < dk;
      *reinterpret_cast<short8_t*>(k_lds + row * KS + v * 8) =
          ok ? stage[u] : short8_t{};
    }
  };
  // consecutive threads take consecutive keys of one channel group, so the
  // transposed 2-byte LDS writes fall in consecutive banks
  auto load_v = [&](int t0, int vc) {
    const bool fast = one_page && t0 + BN <= kv_end;
    const bf16_t* base =
        a.vcache +
        (((int64_t)table[fast ? t0 >> ps_shift : 0] * G + g) * ps +
         (t0 & (ps - 1))) * a.vrow;
#pragma unroll
    for (int u = 0; u < NSV; u++) {
      const int slot = threadIdx.x + u * 256;
      const int v = slot / BN, row = slot - v * BN;
      const int ch = min((vc * DCH * 2 + v) * 8, dv - 8);
      if (fast) {
        stage[u] =
            *reinterpret_cast<const short8_t*>(base + (row * a.vrow + ch));
      } else {
        const int j = min(t0 + row, kv_end - 1);
        stage[u] = *reinterpret_cast<const short8_t*>(
            a.vcache + key_row(j) * a.vrow + ch);
      }
    }
  };
  auto store_v = [&](int t0, int vc) {
#pragma unroll
    for (int u = 0; u < NSV; u++) {
      const int slot = threadIdx.x + u * 256;
      const int v = slot / BN, row = slot - v * BN;
      const bool ok = t0 + row < kv_end && (vc * DCH * 2 + v) * 8 < dv;
      const short8_t x = ok ? stage[u] : short8_t{};
      // key 32 kt + 16 a + 4 g + r of the block goes to 32 kt + 8 g + 4 a + r
      const int col = (row & 32) | ((row & 12) << 1) | ((row & 16) >> 2) |
                      (row & 3);
#pragma unroll
      for (int e = 0; e < 8; e++) vt_lds[(v * 8 + e) * VS + col] = x[e];
    }
  };

  // key blocks: those that hold kept first keys and lie wholly before the
  // window's first block, then the window's blocks
  const int b_lo = kv_begin / BN;
  const int nsink =
      (a.keep_first > 0 && kv_begin > 0)
          ? min((min(a.keep_first, kv_begin) + BN - 1) / BN, b_lo) : 0;
  const int nvb = nsink + (kv_end + BN - 1) / BN - b_lo;
  const int vstep = HEADS ? a.nsplit : 1;
  auto block_t0 = [&](int vb) {
    return (vb < nsink ? vb : vb - nsink + b_lo) * BN;
  };
  const int vb_first = HEADS ? (int)blockIdx.z : 0;
  if (vb_first < nvb) load_k(block_t0(vb_first), 0);
  for (int vb = vb_first; vb < nvb; vb += vstep) {
    const int t0 = block_t0(vb);
    // ---- S^T = K Q^T over key-channel chunks: s[n][r] is the score of
    //      query row lr with key t0 + 16 n + 4 lg + r
    f32x4_t s[4];
#pragma unroll
    for (int n = 0; n < 4; n++) s[n] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int cc = 0; cc < NKCH; cc++) {
      __syncthreads();  // the previous readers of k_lds are done
      store_k(t0, cc);
      if (cc + 1 < NKCH) load_k(t0, cc + 1);
      else load_v(t0, 0);
      __syncthreads();
      if (active)
#pragma unroll
      for (int n = 0; n < 4; n++) {
#pragma unroll
        for (int kc = 0; kc < KCH; kc++) {
          if (cc * KCH + kc < KC) {
            short8_t kb = *reinterpret_cast<const short8_t*>(
                k_lds + (n * 16 + lr) * KS + kc * 32 + lg * 8);
            s[n] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                *reinterpret_cast<bf16x8_t*>(&kb), q_frag[cc * KCH + kc], s[n],
                0, 0, 0);
          }
        }
      }
    }
    // ---- fp32: scale, penalty, mask, weights of query row lr
    float p[4][4];
    // every row of the tile sees every key of the block (uniform)
    const bool all_seen =
        t0 + BN - 1 <= pos_first && (window == 0 || t0 > kv_end - 1 - window);
    if (a.sigmoid && all_seen) {
#pragma unroll
      for (int n = 0; n < 4; n++)
#pragma unroll
        for (int r = 0; r < 4; r++)
          p[n][r] = sigmoid_fast(s[n][r] * my_qmul + my_hb);
    } else if (a.sigmoid) {
      // unnormalised weights: no running maximum, no rescaling
#pragma unroll
      for (int n = 0; n < 4; n++)
#pragma unroll
        for (int r = 0; r < 4; r++) {
          const int j = t0 + n * 16 + lg * 4 + r;
          const bool seen = j <= my_pos && (window == 0 || j > my_pos - window ||
                                            j < a.keep_first);
          p[n][r] = seen ? sigmoid_fast(s[n][r] * my_qmul + my_hb) : 0.f;
        }
    } else {
      float mt = -INFINITY;
#pragma unroll
      for (int n = 0; n < 4; n++)
#pragma unroll
        for (int r = 0; r < 4; r++) {
          const int j = t0 + n * 16 + lg * 4 + r;
          float x = s[n][r] * my_qmul;
          if (EX && a.softcap > 0.f)
            x = a.softcap * tanh_fast(x * a.inv_softcap);
          x += my_hb;
          if (a.has_bias) x -= b1 * log1pf(b2 * (float)max(my_pos - j, 0));
          if (EX && a.dist_bias)
            x += a.dist_bias[(HEADS ? h + (my_ok ? my_row : 0) : h) *
                                 (a.dist_max + 1) +
                             min(max(my_pos - j, 0), a.dist_max)];
          const bool seen = j <= my_pos && (window == 0 || j > my_pos - window ||
                                            j < a.keep_first);
          x = seen ? x : -INFINITY;
          p[n][r] = x;
          mt = fmaxf(mt, x);
        }
      // the row's keys are spread over the four lane groups
      mt = fmaxf(mt, __shfl_xor(mt, 16, 64));
      mt = fmaxf(mt, __shfl_xor(mt, 32, 64));
      // a row may see nothing of the first blocks (window): then every
      // weight is 0 and the running maximum stays -inf
      const float mn = fmaxf(m, mt);
      const float base = mn == -INFINITY ? 0.f : mn;
      const float corr = expf(m - base);
      float rs = 0.f;
#pragma unroll
      for (int n = 0; n < 4; n++)
#pragma unroll
        for (int r = 0; r < 4; r++) {
          p[n][r] = expf(p[n][r] - base);
          rs += p[n][r];
        }
      rs += __shfl_xor(rs, 16, 64);
      rs += __shfl_xor(rs, 32, 64);
      l = l * corr + rs;
      m = mn;
#pragma unroll
      for (int d = 0; d < DN; d++)
#pragma unroll
        for (int r = 0; r < 4; r++) acc_o[d][r] *= corr;
    }
    // ---- the weights as B operands of the second product, a bf16 pair
    // hi + lo each (about 16 bits of mantissa, so the product below sees
    // the fp32 weights almost exactly): half kt of the block takes
    // p[2 kt + a][r] at k index 8 lg + 4 a + r
    bf16x8_t p_hi[2], p_lo[2];
#pragma unroll
    for (int kt = 0; kt < 2; kt++) {
      f32x8_t w;
#pragma unroll
      for (int i = 0; i < 8; i++) w[i] = p[2 * kt + (i >> 2)][i & 3];
      // vector conversions (round to nearest even): packed converts
      p_hi[kt] = __builtin_convertvector(w, bf16x8_t);
      p_lo[kt] = __builtin_convertvector(
          w - __builtin_convertvector(p_hi[kt], f32x8_t), bf16x8_t);
    }
    // ---- O^T += V^T P^T over value-channel chunks, V staged transposed.
    // Every wave has passed this block's barriers after its reads of the
    // previous block's values, so the first chunk may be written at once.
#pragma unroll
    for (int vc = 0; vc < NDCH; vc++) {
      if (vc) __syncthreads();  // the previous chunk's readers are done
      store_v(t0, vc);
      if (vc + 1 < NDCH) load_v(t0, vc + 1);
      else if (vb + vstep < nvb) load_k(block_t0(vb + vstep), 0);
      __syncthreads();
      if (active)
#pragma unroll
      for (int kt = 0; kt < 2; kt++) {
#pragma unroll
        for (int d = 0; d < DCH; d++) {
          if (vc * DCH + d < DN) {
            short8_t vb = *reinterpret_cast<const short8_t*>(
                vt_lds + (d * 16 + lr) * VS + kt * 32 + lg * 8);
            acc_o[vc * DCH + d] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                *reinterpret_cast<bf16x8_t*>(&vb), p_hi[kt],
                acc_o[vc * DCH + d], 0, 0, 0);
            acc_o[vc * DCH + d] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                *reinterpret_cast<bf16x8_t*>(&vb), p_lo[kt],
                acc_o[vc * DCH + d], 0, 0, 0);
          }
        }
      }
    }
  }
  if (!my_ok) return;
  if (HEADS) {
    // ---- partial result of this key split: [token, head, map, split] x
    //      (max, sum, dv unnormalised channels); the row is head h + my_row
    float* o = a.partial +
               ((((int64_t)row0 * H + h + my_row) * a.kmaps + map) * a.nsplit +
                blockIdx.z) * (dv + 2);
    if (lg == 0) {
      o[0] = m;
      o[1] = l;
    }
#pragma unroll
    for (int d = 0; d < DN; d++)
#pragma unroll
      for (int r = 0; r < 4; r++) {
        const int ch = d * 16 + lg * 4 + r;
        if (ch < dv) o[2 + ch] = acc_o[d][r];
      }
    return;
  }
  // ---- normalise and store query row lr, channels 16 d + 4 lg + r
  float inv = a.sigmoid ? 1.f : 1.f / l;
  if (a.sink) {  // exp(sink) joins the denominator
    const float sk = a.sink[h];  // prompt tiles: one head per workgroup
    const float mm = fmaxf(m, sk);
    const float c = expf(m - mm);
    inv = c / (l * c + expf(sk - mm));
  }
  TO* o = out + (((int64_t)(row0 + my_row) * H + h) * a.kmaps + map) * dv;
#pragma unroll
  for (int d = 0; d < DN; d++)
#pragma unroll
    for (int r = 0; r < 4; r++) {
      const int ch = d * 16 + lg * 4 + r;
      if (ch < dv) o[ch] = out_cast<TO>(acc_o[d][r] * inv);
    }
}

// out[t, h, map, :] from the nsplit (<= 16) partial results of a decoded
// token's head. One workgroup per (token, head * kmaps + map); the split
// weights exp(m_z - max) / sum are formed once, then threads own channels.
constexpr int MAXSPLIT = 16;
__global__ void merge_splits_kernel(float* __restrict__ out,
                                    const float* __restrict__ partial,
                                    const int* __restrict__ tok_seq,
                                    const int* __restrict__ seq_len,
                                    int HM, int nsplit, int dv, int plain_sum,
                                    const float* __restrict__ sink,
                                    int kmaps) {
  const int t = blockIdx.x, hm = blockIdx.y;
  if (seq_len[tok_seq[t]] == 0) return;  // padding row
  const int rec = dv + 2;
  const float* p = partial + ((int64_t)t * HM + hm) * nsplit * rec;
  float w[MAXSPLIT];
  const float sk = sink ? sink[hm / kmaps] : -INFINITY;
  float mx = sk;
#pragma unroll
  for (int z = 0; z < MAXSPLIT; z++) {
    w[z] = z < nsplit ? p[z * rec] : -INFINITY;
    mx = fmaxf(mx, w[z]);
  }
  float lt = sink ? expf(sk - mx) : 0.f;
#pragma unroll
  for (int z = 0; z < MAXSPLIT; z++) {
    w[z] = w[z] == -INFINITY ? 0.f : expf(w[z] - mx);
    if (z < nsplit) lt += w[z] * p[z * rec + 1];
    if (plain_sum) w[z] = 1.f;  // unnormalised weights: the splits just add
  }
  const float inv = plain_sum ? 1.f : 1.f / lt;
  for (int ch = threadIdx.x; ch < dv; ch += blockDim.x) {
    float o = 0.f;
#pragma unroll
    for (int z = 0; z < MAXSPLIT; z++)
      if (z < nsplit) o += w[z] * p[z * rec + 2 + ch];
    out[((int64_t)t * HM + hm) * dv + ch] = o * inv;
  }
}

inline size_t lds_bytes(int KC, int DN) {
  const int KCH = KC < 4 ? KC : 4, DCH = DN < 8 ? DN : 8;
  return (size_t)(BN * (KCH * 32 + PADE) + DCH * 16 * (BN + PADE)) *
         sizeof(short);
}

inline bool score_extras(const MfmaArgs& a) {
  return a.softcap > 0.f || a.dist_bias != nullptr;
}

template <int KC, int DN, typename TO, bool EX>
void launch_ex(dim3 grid, TO* out, const MfmaArgs& a) {
  if (a.partial) {
    if constexpr (std::is_same<TO, float>::value)
      hipLaunchKernelGGL(
          (paged_attention_mfma_kernel<KC, DN, float, true, EX>), grid,
          dim3(256), lds_bytes(KC, DN), cur_stream(), out, a);
  } else {
    hipLaunchKernelGGL((paged_attention_mfma_kernel<KC, DN, TO, false, EX>),
                       grid, dim3(256), lds_bytes(KC, DN), cur_stream(), out,
                       a);
  }
}

template <int KC, int DN, typename TO>
void launch(dim3 grid, TO* out, const MfmaArgs& a) {
  if (score_extras(a)) {
    if constexpr (KC <= 8 && KC != 6 && DN <= 16)
      launch_ex<KC, DN, TO, true>(grid, out, a);
    else
      TORCH_CHECK(false, "seqmix: mfma attention sizes with a soft cap or "
                         "distance table");
  } else {
    launch_ex<KC, DN, TO, false>(grid, out, a);
  }
}

// padded sizes the kernel is built for: key chunks of 32, value chunks of 16
inline int pick_kc(int dk) {
  for (int kc : {2, 4, 6, 8, 10, 18})
    if (dk <= kc * 32) return kc;
  return 0;
}
inline int pick_dn(int dv) {
  for (int dn : {4, 8, 16, 32})
    if (dv <= dn * 16) return dn;
  return 0;
}

template <typename TO>
bool dispatch(int KC, int DN, dim3 grid, TO* out, const MfmaArgs& a) {
#define CASE(KC_, DN_)                                  \
  if (KC == KC_ && DN == DN_) {                         \
    launch<KC_, DN_, TO>(grid, out, a);                 \
    return true;                                        \
  }
  CASE(2, 4) CASE(2, 8) CASE(2, 16)
  CASE(4, 4) CASE(4, 8) CASE(4, 16)
  CASE(8, 4) CASE(8, 8) CASE(8, 16)
  if constexpr (std::is_same<TO, float>::value) {
    CASE(6, 8) CASE(10, 16) CASE(18, 32)
  }
#undef CASE
  return false;
}

inline bool combo_ok(int KC, int DN, bool f32out, bool extras = false) {
  if (KC == 0 || DN == 0) return false;
  if (KC <= 8 && KC != 6 && DN <= 16) return true;
  return !extras && f32out && ((KC == 6 && DN == 8) || (KC == 10 && DN == 16) ||
                    (KC == 18 && DN == 32));
}

void check_softmax_options(int64_t H, bool sigmoid, double softcap,
                           const c10::optional<torch::Tensor>& dist_bias,
                           const c10::optional<torch::Tensor>& sink) {
  SEQ_CHECK(softcap >= 0.0 && !(sigmoid && (sink || softcap > 0.0)),
            "soft cap / sink belong to the softmax form");
  if (dist_bias)
    SEQ_CHECK(dist_bias->scalar_type() == torch::kFloat &&
                  dist_bias->is_contiguous() && dist_bias->dim() == 2 &&
                  dist_bias->size(1) >= 1 && dist_bias->size(0) == H,
              "distance bias fp32 [H, D + 1]");
  if (sink)
    SEQ_CHECK(sink->scalar_type() == torch::kFloat && sink->is_contiguous() &&
                  sink->numel() == H, "sink fp32 [H]");
}

void set_softmax_options(MfmaArgs& a, double softcap,
                         const c10::optional<torch::Tensor>& dist_bias,
                         const c10::optional<torch::Tensor>& sink) {
  a.softcap = (float)softcap;
  a.inv_softcap = softcap > 0.0 ? (float)(1.0 / softcap) : 0.f;
  a.dist_bias = dist_bias ? cptr<float>(*dist_bias) : nullptr;
  a.dist_max = dist_bias ? (int)dist_bias->size(1) - 1 : 0;
  a.sink = sink ? cptr<float>(*sink) : nullptr;
}

}  // namespace

// Whether the matrix-core kernel covers these sizes (bf16 caches only).
// `extras`: with a soft cap or a distance table (fewer sizes are built).
bool paged_attention_mfma_supported(int64_t dk, int64_t dv, bool f32out,
                                    bool extras) {
  if (dk % 8 || dv % 8 || dk < 8 || dv < 8) return false;
  return combo_ok(pick_kc((int)dk), pick_dn((int)dv), f32out, extras);
}
bool biased_attention_mfma_supported(int64_t dk, int64_t dv) {
  return paged_attention_mfma_supported(dk, dv, false, false);
}

// Rows are given as tiles: tile i covers rows [tile_row0[i], + tile_rows[i])
// (at most 64, consecutive positions of one sequence). out [T, H, kmaps, dv]
// fp32 or bf16; values from vcache, or from the head of the key rows.
void paged_attention_mfma(torch::Tensor out, torch::Tensor proj, int64_t off_q,
                          torch::Tensor kcache,
                          c10::optional<torch::Tensor> vcache,
                          torch::Tensor page_table, torch::Tensor tile_row0,
                          torch::Tensor tile_rows, int64_t max_tile_rows,
                          torch::Tensor tok_seq, torch::Tensor positions,
                          c10::optional<torch::Tensor> r1,
                          c10::optional<torch::Tensor> r2, double scale,
                          double temp_coef, int64_t temp_every, int64_t kmaps,
                          int64_t window, int64_t keep_first,
                          c10::optional<torch::Tensor> head_bias,
                          bool sigmoid, double softcap,
                          c10::optional<torch::Tensor> dist_bias,
                          c10::optional<torch::Tensor> sink) {
  SEQ_CHECK(out.dim() == 4 && out.is_contiguous() && out.size(2) == kmaps,
            "mfma attention out [T, H, maps, dv]");
  check_softmax_options(out.size(1), sigmoid, softcap, dist_bias, sink);
  SEQ_CHECK(keep_first >= 0, "kept first keys");
  if (head_bias)
    SEQ_CHECK(head_bias->scalar_type() == torch::kFloat &&
                  head_bias->is_contiguous() &&
                  head_bias->numel() == out.size(1), "head bias fp32 [H]");
  const int T_ = out.size(0), H = out.size(1), dv = out.size(3);
  const int G = kcache.size(1), ps = kcache.size(2), krow = kcache.size(3);
  SEQ_CHECK(kmaps >= 1 && krow % kmaps == 0 && window >= 0, "key maps/window");
  const int dk = krow / kmaps;
  const int NT = tile_row0.size(0);
  const bool f32out = out.scalar_type() == torch::kFloat;
  SEQ_CHECK((f32out || out.scalar_type() == torch::kBFloat16) &&
                proj.scalar_type() == torch::kBFloat16 &&
                kcache.scalar_type() == torch::kBFloat16,
            "mfma attention is bf16");
  SEQ_CHECK(kcache.is_contiguous() && G >= 1 && H % G == 0,
            "mfma attention cache");
  const bf16_t* vptr;
  int vrow;
  if (vcache) {
    SEQ_CHECK(vcache->scalar_type() == torch::kBFloat16 &&
                  vcache->is_contiguous() && vcache->size(3) == dv &&
                  vcache->size(1) == G && vcache->size(2) == ps &&
                  vcache->size(0) == kcache.size(0), "mfma value cache");
    vptr = cptr<bf16_t>(*vcache);
    vrow = dv;
  } else {
    SEQ_CHECK(dv <= krow, "values inside the key rows");
    vptr = cptr<bf16_t>(kcache);
    vrow = krow;
  }
  SEQ_CHECK(paged_attention_mfma_supported(
                dk, dv, f32out, softcap > 0.0 || dist_bias.has_value()),
            "mfma attention sizes");
  SEQ_CHECK(reinterpret_cast<uintptr_t>(kcache.data_ptr()) % 16 == 0 &&
                reinterpret_cast<uintptr_t>(vptr) % 16 == 0 && krow % 8 == 0 &&
                vrow % 8 == 0, "mfma attention cache alignment");
  SEQ_CHECK(proj.dim() == 2 && proj.stride(1) == 1 && proj.size(0) == T_ &&
                off_q >= 0 && off_q + H * kmaps * dk <= proj.size(1),
            "mfma attention q");
  SEQ_CHECK(page_table.scalar_type() == torch::kInt && page_table.dim() == 2 &&
                page_table.stride(1) == 1, "page table");
  for (const torch::Tensor* t : {&tok_seq, &positions})
    SEQ_CHECK(t->scalar_type() == torch::kInt && t->is_contiguous() &&
                  t->numel() >= T_, "token descriptors");
  for (const torch::Tensor* t : {&tile_row0, &tile_rows})
    SEQ_CHECK(t->scalar_type() == torch::kInt && t->is_contiguous() &&
                  t->numel() == NT && t->is_cuda(), "tile descriptors");
  SEQ_CHECK(max_tile_rows >= 1 && max_tile_rows <= 64, "tile height");
  SEQ_CHECK(r1.has_value() == r2.has_value(), "bias parameters");
  if (r1)
    SEQ_CHECK(kmaps == 1 && r1->scalar_type() == torch::kFloat &&
                  r1->numel() == H && r2->scalar_type() == torch::kFloat &&
                  r2->numel() == H, "bias parameters");
  SEQ_CHECK(temp_every >= 1, "temperature period");
  if (NT == 0) return;
  MfmaArgs a;
  a.proj = cptr<bf16_t>(proj); a.proj_stride = (int)proj.stride(0);
  a.off_q = (int)off_q;
  a.kcache = cptr<bf16_t>(kcache); a.vcache = vptr;
  a.page_table = cptr<int>(page_table);
  a.table_stride = (int)page_table.stride(0);
  a.tile_row0 = cptr<int>(tile_row0); a.tile_rows = cptr<int>(tile_rows);
  a.tok_seq = cptr<int>(tok_seq); a.positions = cptr<int>(positions);
  a.r1 = r1 ? cptr<float>(*r1) : nullptr;
  a.r2 = r2 ? cptr<float>(*r2) : nullptr;
  a.H = H; a.G = G; a.dk = dk; a.dv = dv; a.ps = ps;
  a.scale = (float)scale; a.temp_coef = (float)temp_coef;
  a.temp_every = (int)temp_every; a.has_bias = r1 ? 1 : 0;
  a.kmaps = (int)kmaps; a.krow = krow; a.vrow = vrow; a.window = (int)window;
  a.keep_first = (int)keep_first;
  a.head_bias = head_bias ? cptr<float>(*head_bias) : nullptr;
  a.sigmoid = sigmoid ? 1 : 0;
  set_softmax_options(a, softcap, dist_bias, sink);
  a.seq_len = nullptr; a.nsplit = 1; a.partial = nullptr;
  const int KC = pick_kc(dk), DN = pick_dn(dv);
  const dim3 grid(NT, H * kmaps);
  const bool ok = f32out ? dispatch<float>(KC, DN, grid, ptr<float>(out), a)
                         : dispatch<bf16_t>(KC, DN, grid, ptr<bf16_t>(out), a);
  TORCH_CHECK(ok, "seqmix: mfma attention sizes");
}

// Decoded tokens (one row each, rows [0, T) of out/proj): the query heads
// that share a kv head form the rows of a matrix-core tile and the keys of
// a token are split over `nsplit` workgroups. out [T, H, kmaps, dv] fp32;
// partial is scratch [T, H, kmaps, nsplit, dv + 2] fp32.
void paged_attention_mfma_decode(torch::Tensor out, torch::Tensor partial,
                                 torch::Tensor proj, int64_t off_q,
                                 torch::Tensor kcache,
                                 c10::optional<torch::Tensor> vcache,
                                 torch::Tensor page_table,
                                 torch::Tensor tok_seq, torch::Tensor positions,
                                 torch::Tensor seq_len, double scale,
                                 double temp_coef, int64_t temp_every,
                                 int64_t kmaps, int64_t window,
                                 int64_t keep_first,
                                 c10::optional<torch::Tensor> head_bias,
                                 bool sigmoid, double softcap,
                                 c10::optional<torch::Tensor> dist_bias,
                                 c10::optional<torch::Tensor> sink) {
  SEQ_CHECK(out.dim() == 4 && out.is_contiguous() && out.size(2) == kmaps &&
                out.scalar_type() == torch::kFloat,
            "mfma decode out [T, H, maps, dv] fp32");
  SEQ_CHECK(temp_every >= 1, "temperature period");
  check_softmax_options(out.size(1), sigmoid, softcap, dist_bias, sink);
  SEQ_CHECK(keep_first >= 0, "kept first keys");
  if (head_bias)
    SEQ_CHECK(head_bias->scalar_type() == torch::kFloat &&
                  head_bias->is_contiguous() &&
                  head_bias->numel() == out.size(1), "head bias fp32 [H]");
  const int T_ = out.size(0), H = out.size(1), dv = out.size(3);
  const int G = kcache.size(1), ps = kcache.size(2), krow = kcache.size(3);
  SEQ_CHECK(kmaps >= 1 && krow % kmaps == 0 && window >= 0, "key maps/window");
  const int dk = krow / kmaps;
  SEQ_CHECK(partial.dim() == 5 && partial.is_contiguous() &&
                partial.scalar_type() == torch::kFloat &&
                partial.size(0) == T_ && partial.size(1) == H &&
                partial.size(2) == kmaps && partial.size(3) >= 1 &&
                partial.size(4) == dv + 2, "mfma decode scratch");
  const int nsplit = partial.size(3);
  SEQ_CHECK(proj.scalar_type() == torch::kBFloat16 &&
                kcache.scalar_type() == torch::kBFloat16 &&
                kcache.is_contiguous() && G >= 1 && H % G == 0,
            "mfma attention is bf16");
  const bf16_t* vptr;
  int vrow;
  if (vcache) {
    SEQ_CHECK(vcache->scalar_type() == torch::kBFloat16 &&
                  vcache->is_contiguous() && vcache->size(3) == dv &&
                  vcache->size(1) == G && vcache->size(2) == ps &&
                  vcache->size(0) == kcache.size(0), "mfma value cache");
    vptr = cptr<bf16_t>(*vcache);
    vrow = dv;
  } else {
    SEQ_CHECK(dv <= krow, "values inside the key rows");
    vptr = cptr<bf16_t>(kcache);
    vrow = krow;
  }
  SEQ_CHECK(paged_attention_mfma_supported(
                dk, dv, true, softcap > 0.0 || dist_bias.has_value()),
            "mfma attention sizes");
  SEQ_CHECK(reinterpret_cast<uintptr_t>(kcache.data_ptr()) % 16 == 0 &&
                reinterpret_cast<uintptr_t>(vptr) % 16 == 0 && krow % 8 == 0 &&
                vrow % 8 == 0, "mfma attention cache alignment");
  SEQ_CHECK(proj.dim() == 2 && proj.stride(1) == 1 && proj.size(0) >= T_ &&
                off_q >= 0 && off_q + H * kmaps * dk <= proj.size(1),
            "mfma attention q");
  SEQ_CHECK(page_table.scalar_type() == torch::kInt && page_table.dim() == 2 &&
                page_table.stride(1) == 1, "page table");
  for (const torch::Tensor* t : {&tok_seq, &positions})
    SEQ_CHECK(t->scalar_type() == torch::kInt && t->is_contiguous() &&
                  t->numel() >= T_, "token descriptors");
  SEQ_CHECK(seq_len.scalar_type() == torch::kInt && seq_len.is_contiguous() &&
                seq_len.numel() <= page_table.size(0), "seq_len");
  if (T_ == 0) return;
  MfmaArgs a;
  a.proj = cptr<bf16_t>(proj); a.proj_stride = (int)proj.stride(0);
  a.off_q = (int)off_q;
  a.kcache = cptr<bf16_t>(kcache); a.vcache = vptr;
  a.page_table = cptr<int>(page_table);
  a.table_stride = (int)page_table.stride(0);
  a.tile_row0 = nullptr; a.tile_rows = nullptr;
  a.tok_seq = cptr<int>(tok_seq); a.positions = cptr<int>(positions);
  a.r1 = nullptr; a.r2 = nullptr;
  a.H = H; a.G = G; a.dk = dk; a.dv = dv; a.ps = ps;
  a.scale = (float)scale; a.temp_coef = (float)temp_coef;
  a.temp_every = (int)temp_every; a.has_bias = 0;
  a.kmaps = (int)kmaps; a.krow = krow; a.vrow = vrow; a.window = (int)window;
  a.keep_first = (int)keep_first;
  a.head_bias = head_bias ? cptr<float>(*head_bias) : nullptr;
  a.sigmoid = sigmoid ? 1 : 0;
  set_softmax_options(a, softcap, dist_bias, sink);
  a.sink = nullptr;  // the merge of the key splits adds the sink
  a.seq_len = cptr<int>(seq_len); a.nsplit = nsplit;
  a.partial = ptr<float>(partial);
  const int KC = pick_kc(dk), DN = pick_dn(dv);
  const int gsz = H / G, nhb = (gsz + 63) / 64;
  const dim3 grid(T_, G * kmaps * nhb, nsplit);
  TORCH_CHECK(dispatch<float>(KC, DN, grid, ptr<float>(out), a),
              "seqmix: mfma attention sizes");
  SEQ_CHECK(nsplit <= MAXSPLIT, "too many key splits");
  hipLaunchKernelGGL(merge_splits_kernel, dim3(T_, H * kmaps),
                     dim3(dv <= 64 ? 64 : (dv <= 128 ? 128 : 256)), 0,
                     cur_stream(), ptr<float>(out), cptr<float>(partial),
                     cptr<int>(tok_seq), cptr<int>(seq_len), H * (int)kmaps,
                     nsplit, dv, sigmoid ? 1 : 0,
                     sink ? cptr<float>(*sink) : (const float*)nullptr,
                     (int)kmaps);
}

void biased_attention_mfma(torch::Tensor out, torch::Tensor proj, int64_t off_q,
                           torch::Tensor kcache, torch::Tensor vcache,
                           torch::Tensor page_table, torch::Tensor tile_row0,
                           torch::Tensor tile_rows, int64_t max_tile_rows,
                           torch::Tensor tok_seq, torch::Tensor positions,
                           c10::optional<torch::Tensor> r1,
                           c10::optional<torch::Tensor> r2, double scale,
                           double temp_coef, int64_t temp_every) {
  SEQ_CHECK(out.dim() == 3 && out.is_contiguous(), "mfma attention out");
  paged_attention_mfma(out.unsqueeze(2), proj, off_q, kcache, vcache,
                       page_table, tile_row0, tile_rows, max_tile_rows, tok_seq,
                       positions, r1, r2, scale, temp_coef, temp_every, 1, 0, 0,
                       c10::nullopt, false, 0.0, c10::nullopt, c10::nullopt);
}
