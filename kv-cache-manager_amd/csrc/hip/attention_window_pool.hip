// Attention over a sliding window of tokens and, beside them, one pooled key and value for every
// block of P tokens that lies wholly before the window; rotary positions by interleaved pairs on the
// first dims of a head; keys and values of different sizes.
//
//   row at position i sees   tokens j with 0 <= i - j < window
//                            blocks b with b*P + P - 1 <= i - window   (mean key, mean value of its P tokens)
//                            tokens j < keep_first (the sequence's first tokens stay visible beyond the window)
//   and all of them share one softmax; score = (q . k) * scale_h with a factor per query head, and with a cap c > 0
//   score <- c tanh(score / c); then, with a slope per query head, score <- score - slope_h * (i - j) for token j (a bias
//   that grows with the distance; not offered together with pooled blocks, which have no one distance).  The output may be
//   multiplied element by element with sigmoid(gate) (32-bit gate logits of the output's shape) before it is stored.
//
// Pages: keys [pages, kv_heads, B, d], values transposed [pages, kv_heads, dv, B] (as the other
// attentions of this library keep them).  Pooled entries are 32-bit and live with the page that holds
// their block's last token: [pages, kv_heads, E, d] and [pages, kv_heads, E, dv] with E = ceil(B / P)
// entries a page; block b, whose last token e = b*P + P - 1 lies in the sequence's page number e / B,
// is entry b - floor((e / B) * B / P) there.  An entry is made by the step that stores its block's last
// token, from the P keys and values as the pages hold them, added in ascending position: it does not
// depend on how the prompt was cut.  Giving a page back gives its entries back.
//
// Four waves per (row, query head); blocks are walked 64 at a time from block 0, tokens 64 at a time in
// chunks that start at absolute multiples of 64, with a running maximum: a row's result is a fixed
// sequence of operations on its own keys, whatever else the launch holds and whichever pages it reads.
#include <cfloat>

#include "common.h"
#include "kvcm_hip.h"

namespace kvcm {

constexpr int kWpWaves = 4;
constexpr int kWpMaxValueDim = 512;

// ------------------------------------------------------------------------- angles of a step
// cos_sin[t, i] = (cos, sin) of position * base^(-2i/dims).  The angle is formed in double precision
// (a 32-bit product of a position in the thousands loses the low bits of the angle).
__global__ void rotary_pairs_table_kernel(const int* __restrict__ positions, float2* __restrict__ cos_sin, int T, int half,
                                          double log_base, int dims) {
  const int idx = blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= T * half) return;
  const int t = idx / half, i = idx % half;
  const double freq = exp(-log_base * (2.0 * i) / double(dims));
  const double a = double(positions[t]) * freq;
  cos_sin[idx] = float2{static_cast<float>(cos(a)), static_cast<float>(sin(a))};
}

// cos_sin[t, i] = factor * (cos, sin) of position * freqs[i], for rotations whose frequencies are not a plain power
// law (rescaled for longer contexts pair by pair): the caller brings them as a table, in double precision.
__global__ void rotary_freq_table_kernel(const int* __restrict__ positions, const double* __restrict__ freqs,
                                         float2* __restrict__ cos_sin, int T, int half, double factor) {
  const int idx = blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= T * half) return;
  const double a = double(positions[idx / half]) * freqs[idx % half];
  cos_sin[idx] = float2{static_cast<float>(factor * cos(a)), static_cast<float>(factor * sin(a))};
}

// ------------------------------------------------------- rotation and the page write of a step
// src [T, nh*d + nkv*d + nkv*dv] 32-bit (q | k | v); or q alone there and (k | v) in rows of their own, kv_src
// [T, nkv*d + nkv*dv] (a query that is made by a later product than the keys).  q (rotated) -> q_out [T, nh*d]; k
// (rotated) and v -> their page slot; a row without a slot reads no k and no v.  halves 0: the pair (2i, 2i+1),
// i < rot/2, is turned; halves 1: the pair (i, i + rot/2); the rest passes.
template <class T>
__global__ void __launch_bounds__(256)
    rotate_store_kernel(const float* __restrict__ src, int ld, const float* __restrict__ kv_src, int ldkv,
                        const float2* __restrict__ cos_sin, int rot, int halves,
                        const int* __restrict__ slots, T* __restrict__ q_out, int ldq, T* __restrict__ kcache,
                        T* __restrict__ vcache, int nh, int nkv, int d, int dv, int B) {
  const int row = blockIdx.x;
  const float* rq = src + size_t(row) * ld;
  const float* rk = kv_src ? kv_src + size_t(row) * ldkv : rq + size_t(nh) * d;      // (k | v) of the row
  const float2* cs = cos_sin + size_t(row) * (rot / 2);
  const int slot = slots ? slots[row] : -1;
  const int heads = slot >= 0 ? nh + nkv : nh;
  // grid (rows, 1): one workgroup does a whole row; grid (rows, nh + nkv + 1), for steps of few rows: workgroup y does
  // head y of q | k and the last one the values (the same operations on every element either way)
  int e0 = 0, e1 = heads * d;
  bool values = true;
  if (gridDim.y > 1) {
    const int part = blockIdx.y;
    values = part == nh + nkv;
    e0 = values || part >= heads ? 0 : part * d;
    e1 = values || part >= heads ? 0 : e0 + d;
  }
  for (int e = e0 + threadIdx.x; e < e1; e += blockDim.x) {
    const int head = e / d, i = e % d;
    const float* r = head < nh ? rq + size_t(head) * d : rk + size_t(head - nh) * d;      // this head's entries
    float x = r[i];
    if (i < rot) {      // rot is even: the partner lies inside the rotated part too
      const int hr = rot / 2;
      const bool second = halves ? i >= hr : (i & 1);
      const float y = r[halves ? (second ? i - hr : i + hr) : (i ^ 1)];
      const float2 a = cs[halves ? (second ? i - hr : i) : i / 2];
      x = second ? __fmaf_rn(x, a.x, __fmul_rn(y, a.y)) : __fmaf_rn(x, a.x, -__fmul_rn(y, a.y));
    }
    if (head < nh) store_f(q_out + size_t(row) * ldq + e, x);
    else if (slot >= 0) store_f(kcache + ((size_t(slot / B) * nkv + (head - nh)) * B + slot % B) * d + i, x);
  }
  if (slot < 0 || !values) return;
  const float* v = rk + size_t(nkv) * d;
  for (int e = threadIdx.x; e < nkv * dv; e += blockDim.x) {
    const int head = e / dv, i = e % dv;
    store_f(vcache + ((size_t(slot / B) * nkv + head) * dv + i) * B + slot % B, v[e]);
  }
}

// rotate_store with what some attentions do to the projection before the rotation.  q and k are each divided by the
// root mean square over their WHOLE stretch of the row (all heads at once, eps inside the root) and multiplied by a weight
// of that size (wq, wk; null: that stretch passes as it is).  v may be blended with the values another layer made for the
// same row, v <- (1 - mix) v + mix * v_other (v_other null: none); v_keep (null: none) receives the row's values as the
// projection made them, for later layers to blend with.  What is stored in the pages is the blended v.
// Grid (rows, parts).  parts 1: one workgroup does a whole row.  parts nh + nkv + 1, for steps of few rows: workgroup y
// does head y of q | k (it sums the squares of that head's whole stretch itself, in the same order, so the bits are those
// of the one-workgroup form) and the last one the values.
constexpr int kNormRotateFewRows = 16;

template <class T>
__global__ void __launch_bounds__(256)
    norm_rotate_store_kernel(const float* __restrict__ src, int ld, const float* __restrict__ wq, const float* __restrict__ wk,
                             float eps, const float* __restrict__ v_other, int ldvo, float mix, float* __restrict__ v_keep,
                             int ldvk, const float2* __restrict__ cos_sin, int rot, int halves, const int* __restrict__ slots,
                             T* __restrict__ q_out, int ldq, T* __restrict__ kcache, T* __restrict__ vcache, int nh, int nkv,
                             int d, int dv, int B) {
  __shared__ float scratch[256 / kWave + 1];
  const int row = blockIdx.x;
  const float* r = src + size_t(row) * ld;
  const int nq = nh * d, nk = nkv * d;
  int e0 = 0, e1 = nq + nk;
  bool values = true;
  if (gridDim.y > 1) {
    const int part = blockIdx.y;
    values = part == nh + nkv;
    e0 = values ? 0 : part * d;
    e1 = values ? 0 : e0 + d;
  }
  float inv_q = 1.f, inv_k = 1.f;
  if (wq && e0 < nq && e1 > e0) {
    float ss = 0.f;
    for (int e = threadIdx.x; e < nq; e += 256) ss = fmaf(r[e], r[e], ss);
    inv_q = 1.0f / sqrtf(block_sum<256>(ss, scratch) / float(nq) + eps);
  }
  if (wk && e1 > nq) {
    float ss = 0.f;
    for (int e = threadIdx.x; e < nk; e += 256) ss = fmaf(r[nq + e], r[nq + e], ss);
    inv_k = 1.0f / sqrtf(block_sum<256>(ss, scratch) / float(nk) + eps);
  }
  auto normed = [&](int e) {
    const float x = r[e];
    if (e < nq) return wq ? x * inv_q * wq[e] : x;
    return wk ? x * inv_k * wk[e - nq] : x;
  };
  const float2* cs = cos_sin + size_t(row) * (rot / 2);
  const int slot = slots ? slots[row] : -1;
  for (int e = e0 + threadIdx.x; e < e1; e += 256) {
    const int head = e / d, i = e % d;
    float x = normed(e);
    if (i < rot) {
      const int hr = rot / 2;
      const bool second = halves ? i >= hr : (i & 1);
      const float y = normed(head * d + (halves ? (second ? i - hr : i + hr) : (i ^ 1)));
      const float2 a = cs[halves ? (second ? i - hr : i) : i / 2];
      x = second ? __fmaf_rn(x, a.x, __fmul_rn(y, a.y)) : __fmaf_rn(x, a.x, -__fmul_rn(y, a.y));
    }
    if (head < nh) store_f(q_out + size_t(row) * ldq + e, x);
    else if (slot >= 0) store_f(kcache + ((size_t(slot / B) * nkv + (head - nh)) * B + slot % B) * d + i, x);
  }
  if (!values) return;
  const float* v = r + nq + nk;
  for (int e = threadIdx.x; e < nkv * dv; e += 256) {
    float x = v[e];
    if (v_keep) v_keep[size_t(row) * ldvk + e] = x;
    if (v_other) x = __fmaf_rn(mix, v_other[size_t(row) * ldvo + e], __fmul_rn(1.0f - mix, x));
    if (slot >= 0) store_f(vcache + ((size_t(slot / B) * nkv + e / dv) * dv + e % dv) * B + slot % B, x);
  }
}

// ------------------------------------------------------------------- pooled entries of a step
// A row whose position is the last of a block of P makes that block's entry from the pages.
template <class T>
__global__ void __launch_bounds__(kWave)
    pool_update_kernel(const T* __restrict__ kcache, const T* __restrict__ vcache, float* __restrict__ pk,
                       float* __restrict__ pv, const int* __restrict__ tables, int table_stride,
                       const int* __restrict__ row_seq, const int* __restrict__ positions, const int* __restrict__ slots,
                       int nkv, int d, int dv, int B, int P, int E) {
  const int row = blockIdx.x, kvh = blockIdx.y, lane = threadIdx.x;
  const int slot = slots[row];
  const int p = positions[row];
  if (slot < 0 || (p + 1) % P != 0) return;
  const int* table = tables + size_t(row_seq[row]) * table_stride;
  const int pgi = p / B;
  const int entry = p / P - (pgi * B) / P;
  const size_t at = (size_t(slot / B) * nkv + kvh) * E + entry;
  const float inv = 1.0f / float(P);
  for (int i = lane; i < d; i += kWave) {
    float acc = 0.f;
    for (int t = p - P + 1; t <= p; ++t)
      acc += load_f(kcache + ((size_t(table[t / B]) * nkv + kvh) * B + t % B) * d + i);
    pk[at * d + i] = acc * inv;
  }
  for (int i = lane; i < dv; i += kWave) {
    float acc = 0.f;
    for (int t = p - P + 1; t <= p; ++t)
      acc += load_f(vcache + ((size_t(table[t / B]) * nkv + kvh) * dv + i) * B + t % B);
    pv[at * dv + i] = acc * inv;
  }
}

// -------------------------------------------------------------------------------- attention
// dot of a 32-bit vector (LDS) with a stored row, 16 bytes of the row at a time where its length allows
template <class T> struct RowPiece;
template <> struct RowPiece<float> { static constexpr int N = 4; };
template <> struct RowPiece<bf16_t> { static constexpr int N = 8; };

__device__ __forceinline__ void unpack_piece(const float* p, float* f) {
  const float4 v = *reinterpret_cast<const float4*>(p);
  f[0] = v.x; f[1] = v.y; f[2] = v.z; f[3] = v.w;
}
__device__ __forceinline__ void unpack_piece(const bf16_t* p, float* f) {
  const uint4 v = *reinterpret_cast<const uint4*>(p);
  f[0] = bf16_bits_to_float(v.x & 0xffffu); f[1] = bf16_bits_to_float(v.x >> 16);
  f[2] = bf16_bits_to_float(v.y & 0xffffu); f[3] = bf16_bits_to_float(v.y >> 16);
  f[4] = bf16_bits_to_float(v.z & 0xffffu); f[5] = bf16_bits_to_float(v.z >> 16);
  f[6] = bf16_bits_to_float(v.w & 0xffffu); f[7] = bf16_bits_to_float(v.w >> 16);
}

// (four pieces of the row are requested before the first is multiplied: a load per trip of the loop would wait for
// each one in turn)
template <class T>
__device__ __forceinline__ float dot_row(const float* qs, const T* kp, int d, bool wide) {
  constexpr int N = RowPiece<T>::N;
  float s = 0.f;
  if (wide) {
    int i = 0;
    for (; i + 4 * N <= d; i += 4 * N) {
      float f[4][N];
#pragma unroll
      for (int g = 0; g < 4; ++g) unpack_piece(kp + i + g * N, f[g]);
#pragma unroll
      for (int g = 0; g < 4; ++g)
#pragma unroll
        for (int e = 0; e < N; ++e) s = fmaf(qs[i + g * N + e], f[g][e], s);
    }
    for (; i < d; i += N) {
      float f[N];
      unpack_piece(kp + i, f);
#pragma unroll
      for (int e = 0; e < N; ++e) s = fmaf(qs[i + e], f[e], s);
    }
  } else {
    for (int i = 0; i < d; ++i) s = fmaf(qs[i], load_f(kp + i), s);
  }
  return s;
}

// One workgroup of four waves per (row, query head).  The row's chunks (pooled blocks 64 at a time from block 0,
// then tokens in chunks that start at absolute multiples of 64) are dealt to the waves in turn by their number;
// each wave keeps a running maximum over its chunks and the four results are merged at the end in wave order.
// Inside a chunk a lane takes one key for the scores; for the values a lane takes value columns and reads the
// tokens of its column 16 bytes at a time (values are stored transposed: a column's tokens lie side by side).
template <class T>
__global__ void __launch_bounds__(kWpWaves* kWave)
    attention_window_pool_kernel(const T* __restrict__ q, int ldq, T* __restrict__ out, int ldo,
                                 const T* __restrict__ kcache, const T* __restrict__ vcache,
                                 const float* __restrict__ pk, const float* __restrict__ pv,
                                 const int* __restrict__ tables, int table_stride, const int* __restrict__ row_seq,
                                 const int* __restrict__ ctx_lens, const float* __restrict__ head_scale,
                                 const float* __restrict__ dist_slope, const float* __restrict__ gate, int ldg,
                                 int nh, int nkv, int d, int dv, int B, float scale, int window, int P, int E, int keep_first,
                                 float softcap) {
  extern __shared__ float lds[];      // [d] q * scale * head_scale[h]; [waves][64] probabilities; [waves][dv + 2] results
  constexpr int N = RowPiece<T>::N, COLS = kWpMaxValueDim / kWave;
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const int row = blockIdx.x / nh, head = blockIdx.x % nh;
  float* qs = lds;
  float* ps = lds + d + wave * kWave;
  float* merge = lds + d + kWpWaves * kWave;
  {
    const float f = head_scale ? scale * head_scale[head] : scale;
    for (int i = threadIdx.x; i < d; i += kWpWaves * kWave) qs[i] = load_f(q + size_t(row) * ldq + size_t(head) * d + i) * f;
  }
  __syncthreads();
  const int kvh = head / (nh / nkv);
  const int ctx = ctx_lens[row];
  T* orow = out + size_t(row) * ldo + size_t(head) * dv;
  if (ctx <= 0) {
    for (int i = threadIdx.x; i < dv; i += kWpWaves * kWave) store_f(orow + i, 0.f);
    return;
  }
  const int* table = tables + size_t(row_seq[row]) * table_stride;
  const int first = (window > 0 && ctx > window) ? ctx - window : 0;
  const int blocks = (P > 0 && window > 0 && ctx - window >= P) ? (ctx - window) / P : 0;      // those that end at or before ctx - 1 - window
  const int block_chunks = (blocks + kWave - 1) / kWave;
  // tokens at the sequence's start that stay visible beyond the window: those of them that lie before the window's
  // first token get chunks of their own, from token 0, walked after the blocks and before the window
  const int kept = keep_first < first ? keep_first : first;
  const int head_chunks = block_chunks + (kept + kWave - 1) / kWave;
  const int first_chunk = first / kWave, chunks = head_chunks + ((ctx - 1) / kWave - first_chunk + 1);
  const float inv_cap = softcap > 0.f ? 1.0f / softcap : 0.f;
  const float slope = dist_slope ? dist_slope[head] : 0.f;
  const bool wide_k = (d % N == 0) && (reinterpret_cast<uintptr_t>(kcache) % 16 == 0);
  const bool wide_pk = (d % 4 == 0);
  const bool wide_v = (B % N == 0) && (reinterpret_cast<uintptr_t>(vcache) % 16 == 0);
  const size_t khead = size_t(B) * d, kpage = khead * nkv;
  const size_t vhead = size_t(B) * dv, vpage = vhead * nkv;

  float m = -INFINITY, l = 0.f;
  float o[COLS];
#pragma unroll
  for (int i = 0; i < COLS; ++i) o[i] = 0.f;

  for (int c = wave; c < chunks; c += kWpWaves) {
    const bool pooled = c < block_chunks, early = !pooled && c < head_chunks;
    const int c0 = pooled ? c * kWave : early ? (c - block_chunks) * kWave : (first_chunk + (c - head_chunks)) * kWave;
    // the stretch of tokens this chunk may see: the kept first tokens before the window, or the window
    const int lo = early ? 0 : first, hi = early ? kept : ctx;
    const int t = c0 + lane;
    float s = -INFINITY;
    int page = 0, entry = 0;
    bool valid;
    if (pooled) {
      valid = t < blocks;
      if (valid) {
        const int e = t * P + P - 1, pgi = e / B;
        page = table[pgi];
        entry = t - (pgi * B) / P;
        s = dot_row<float>(qs, pk + ((size_t(page) * nkv + kvh) * E + entry) * d, d, wide_pk);
      }
    } else {
      valid = t >= lo && t < hi;
      if (valid) s = dot_row<T>(qs, kcache + size_t(table[t / B]) * kpage + kvh * khead + size_t(t % B) * d, d, wide_k);
    }
    if (softcap > 0.f && valid) s = softcap * tanhf(s * inv_cap);
    if (dist_slope && valid) s = fmaf(-slope, float(ctx - 1 - t), s);
    const float m_new = fmaxf(m, wave_max(s));
    const float alpha = expf(m - m_new);
    const float p = valid ? expf(s - m_new) : 0.f;
    l = l * alpha + wave_sum(p);
#pragma unroll
    for (int i = 0; i < COLS; ++i) o[i] *= alpha;
    m = m_new;
    __builtin_amdgcn_wave_barrier();
    ps[lane] = p;
    __builtin_amdgcn_wave_barrier();
    if (pooled) {
      const int n = blocks - c0 < kWave ? blocks - c0 : kWave;
      for (int j = 0; j < n; ++j) {
        const int page_j = __shfl(page, j, kWave), entry_j = __shfl(entry, j, kWave);
        const float* vp = pv + ((size_t(page_j) * nkv + kvh) * E + entry_j) * dv;
        const float pj = ps[j];
#pragma unroll
        for (int i = 0; i < COLS; ++i) {
          const int cc = lane + i * kWave;
          if (cc < dv) o[i] = fmaf(pj, vp[cc], o[i]);
        }
      }
    } else {
      const int j_lo = lo > c0 ? lo - c0 : 0;
      const int j_hi = hi - c0 < kWave ? hi - c0 : kWave;
      if (wide_v) {
        // all of the chunk's pieces (N tokens of one page each) are requested at once, from places clamped into the
        // context; probabilities of tokens before the window are zero, values beyond the context are cut
        // (pages that the window has passed may have been given back: nothing before the window's first piece is read)
        const int last_piece = ((hi - 1) / N) * N, first_piece = (lo / N) * N;
#pragma unroll
        for (int i = 0; i < COLS; ++i) {
          if (i * kWave >= dv) break;      // the same for every lane: 64 columns at a time, each with its own trip of loads
          const int cc = lane + i * kWave;
          const int col = cc < dv ? cc : dv - 1;
          float f[kWave / N][N];
#pragma unroll
          for (int g = 0; g < kWave / N; ++g) {
            const int tg = c0 + g * N < first_piece ? first_piece : c0 + g * N;
            const int tj = tg < last_piece ? tg : last_piece;
            unpack_piece(vcache + size_t(table[tj / B]) * vpage + kvh * vhead + size_t(col) * B + tj % B, f[g]);
          }
          float acc = o[i];
#pragma unroll
          for (int g = 0; g < kWave / N; ++g)
#pragma unroll
            for (int e = 0; e < N; ++e) {
              const int j = g * N + e;
              acc = fmaf(ps[j], (j >= j_lo && j < j_hi) ? f[g][e] : 0.f, acc);
            }
          if (cc < dv) o[i] = acc;
        }
      } else {
        for (int j = j_lo; j < j_hi; ++j) {
          const int tj = c0 + j;
          const T* vp = vcache + size_t(table[tj / B]) * vpage + kvh * vhead + tj % B;
          const float pj = ps[j];
#pragma unroll
          for (int i = 0; i < COLS; ++i) {
            const int cc = lane + i * kWave;
            if (cc < dv) o[i] = fmaf(pj, load_f(vp + size_t(cc) * B), o[i]);
          }
        }
      }
    }
  }
  // merge the waves' results in wave order
  float* mine = merge + wave * (dv + 2);
#pragma unroll
  for (int i = 0; i < COLS; ++i) {
    const int cc = lane + i * kWave;
    if (cc < dv) mine[cc] = o[i];
  }
  if (lane == 0) {
    mine[dv] = m;
    mine[dv + 1] = l;
  }
  __syncthreads();
  float mm = -INFINITY;
#pragma unroll
  for (int w = 0; w < kWpWaves; ++w) mm = fmaxf(mm, merge[w * (dv + 2) + dv]);
  float wgt[kWpWaves], ll = 0.f;
#pragma unroll
  for (int w = 0; w < kWpWaves; ++w) {
    const float mw = merge[w * (dv + 2) + dv];
    wgt[w] = mw == -INFINITY ? 0.f : expf(mw - mm);
    ll = fmaf(merge[w * (dv + 2) + dv + 1], wgt[w], ll);
  }
  for (int cc = threadIdx.x; cc < dv; cc += kWpWaves * kWave) {
    float acc = 0.f;
#pragma unroll
    for (int w = 0; w < kWpWaves; ++w) acc = fmaf(merge[w * (dv + 2) + cc], wgt[w], acc);
    float res = acc / ll;
    if (gate) res *= 1.0f / (1.0f + expf(-gate[size_t(row) * ldg + size_t(head) * dv + cc]));      // a gate per element of the output
    store_f(orow + cc, res);
  }
}

}  // namespace kvcm

using namespace kvcm;

extern "C" {

int kvcm_rotary_pairs_table(const int* positions, float* cos_sin, int T, int dims, float base, hipStream_t s) {
  if (T == 0 || dims == 0) return 0;
  KVCM_REQUIRE(T > 0 && dims > 0 && dims % 2 == 0 && base > 0.f, "rotary_pairs_table: bad sizes T=%d dims=%d base=%g", T,
               dims, double(base));
  const int n = T * (dims / 2);
  rotary_pairs_table_kernel<<<(n + 255) / 256, 256, 0, s>>>(positions, reinterpret_cast<float2*>(cos_sin), T, dims / 2,
                                                            log(double(base)), dims);
  return launch_status("rotary_pairs_table");
}

int kvcm_rotary_freq_table(const int* positions, const double* freqs, float* cos_sin, int T, int dims, float factor,
                           hipStream_t s) {
  if (T == 0) return 0;
  KVCM_REQUIRE(T > 0 && dims > 0 && dims % 2 == 0 && positions && freqs && cos_sin, "rotary_freq_table: bad sizes T=%d dims=%d", T, dims);
  const int n = T * (dims / 2);
  rotary_freq_table_kernel<<<(n + 255) / 256, 256, 0, s>>>(positions, freqs, reinterpret_cast<float2*>(cos_sin), T, dims / 2,
                                                           double(factor));
  return launch_status("rotary_freq_table");
}

int kvcm_rotate_store(const float* src, int ld, const float* kv_src, int ldkv, const float* cos_sin, int rot, int halves,
                      const int* slots, void* q_out, int dtype, int ldq, void* kcache, void* vcache, int T, int nh, int nkv, int d,
                      int dv, int B, hipStream_t s) {
  if (T == 0) return 0;
  KVCM_REQUIRE(T > 0 && nh > 0 && nkv > 0 && d > 0 && dv > 0 && B > 0, "rotate_store: bad sizes");
  KVCM_REQUIRE(rot % 2 == 0 && rot >= 0 && rot <= d, "rotate_store: %d rotated of %d dims is not supported "
               "(an even number, at most the head's size)", rot, d);
  KVCM_REQUIRE(rot == 0 || cos_sin != nullptr, "rotate_store: a rotation needs its table");
  if (kv_src) KVCM_REQUIRE(ld >= nh * d && ldkv >= nkv * (d + dv) && ldq >= nh * d, "rotate_store: row strides too small");
  else KVCM_REQUIRE(ld >= (slots ? (nh + nkv) * d + nkv * dv : nh * d) && ldq >= nh * d, "rotate_store: row strides too small");
  KVCM_REQUIRE(!slots || (kcache && vcache), "rotate_store: slots without pages");
  const float2* cs = reinterpret_cast<const float2*>(cos_sin);
  const dim3 T_by_parts(T, T <= kNormRotateFewRows ? nh + nkv + 1 : 1);
  if (dtype == kF32)
    rotate_store_kernel<float><<<T_by_parts, 256, 0, s>>>(src, ld, kv_src, ldkv, cs, rot, halves, slots, static_cast<float*>(q_out), ldq,
                                                  static_cast<float*>(kcache), static_cast<float*>(vcache), nh, nkv, d, dv, B);
  else if (dtype == kBF16)
    rotate_store_kernel<bf16_t><<<T_by_parts, 256, 0, s>>>(src, ld, kv_src, ldkv, cs, rot, halves, slots, static_cast<bf16_t*>(q_out), ldq,
                                                   static_cast<bf16_t*>(kcache), static_cast<bf16_t*>(vcache), nh, nkv, d, dv, B);
  else KVCM_REQUIRE(false, "rotate_store: unknown dtype %d", dtype);
  return launch_status("rotate_store");
}

int kvcm_norm_rotate_store(const float* src, int ld, const float* wq, const float* wk, float eps, const float* v_other, int ldvo,
                           float mix, float* v_keep, int ldvk, const float* cos_sin, int rot, int halves, const int* slots,
                           void* q_out, int dtype, int ldq, void* kcache, void* vcache, int T, int nh, int nkv, int d, int dv, int B,
                           hipStream_t s) {
  if (T == 0) return 0;
  KVCM_REQUIRE(T > 0 && nh > 0 && nkv > 0 && d > 0 && dv > 0 && B > 0, "norm_rotate_store: bad sizes");
  KVCM_REQUIRE(rot % 2 == 0 && rot >= 0 && rot <= d, "norm_rotate_store: %d rotated of %d dims is not supported "
               "(an even number, at most the head's size)", rot, d);
  KVCM_REQUIRE(rot == 0 || cos_sin != nullptr, "norm_rotate_store: a rotation needs its table");
  KVCM_REQUIRE(ld >= (nh + nkv) * d + nkv * dv && ldq >= nh * d, "norm_rotate_store: row strides too small");
  KVCM_REQUIRE((!v_other || ldvo >= nkv * dv) && (!v_keep || ldvk >= nkv * dv), "norm_rotate_store: rows of values too short");
  KVCM_REQUIRE(!slots || (kcache && vcache), "norm_rotate_store: slots without pages");
  const float2* cs = reinterpret_cast<const float2*>(cos_sin);
  // few rows: a workgroup per head, so that a single row is not the work of one compute unit (the same bits either way)
  const dim3 grid(T, T <= kNormRotateFewRows ? nh + nkv + 1 : 1);
  if (dtype == kF32)
    norm_rotate_store_kernel<float><<<grid, 256, 0, s>>>(src, ld, wq, wk, eps, v_other, ldvo, mix, v_keep, ldvk, cs, rot, halves, slots,
                                                       static_cast<float*>(q_out), ldq, static_cast<float*>(kcache),
                                                       static_cast<float*>(vcache), nh, nkv, d, dv, B);
  else if (dtype == kBF16)
    norm_rotate_store_kernel<bf16_t><<<grid, 256, 0, s>>>(src, ld, wq, wk, eps, v_other, ldvo, mix, v_keep, ldvk, cs, rot, halves, slots,
                                                        static_cast<bf16_t*>(q_out), ldq, static_cast<bf16_t*>(kcache),
                                                        static_cast<bf16_t*>(vcache), nh, nkv, d, dv, B);
  else KVCM_REQUIRE(false, "norm_rotate_store: unknown dtype %d", dtype);
  return launch_status("norm_rotate_store");
}

int kvcm_pool_update(const void* kcache, const void* vcache, int dtype, float* pk, float* pv, const int* tables,
                     int table_stride, const int* row_seq, const int* positions, const int* slots, int T, int nkv, int d,
                     int dv, int B, int P, int E, hipStream_t s) {
  if (T == 0 || P <= 0) return 0;
  KVCM_REQUIRE(T > 0 && nkv > 0 && d > 0 && dv > 0 && B > 0, "pool_update: bad sizes");
  KVCM_REQUIRE(E == (B + P - 1) / P, "pool_update: %d entries a page do not fit pages of %d and blocks of %d", E, B, P);
  KVCM_REQUIRE(nkv <= 65535, "pool_update: too many kv heads");
  const dim3 grid(T, nkv);
  if (dtype == kF32)
    pool_update_kernel<float><<<grid, kWave, 0, s>>>(static_cast<const float*>(kcache), static_cast<const float*>(vcache), pk,
                                                      pv, tables, table_stride, row_seq, positions, slots, nkv, d, dv, B, P, E);
  else if (dtype == kBF16)
    pool_update_kernel<bf16_t><<<grid, kWave, 0, s>>>(static_cast<const bf16_t*>(kcache), static_cast<const bf16_t*>(vcache),
                                                       pk, pv, tables, table_stride, row_seq, positions, slots, nkv, d, dv, B, P, E);
  else KVCM_REQUIRE(false, "pool_update: unknown dtype %d", dtype);
  return launch_status("pool_update");
}

int kvcm_attention_window_pool(const void* q, int dtype, int ldq, void* out, int ldo, const void* kcache, const void* vcache,
                               const float* pk, const float* pv, const int* tables, int table_stride, const int* row_seq,
                               const int* ctx_lens, const float* head_scale, const float* dist_slope, const float* gate, int ldg,
                               int T, int nh, int nkv, int d, int dv, int B, float scale, int window, int P, int E, int keep_first,
                               float softcap, hipStream_t s) {
  if (T == 0) return 0;
  KVCM_REQUIRE(T > 0 && nh > 0 && nkv > 0 && B > 0 && d > 0, "attention_window_pool: bad sizes T=%d heads=%d kv_heads=%d", T, nh, nkv);
  KVCM_REQUIRE(nh % nkv == 0, "attention_window_pool: %d query heads are not a multiple of %d kv heads", nh, nkv);
  KVCM_REQUIRE(dv > 0 && dv <= kWpMaxValueDim, "attention_window_pool: value size %d is not supported (up to %d)", dv, kWpMaxValueDim);
  KVCM_REQUIRE(d <= 1024, "attention_window_pool: key size %d is not supported (up to 1024)", d);
  KVCM_REQUIRE(ldq >= nh * d && ldo >= nh * dv, "attention_window_pool: row strides too small");
  KVCM_REQUIRE(window >= 0 && P >= 0, "attention_window_pool: negative window or block");
  KVCM_REQUIRE(P == 0 || (pk && pv && E == (B + P - 1) / P), "attention_window_pool: pooled blocks need their entries");
  KVCM_REQUIRE(keep_first >= 0 && softcap >= 0.f, "attention_window_pool: negative count of kept tokens or score cap");
  KVCM_REQUIRE(!dist_slope || P == 0, "attention_window_pool: a distance bias beside pooled blocks is not supported");
  KVCM_REQUIRE(!gate || ldg >= nh * dv, "attention_window_pool: the gate's rows are too short");
  const long long blocks = static_cast<long long>(T) * nh;
  KVCM_REQUIRE(blocks < (1ll << 31), "attention_window_pool: too many rows");
  const size_t lds = sizeof(float) * (d + kWpWaves * kWave + kWpWaves * (dv + 2));
  if (dtype == kF32)
    attention_window_pool_kernel<float><<<static_cast<unsigned>(blocks), kWpWaves * kWave, lds, s>>>(
        static_cast<const float*>(q), ldq, static_cast<float*>(out), ldo, static_cast<const float*>(kcache),
        static_cast<const float*>(vcache), pk, pv, tables, table_stride, row_seq, ctx_lens, head_scale, dist_slope, gate,
        ldg, nh, nkv, d, dv, B, scale, window, P, E, keep_first, softcap);
  else if (dtype == kBF16)
    attention_window_pool_kernel<bf16_t><<<static_cast<unsigned>(blocks), kWpWaves * kWave, lds, s>>>(
        static_cast<const bf16_t*>(q), ldq, static_cast<bf16_t*>(out), ldo, static_cast<const bf16_t*>(kcache),
        static_cast<const bf16_t*>(vcache), pk, pv, tables, table_stride, row_seq, ctx_lens, head_scale, dist_slope, gate,
        ldg, nh, nkv, d, dv, B, scale, window, P, E, keep_first, softcap);
  else KVCM_REQUIRE(false, "attention_window_pool: unknown dtype %d", dtype);
  return launch_status("attention_window_pool");
}

}  // extern "C"
