// A routed feed-forward: every row picks `top` of E small experts by the softmax of its router logits and gets the
// sum of their outputs weighted by the chosen scores as they are (not renormalized).
//
//   moe_route      32-bit router logits [T, E] -> chosen[T, top] (expert numbers, best first; equal scores: the lower
//                  number) and weight[T, top]: their softmax scores over all E, or (over_chosen) the softmax over the
//                  chosen logits alone, which add up to one.  One wave per row.
//   moe_table_route  chosen[T, top] = table[token of the row, :] (a table of expert numbers per token id), weight = 1 / top
//   moe_up         act[T, top, F] = a(W_up[e] h) for each row's chosen experts, a = square of relu, rounded to the
//                  compute dtype; or, gated, act = silu(W_gate[e] h) * (W_up[e] h) with the two matrices of an expert
//                  stored as one, their rows interleaved sixteen at a time (gate 0..15, up 0..15, gate 16..31, ...)
//   moe_down       out[T, H] (32-bit) = (add +) sum over the row's slots of weight * W_down[e] act[slot]
//
// The two products here take a row at a time: a workgroup owns one (row, slot) and a stretch of output columns, keeps
// the row in LDS as 32-bit values and streams the chosen expert's weight rows, a wave per output column, 16 bytes per
// lane and load, summed across the wave.  A row's result is one fixed sequence of operations on its own data, whatever
// else the step holds.  Only the chosen experts' weights are read: the kernels of steps with few rows.  Steps with
// many rows sort their (row, slot) pairs by expert and run tiles on the matrix cores (moe_grouped.hip).
#include <cfloat>

#include "common.h"
#include "kvcm_hip.h"

namespace kvcm {

constexpr int kMoeMaxTop = 16;
constexpr int kMoeMaxExperts = 1024;      // a row's logits are kept in LDS while its experts are picked

__global__ void __launch_bounds__(256)
    moe_route_kernel(const float* __restrict__ logits, int ld, int splits, size_t split_stride, int E, int top, int over_chosen,
                     int* __restrict__ chosen, float* __restrict__ weight, int T) {
  // up to 64 experts a lane group: the row's logits are formed once (a router product that was split along K arrives as
  // slices, which are added here in their order) and kept in LDS
  __shared__ float zs[256 / kWave][kMoeMaxExperts];
  const int row = blockIdx.x * (256 / kWave) + threadIdx.x / kWave, lane = threadIdx.x % kWave;
  if (row >= T) return;
  float* z = zs[threadIdx.x / kWave];
  for (int e = lane; e < E; e += kWave) {
    float v = logits[size_t(row) * ld + e];
    for (int sl = 1; sl < splits; ++sl) v += logits[size_t(sl) * split_stride + size_t(row) * ld + e];
    z[e] = v;
  }
  __builtin_amdgcn_wave_barrier();
  float mx = -FLT_MAX;
  for (int e = lane; e < E; e += kWave) mx = fmaxf(mx, z[e]);
  mx = wave_max(mx);
  float sum = 0.f;
  for (int e = lane; e < E; e += kWave) sum += expf(z[e] - mx);
  sum = wave_sum(sum);
  const float inv = 1.0f / sum;
  int taken[kMoeMaxTop];
  float picked[kMoeMaxTop];
  for (int s = 0; s < top; ++s) {
    float best = -FLT_MAX;
    int at = 0x7fffffff;
    for (int e = lane; e < E; e += kWave) {
      bool used = false;
      for (int p = 0; p < s; ++p) used |= taken[p] == e;
      const float val = z[e];
      if (!used && (val > best || (val == best && e < at))) { best = val; at = e; }
    }
#pragma unroll
    for (int o = kWave / 2; o > 0; o >>= 1) {
      const float ob = __shfl_xor(best, o, kWave);
      const int oa = __shfl_xor(at, o, kWave);
      if (ob > best || (ob == best && oa < at)) { best = ob; at = oa; }
    }
    taken[s] = at;
    picked[s] = expf(best - mx);      // the first pick is the largest logit: exp(0)
    if (lane == 0) {
      chosen[size_t(row) * top + s] = at;
      if (!over_chosen) weight[size_t(row) * top + s] = picked[s] * inv;
    }
  }
  if (over_chosen && lane == 0) {
    float among = 0.f;
    for (int s = 0; s < top; ++s) among += picked[s];
    const float inv_among = 1.0f / among;
    for (int s = 0; s < top; ++s) weight[size_t(row) * top + s] = picked[s] * inv_among;
  }
}

__global__ void __launch_bounds__(256)
    moe_table_route_kernel(const int* __restrict__ tokens, const int* __restrict__ table, int vocab, int ld, int top,
                           int* __restrict__ chosen, float* __restrict__ weight, int n) {
  const int idx = blockIdx.x * 256 + threadIdx.x;
  if (idx >= n) return;
  const int row = idx / top, s = idx % top;
  const int tok = tokens[row];
  chosen[idx] = (tok >= 0 && tok < vocab) ? table[size_t(tok) * ld + s] : -1;      // (an expert number out of range is skipped by the products)
  weight[idx] = 1.0f / float(top);
}

template <class T> struct Piece;
template <> struct Piece<float> { static constexpr int N = 4; };
template <> struct Piece<bf16_t> { static constexpr int N = 8; };

__device__ __forceinline__ void unpack16(const float* p, float* f) {
  const float4 v = *reinterpret_cast<const float4*>(p);
  f[0] = v.x; f[1] = v.y; f[2] = v.z; f[3] = v.w;
}
__device__ __forceinline__ void unpack16(const bf16_t* p, float* f) {
  const uint4 v = *reinterpret_cast<const uint4*>(p);
  f[0] = bf16_bits_to_float(v.x & 0xffffu); f[1] = bf16_bits_to_float(v.x >> 16);
  f[2] = bf16_bits_to_float(v.y & 0xffffu); f[3] = bf16_bits_to_float(v.y >> 16);
  f[4] = bf16_bits_to_float(v.z & 0xffffu); f[5] = bf16_bits_to_float(v.z >> 16);
  f[6] = bf16_bits_to_float(v.w & 0xffffu); f[7] = bf16_bits_to_float(v.w >> 16);
}

// CW sums at once: out[c] = sum over k of xs[k] * w[c * stride + k], c < CW (columns beyond ``cols`` repeat the last
// one and are dropped by the caller), xs the row in LDS; a lane takes 16-byte pieces of every column's stored row in
// turn, so that CW loads are on their way per trip and the row's values are read from LDS once for all of them.
template <class T, int CW>
__device__ __forceinline__ void wave_dots(const float* xs, const T* w, size_t stride, int cols, int K, int lane, bool vec,
                                          float* out) {
  constexpr int N = Piece<T>::N;
  float acc[CW];
  const T* wc[CW];
#pragma unroll
  for (int c = 0; c < CW; ++c) {
    acc[c] = 0.f;
    wc[c] = w + size_t(c < cols ? c : cols - 1) * stride;
  }
  if (vec) {
    // (two trips' pieces on their way at once; four were measured and gained nothing: the walk is bound by its chain of
    // dependent sums, not by bytes in flight)
#pragma unroll 2
    for (int k = lane * N; k < K; k += kWave * N) {
      float f[CW][N];
#pragma unroll
      for (int c = 0; c < CW; ++c) unpack16(wc[c] + k, f[c]);
      float xv[N];
#pragma unroll
      for (int e = 0; e < N; e += 4) {
        const float4 v = *reinterpret_cast<const float4*>(xs + k + e);
        xv[e] = v.x; xv[e + 1] = v.y; xv[e + 2] = v.z; xv[e + 3] = v.w;
      }
#pragma unroll
      for (int c = 0; c < CW; ++c)
#pragma unroll
        for (int e = 0; e < N; ++e) acc[c] = fmaf(xv[e], f[c][e], acc[c]);
    }
  } else {
    for (int k = lane; k < K; k += kWave) {
      const float x = xs[k];
#pragma unroll
      for (int c = 0; c < CW; ++c) acc[c] = fmaf(x, load_f(wc[c] + k), acc[c]);
    }
  }
#pragma unroll
  for (int c = 0; c < CW; ++c) out[c] = wave_sum(acc[c]);
}

// grid (T * top, column blocks of 4 CW).  h [T, K] in T; w_up [E, F, K]; act [T * top, F].
template <class T, int CW>
__global__ void __launch_bounds__(256)
    moe_up_kernel(const T* __restrict__ h, int ldh, const T* __restrict__ w_up, const int* __restrict__ chosen,
                  T* __restrict__ act, int K, int F, int top, int E, int gated) {
  extern __shared__ __attribute__((aligned(16))) float xs[];
  const int item = blockIdx.x, row = item / top;
  const int e = chosen[item];
  for (int k = threadIdx.x; k < K; k += 256) xs[k] = load_f(h + size_t(row) * ldh + k);
  __syncthreads();
  if (e < 0 || e >= E) return;
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const bool vec = K % Piece<T>::N == 0;
  const int c0 = (blockIdx.y * 4 + wave) * CW;
  if (c0 >= F) return;
  const int cols = F - c0 < CW ? F - c0 : CW;
  float z[CW];
  if (gated) {
    // (F is a multiple of 16 and c0 one of CW <= 4: the wave's columns lie in one stretch of sixteen)
    const T* gate = w_up + (size_t(e) * 2 * F + size_t(c0 / 16) * 32 + c0 % 16) * K;
    float u[CW];
    wave_dots<T, CW>(xs, gate, K, cols, K, lane, vec, z);
    wave_dots<T, CW>(xs, gate + size_t(16) * K, K, cols, K, lane, vec, u);
    if (lane == 0)
      for (int c = 0; c < cols; ++c) store_f(act + size_t(item) * F + c0 + c, silu<T>(z[c]) * u[c]);
    return;
  }
  wave_dots<T, CW>(xs, w_up + (size_t(e) * F + c0) * K, K, cols, K, lane, vec, z);
  if (lane == 0)
    for (int c = 0; c < cols; ++c) {
      const float r = fmaxf(z[c], 0.f);
      store_f(act + size_t(item) * F + c0 + c, r * r);
    }
}

// grid (T, column blocks of 4 CW).  act [T * top, F] in T; w_down [E, H, F]; out [T, H] 32-bit.
template <class T, int CW>
__global__ void __launch_bounds__(256)
    moe_down_kernel(const T* __restrict__ act, const T* __restrict__ w_down, const int* __restrict__ chosen,
                    const float* __restrict__ weight, const float* __restrict__ add, float* __restrict__ out, int F, int H,
                    int top, int E) {
  extern __shared__ __attribute__((aligned(16))) float xs[];      // [top][F4], F4: F rounded up to 4
  const int row = blockIdx.x;
  const int F4 = (F + 3) & ~3;
  for (int k = threadIdx.x; k < top * F; k += 256) xs[(k / F) * F4 + k % F] = load_f(act + size_t(row) * top * F + k);
  __syncthreads();
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const bool vec = F % Piece<T>::N == 0;
  const int c0 = (blockIdx.y * 4 + wave) * CW;
  if (c0 >= H) return;
  const int cols = H - c0 < CW ? H - c0 : CW;
  float acc[CW];
#pragma unroll
  for (int c = 0; c < CW; ++c) acc[c] = 0.f;
  for (int s = 0; s < top; ++s) {
    const int e = chosen[size_t(row) * top + s];
    if (e < 0 || e >= E) continue;
    float z[CW];
    wave_dots<T, CW>(xs + s * F4, w_down + (size_t(e) * H + c0) * F, F, cols, F, lane, vec, z);
    const float g = weight[size_t(row) * top + s];
#pragma unroll
    for (int c = 0; c < CW; ++c) acc[c] = fmaf(g, z[c], acc[c]);
  }
  if (lane == 0)
    for (int c = 0; c < cols; ++c) out[size_t(row) * H + c0 + c] = add ? add[size_t(row) * H + c0 + c] + acc[c] : acc[c];
}

// columns a wave takes at once: as many as still leave the chip a few workgroups per CU
inline int moe_cols_per_wave(long long rows, int cols) {
  for (int cw = 4; cw > 1; cw /= 2)
    if (rows * ((cols + 4 * cw - 1) / (4 * cw)) >= 512) return cw;
  return 1;
}

}  // namespace kvcm

using namespace kvcm;

extern "C" {

int kvcm_moe_route(const float* logits, int ld, int splits, long long split_stride, int E, int top, int over_chosen, int* chosen,
                   float* weight, int T, hipStream_t s) {
  if (T == 0) return 0;
  KVCM_REQUIRE(T > 0 && E > 0 && top > 0 && top <= E && ld >= E, "moe_route: bad sizes T=%d experts=%d top=%d", T, E, top);
  KVCM_REQUIRE(top <= kMoeMaxTop, "moe_route: %d experts a row are not supported (up to %d)", top, kMoeMaxTop);
  KVCM_REQUIRE(E <= kMoeMaxExperts, "moe_route: %d experts are not supported (up to %d)", E, kMoeMaxExperts);
  KVCM_REQUIRE(splits >= 1 && split_stride >= 0, "moe_route: the logits have at least one slice");
  moe_route_kernel<<<(T + 3) / 4, 256, 0, s>>>(logits, ld, splits, static_cast<size_t>(split_stride), E, top, over_chosen, chosen, weight, T);
  return launch_status("moe_route");
}

int kvcm_moe_table_route(const int* tokens, const int* table, int vocab, int ld, int top, int* chosen, float* weight, int T,
                         hipStream_t s) {
  if (T == 0) return 0;
  KVCM_REQUIRE(T > 0 && vocab > 0 && top > 0 && ld >= top && tokens && table && chosen && weight,
               "moe_table_route: bad sizes T=%d vocab=%d top=%d", T, vocab, top);
  KVCM_REQUIRE(static_cast<long long>(T) * top < (1ll << 31), "moe_table_route: too many rows");
  const int n = T * top;
  moe_table_route_kernel<<<(n + 255) / 256, 256, 0, s>>>(tokens, table, vocab, ld, top, chosen, weight, n);
  return launch_status("moe_table_route");
}

// h [T, K] and act [T * top, F] in dtype; w_up [E, F, K] contiguous: act = square(relu(W_up[chosen] h)).  gated: w_up
// [E, 2F, K], an expert's gate and up rows interleaved sixteen at a time: act = silu(W_gate[chosen] h) * (W_up[chosen] h).
int kvcm_moe_up(const void* h, int dtype, int ldh, const void* w_up, const int* chosen, void* act, int T, int K, int F, int top,
                int E, int gated, hipStream_t s) {
  if (T == 0) return 0;
  KVCM_REQUIRE(T > 0 && K > 0 && F > 0 && top > 0 && E > 0 && ldh >= K, "moe_up: bad sizes");
  KVCM_REQUIRE(!gated || F % 16 == 0, "moe_up: gated experts of %d columns are not supported (a multiple of 16)", F);
  KVCM_REQUIRE(static_cast<long long>(T) * top < (1ll << 31) && (F + 3) / 4 <= 65535, "moe_up: too many rows or columns");
  KVCM_REQUIRE(K * sizeof(float) <= 64 * 1024, "moe_up: rows of %d values do not fit the local memory", K);
  KVCM_REQUIRE(reinterpret_cast<uintptr_t>(w_up) % 16 == 0, "moe_up: weights must be 16-byte aligned");
  KVCM_REQUIRE(dtype == kF32 || dtype == kBF16, "moe_up: unknown dtype %d", dtype);
  const int cw = moe_cols_per_wave(static_cast<long long>(T) * top, F);
  const dim3 grid(T * top, (F + 4 * cw - 1) / (4 * cw));
  const size_t lds = K * sizeof(float);
#define KVCM_MOE_UP(TT, CW)                                                                                              \
  moe_up_kernel<TT, CW><<<grid, 256, lds, s>>>(static_cast<const TT*>(h), ldh, static_cast<const TT*>(w_up), chosen,     \
                                               static_cast<TT*>(act), K, F, top, E, gated)
  if (dtype == kF32) { if (cw == 4) KVCM_MOE_UP(float, 4); else if (cw == 2) KVCM_MOE_UP(float, 2); else KVCM_MOE_UP(float, 1); }
  else { if (cw == 4) KVCM_MOE_UP(bf16_t, 4); else if (cw == 2) KVCM_MOE_UP(bf16_t, 2); else KVCM_MOE_UP(bf16_t, 1); }
#undef KVCM_MOE_UP
  return launch_status("moe_up");
}

// act [T * top, F] in dtype; w_down [E, H, F] contiguous; out [T, H] 32-bit; add [T, H] 32-bit or null (out = add + sum).
int kvcm_moe_down(const void* act, int dtype, const void* w_down, const int* chosen, const float* weight, const float* add,
                  float* out, int T, int F, int H, int top, int E, hipStream_t s) {
  if (T == 0) return 0;
  KVCM_REQUIRE(T > 0 && H > 0 && F > 0 && top > 0 && E > 0, "moe_down: bad sizes");
  const size_t lds = static_cast<size_t>(top) * ((F + 3) & ~3) * sizeof(float);
  KVCM_REQUIRE(lds <= 64 * 1024, "moe_down: %d activations of %d values do not fit the local memory", top, F);
  KVCM_REQUIRE(reinterpret_cast<uintptr_t>(w_down) % 16 == 0, "moe_down: weights must be 16-byte aligned");
  KVCM_REQUIRE((H + 3) / 4 <= 65535, "moe_down: too many columns");
  KVCM_REQUIRE(dtype == kF32 || dtype == kBF16, "moe_down: unknown dtype %d", dtype);
  const int cw = moe_cols_per_wave(T, H);
  const dim3 grid(T, (H + 4 * cw - 1) / (4 * cw));
#define KVCM_MOE_DOWN(TT, CW)                                                                                                \
  moe_down_kernel<TT, CW><<<grid, 256, lds, s>>>(static_cast<const TT*>(act), static_cast<const TT*>(w_down), chosen, weight, \
                                                 add, out, F, H, top, E)
  if (dtype == kF32) { if (cw == 4) KVCM_MOE_DOWN(float, 4); else if (cw == 2) KVCM_MOE_DOWN(float, 2); else KVCM_MOE_DOWN(float, 1); }
  else { if (cw == 4) KVCM_MOE_DOWN(bf16_t, 4); else if (cw == 2) KVCM_MOE_DOWN(bf16_t, 2); else KVCM_MOE_DOWN(bf16_t, 1); }
#undef KVCM_MOE_DOWN
  return launch_status("moe_down");
}

}  // extern "C"
