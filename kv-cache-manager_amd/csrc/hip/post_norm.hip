// Layers that norm AFTER the sum: x <- ln(alpha * x + y) * w, with y a sublayer's output and
// ln(v) = (v - mean(v)) / sqrt(mean((v - mean(v))^2) + eps), a layer norm with a weight and no bias.
//
//   layernorm_post   v = alpha * x + y (+ bias); x <- ln(v) * w in place, and the new rows once more in the compute
//                    dtype for the sublayer that reads them next, one launch for all of it.  y may be the un-added
//                    slices of a product that was split along K: they are added here, in their order.  With a row
//                    gather (the model's last norm, on the rows whose logits are wanted) nothing is written back.
//   head_norm_store  what an attention with a norm per head does between its projection and its pages: biases, each q and
//                    k head divided by its own root mean square and multiplied by one weight of the head's size, the query
//                    times a temperature that grows with the logarithm of its position, k to its page slot, and as values
//                    either the projection's own or the keys as projected (before their norm).
//
// All arithmetic is 32-bit; a row's result is one fixed sequence of operations on that row alone.
#include "common.h"
#include "kvcm_hip.h"

namespace kvcm {

constexpr int kPostThreads = 256;

// Sum over the workgroup's four waves with one barrier: every thread adds the waves' sums itself, in wave order.  Each
// reduction of a kernel brings a scratch array of its own, so that none has to wait for the readers of the one before.
__device__ __forceinline__ float post_block_sum(float v, float* scratch /* kPostThreads / 64 floats, not shared with another sum */) {
  v = wave_sum(v);
  if (threadIdx.x % kWave == 0) scratch[threadIdx.x / kWave] = v;
  __syncthreads();
  float s = 0.f;
#pragma unroll
  for (int w = 0; w < kPostThreads / kWave; ++w) s += scratch[w];
  return s;
}

// any row length: the row is formed three times from its sources (mean, deviations, result)
template <class TO>
__global__ void __launch_bounds__(kPostThreads)
    layernorm_post_kernel(float* __restrict__ x, const float* __restrict__ a, int a_splits, size_t split_stride,
                          const float* __restrict__ bias, float alpha, const float* __restrict__ w,
                          const int* __restrict__ rows, TO* __restrict__ out, int H, float eps) {
  __shared__ float scratch_mean[kPostThreads / kWave], scratch_var[kPostThreads / kWave];
  const int r = blockIdx.x;
  const int src = rows ? rows[r] : r;
  float* xr = x + size_t(src) * H;
  const float* ar = a ? a + size_t(src) * H : nullptr;
  auto value = [&](int i) {
    float v = alpha * xr[i];
    if (ar) {
      float y = ar[i];
      for (int sl = 1; sl < a_splits; ++sl) y += ar[size_t(sl) * split_stride + i];
      v += y;
    }
    if (bias) v += bias[i];
    return v;
  };
  const float inv_h = 1.0f / float(H);
  float sum = 0.f;
  for (int i = threadIdx.x; i < H; i += kPostThreads) sum += value(i);
  const float mean = post_block_sum(sum, scratch_mean) * inv_h;
  float sq = 0.f;
  for (int i = threadIdx.x; i < H; i += kPostThreads) {
    const float c = value(i) - mean;
    sq = fmaf(c, c, sq);
  }
  const float inv = 1.0f / sqrtf(post_block_sum(sq, scratch_var) * inv_h + eps);
  __syncthreads();      // nobody writes the stream before everybody has read it for the last statistic
  for (int i = threadIdx.x; i < H; i += kPostThreads) {
    const float y = (value(i) - mean) * inv * w[i];
    if (!rows) xr[i] = y;      // each element is read and written by one thread only
    if (out) store_f(out + size_t(r) * H + i, y);
  }
}

// rows of a multiple of four values, at most 1024 * G of them: read once, 16 bytes a load, kept in registers
template <class TO, int G>
__global__ void __launch_bounds__(kPostThreads)
    layernorm_post_rows_kernel(float* __restrict__ x, const float* __restrict__ a, int a_splits, size_t split_stride,
                               const float* __restrict__ bias, float alpha, const float* __restrict__ w,
                               const int* __restrict__ rows, TO* __restrict__ out, int H, float eps) {
  __shared__ float scratch_mean[kPostThreads / kWave], scratch_var[kPostThreads / kWave];
  const int r = blockIdx.x;
  const int src = rows ? rows[r] : r;
  float* xr = x + size_t(src) * H;
  float v[G][4];
  bool in[G];
#pragma unroll
  for (int g = 0; g < G; ++g) {
    const int i = (g * kPostThreads + threadIdx.x) * 4;
    in[g] = i < H;
    const int ic = in[g] ? i : 0;
    const float4 vx = *reinterpret_cast<const float4*>(xr + ic);
    v[g][0] = alpha * vx.x; v[g][1] = alpha * vx.y; v[g][2] = alpha * vx.z; v[g][3] = alpha * vx.w;
    if (a) {
      const float* p = a + size_t(src) * H + ic;
      float4 y = *reinterpret_cast<const float4*>(p);
#pragma unroll 4
      for (int sl = 1; sl < a_splits; ++sl) {
        const float4 t = *reinterpret_cast<const float4*>(p + size_t(sl) * split_stride);
        y.x += t.x; y.y += t.y; y.z += t.z; y.w += t.w;
      }
      v[g][0] += y.x; v[g][1] += y.y; v[g][2] += y.z; v[g][3] += y.w;
    }
    if (bias) {
      const float4 t = *reinterpret_cast<const float4*>(bias + ic);
      v[g][0] += t.x; v[g][1] += t.y; v[g][2] += t.z; v[g][3] += t.w;
    }
  }
  const float inv_h = 1.0f / float(H);
  float sum = 0.f;
#pragma unroll
  for (int g = 0; g < G; ++g)
#pragma unroll
    for (int e = 0; e < 4; ++e)
      if (in[g]) sum += v[g][e];
  const float mean = post_block_sum(sum, scratch_mean) * inv_h;
  float sq = 0.f;
#pragma unroll
  for (int g = 0; g < G; ++g)
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      v[g][e] -= mean;
      if (in[g]) sq = fmaf(v[g][e], v[g][e], sq);
    }
  const float inv = 1.0f / sqrtf(post_block_sum(sq, scratch_var) * inv_h + eps);
#pragma unroll
  for (int g = 0; g < G; ++g) {
    if (!in[g]) continue;
    const int i = (g * kPostThreads + threadIdx.x) * 4;
    const float4 ww = *reinterpret_cast<const float4*>(w + i);
    const float4 y = float4{v[g][0] * inv * ww.x, v[g][1] * inv * ww.y, v[g][2] * inv * ww.z, v[g][3] * inv * ww.w};
    if (!rows) *reinterpret_cast<float4*>(xr + i) = y;
    if (out) {
      TO* o = out + size_t(r) * H + i;
      store_f(o, y.x); store_f(o + 1, y.y); store_f(o + 2, y.z); store_f(o + 3, y.w);
    }
  }
}

// One wave per (row, head): the nh query heads, the nkv key heads and, where the projection brings values of its own,
// the nkv value heads of a row [q (nh*d) | k (nkv*d) | v (nkv*dv)].
template <class T>
__global__ void __launch_bounds__(256)
    head_norm_store_kernel(const float* __restrict__ src, int ld, const float* __restrict__ bias, const float* __restrict__ wq,
                           const float* __restrict__ wk, float eps, const int* __restrict__ positions, float temp_coef,
                           int temp_every, int values_are_keys, const int* __restrict__ slots, T* __restrict__ q_out, int ldq,
                           T* __restrict__ kcache, T* __restrict__ vcache, long long items, int nh, int nkv, int d, int dv, int B) {
  const long long item = static_cast<long long>(blockIdx.x) * (256 / kWave) + threadIdx.x / kWave;
  if (item >= items) return;
  const int lane = threadIdx.x % kWave;
  const int per_row = nh + nkv + (values_are_keys ? 0 : nkv);
  const int row = static_cast<int>(item / per_row), part = static_cast<int>(item % per_row);
  const float* r = src + size_t(row) * ld;
  const int slot = slots ? slots[row] : -1;
  if (part >= nh + nkv) {      // a value head of the projection's own
    if (slot < 0) return;
    const int head = part - nh - nkv, at = (nh + nkv) * d + head * dv;
    for (int i = lane; i < dv; i += kWave)
      store_f(vcache + ((size_t(slot / B) * nkv + head) * dv + i) * B + slot % B, r[at + i] + (bias ? bias[at + i] : 0.f));
    return;
  }
  const bool query = part < nh;
  if (!query && slot < 0) return;
  const int at = part * d;
  const float* w = query ? wq : wk;
  float inv = 1.f;
  if (w) {
    float ss = 0.f;
    for (int i = lane; i < d; i += kWave) {
      const float x = r[at + i] + (bias ? bias[at + i] : 0.f);
      ss = fmaf(x, x, ss);
    }
    inv = 1.0f / sqrtf(wave_sum(ss) / float(d) + eps);
  }
  if (query) {
    float temp = 1.f;
    if (temp_every > 0) temp = fmaf(temp_coef, logf(float((positions[row] + 1) / temp_every + 1)), 1.0f);
    for (int i = lane; i < d; i += kWave) {
      const float x = r[at + i] + (bias ? bias[at + i] : 0.f);
      store_f(q_out + size_t(row) * ldq + at + i, (w ? x * inv * w[i] : x) * temp);
    }
    return;
  }
  const int head = part - nh;
  for (int i = lane; i < d; i += kWave) {
    const float x = r[at + i] + (bias ? bias[at + i] : 0.f);
    store_f(kcache + ((size_t(slot / B) * nkv + head) * B + slot % B) * d + i, w ? x * inv * w[i] : x);
    if (values_are_keys) store_f(vcache + ((size_t(slot / B) * nkv + head) * dv + i) * B + slot % B, x);
  }
}

}  // namespace kvcm

using namespace kvcm;

extern "C" {

// x [T, H] 32-bit.  a: the sublayer's output [T, H] or its un-added slices [a_splits][T][H], split_stride floats apart
// (null: nothing is added); bias [H] or null; rows: source rows of the R outputs (null: row r, and x is updated in
// place); out [R, H] in out_dtype or null.
int kvcm_layernorm_post(float* x, const float* a, int a_splits, long long split_stride, const float* bias, float alpha,
                        const float* weight, const int* rows, void* out, int out_dtype, int R, int H, float eps, hipStream_t s) {
  if (R == 0) return 0;
  KVCM_REQUIRE(R > 0 && H > 0 && x && weight, "layernorm_post: bad sizes R=%d H=%d", R, H);
  KVCM_REQUIRE(out || !rows, "layernorm_post: gathered rows need an output");
  KVCM_REQUIRE(a_splits >= 1 && split_stride >= 0, "layernorm_post: an addition has at least one slice");
  KVCM_REQUIRE(!out || out_dtype == kF32 || out_dtype == kBF16, "layernorm_post: unknown output dtype %d", out_dtype);
  const bool f32 = !out || out_dtype == kF32;
  auto aligned = [](const void* p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; };
  const size_t stride = static_cast<size_t>(split_stride);
  if (H % 4 == 0 && H <= 8192 && aligned(x) && aligned(a) && aligned(bias) && aligned(weight) && (a_splits == 1 || stride % 4 == 0)) {
#define KVCM_POST_ROWS(TO, G) \
  layernorm_post_rows_kernel<TO, G><<<R, kPostThreads, 0, s>>>(x, a, a_splits, stride, bias, alpha, weight, rows, static_cast<TO*>(out), H, eps)
    if (H <= 2048) { if (f32) KVCM_POST_ROWS(float, 2); else KVCM_POST_ROWS(bf16_t, 2); }
    else if (H <= 4096) { if (f32) KVCM_POST_ROWS(float, 4); else KVCM_POST_ROWS(bf16_t, 4); }
    else { if (f32) KVCM_POST_ROWS(float, 8); else KVCM_POST_ROWS(bf16_t, 8); }
#undef KVCM_POST_ROWS
    return launch_status("layernorm_post");
  }
  if (f32) layernorm_post_kernel<float><<<R, kPostThreads, 0, s>>>(x, a, a_splits, stride, bias, alpha, weight, rows, static_cast<float*>(out), H, eps);
  else layernorm_post_kernel<bf16_t><<<R, kPostThreads, 0, s>>>(x, a, a_splits, stride, bias, alpha, weight, rows, static_cast<bf16_t*>(out), H, eps);
  return launch_status("layernorm_post");
}

// src [T, ld] 32-bit rows [q (nh*d) | k (nkv*d) | v (nkv*dv), the last only without values_are_keys]; bias: a row of the
// same layout or null; wq, wk [d] or null (that kind of head passes un-normed); positions [T] (read with temp_every > 0:
// q <- q * (1 + temp_coef * ln(floor((p + 1) / temp_every) + 1))); slots [T] or null (nothing is stored).
int kvcm_head_norm_store(const float* src, int ld, const float* bias, const float* wq, const float* wk, float eps,
                         const int* positions, float temp_coef, int temp_every, int values_are_keys, const int* slots, void* q_out,
                         int dtype, int ldq, void* kcache, void* vcache, int T, int nh, int nkv, int d, int dv, int B, hipStream_t s) {
  if (T == 0) return 0;
  KVCM_REQUIRE(T > 0 && nh > 0 && nkv > 0 && d > 0 && dv > 0 && B > 0 && src && q_out, "head_norm_store: bad sizes");
  KVCM_REQUIRE(!values_are_keys || dv == d, "head_norm_store: keys of %d entries cannot be values of %d", d, dv);
  KVCM_REQUIRE(ld >= (nh + nkv) * d + (values_are_keys ? 0 : nkv * dv) && ldq >= nh * d, "head_norm_store: row strides too small");
  KVCM_REQUIRE(temp_every <= 0 || positions, "head_norm_store: a temperature by position needs the positions");
  KVCM_REQUIRE(!slots || (kcache && vcache), "head_norm_store: slots without pages");
  const long long items = static_cast<long long>(T) * (nh + nkv + (values_are_keys ? 0 : nkv));
  const long long blocks = (items + 3) / 4;
  KVCM_REQUIRE(blocks < (1ll << 31), "head_norm_store: too many rows");
  if (dtype == kF32)
    head_norm_store_kernel<float><<<static_cast<unsigned>(blocks), 256, 0, s>>>(
        src, ld, bias, wq, wk, eps, positions, temp_coef, temp_every, values_are_keys, slots, static_cast<float*>(q_out), ldq,
        static_cast<float*>(kcache), static_cast<float*>(vcache), items, nh, nkv, d, dv, B);
  else if (dtype == kBF16)
    head_norm_store_kernel<bf16_t><<<static_cast<unsigned>(blocks), 256, 0, s>>>(
        src, ld, bias, wq, wk, eps, positions, temp_coef, temp_every, values_are_keys, slots, static_cast<bf16_t*>(q_out), ldq,
        static_cast<bf16_t*>(kcache), static_cast<bf16_t*>(vcache), items, nh, nkv, d, dv, B);
  else KVCM_REQUIRE(false, "head_norm_store: unknown dtype %d", dtype);
  return launch_status("head_norm_store");
}

}  // extern "C"
