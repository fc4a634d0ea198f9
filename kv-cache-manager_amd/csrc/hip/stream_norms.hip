// Elementwise work around a 32-bit residual stream whose layers run a mixer and a feed-forward side by side:
//
//   dyt_norm       x <- x + a + b (the two sublayer outputs of the layer before), then up to two norms of the
//                  new x in one pass, each  tanh(alpha * x) * w + bias  (a norm without statistics: no sum over
//                  the row, so an element needs nothing but itself), rounded once to the compute dtype; with a
//                  row gather for the head's rows
//   stream_pack    [x + a + b | x0] as rows of the compute dtype: the input of a product that mixes the stream
//                  with the embedding again
//   scale_rows     32-bit values times a factor, in place (a head's logit scale)
//   head_gate      an attention's output times one sigmoid gate per (row, head), or one per element, in place
//   rms_groups     32-bit rows: groups of consecutive columns divided by their root mean square and weighted,
//                  in place (the small latent vector that a latent attention keeps per token) or into rows of the
//                  compute dtype (a latent that the next product reads)
//
// Everything here is 32-bit arithmetic on 32-bit inputs; only the outputs that feed products are rounded.
#include "common.h"
#include "kvcm_hip.h"

namespace kvcm {

template <class TO>
__global__ void __launch_bounds__(256)
    dyt_norm_kernel(float* __restrict__ x, int use_x, const float* __restrict__ a, int a_splits, long long a_stride,
                    const float* __restrict__ b, const int* __restrict__ rows, int write_back, const float* __restrict__ w1,
                    const float* __restrict__ b1, float alpha1, TO* __restrict__ out1, const float* __restrict__ w2,
                    const float* __restrict__ b2, float alpha2, TO* __restrict__ out2, long long n, int H) {
  for (long long idx = static_cast<long long>(blockIdx.x) * 256 + threadIdx.x; idx < n; idx += static_cast<long long>(gridDim.x) * 256) {
    const int r = static_cast<int>(idx / H), c = static_cast<int>(idx % H);
    const size_t src = size_t(rows ? rows[r] : r) * H + c;
    float v = use_x ? x[src] : 0.f;
    if (a)
      for (int sp = 0; sp < a_splits; ++sp) v += a[sp * a_stride + src];      // (the slices of a split product, in split order)
    if (b) v += b[src];
    if (write_back) x[idx] = v;
    if (out1) store_f(out1 + idx, fmaf(tanhf(alpha1 * v), w1[c], b1[c]));
    if (out2) store_f(out2 + idx, fmaf(tanhf(alpha2 * v), w2[c], b2[c]));
  }
}

template <class TO>
__global__ void __launch_bounds__(256)
    stream_pack_kernel(const float* __restrict__ x, const float* __restrict__ a, const float* __restrict__ b,
                       const float* __restrict__ x0, TO* __restrict__ out, long long n, int H) {
  for (long long idx = static_cast<long long>(blockIdx.x) * 256 + threadIdx.x; idx < n; idx += static_cast<long long>(gridDim.x) * 256) {
    const long long r = idx / H;
    const int c = static_cast<int>(idx % H);
    float v = x[idx];
    if (a) v += a[idx];
    if (b) v += b[idx];
    store_f(out + r * 2 * H + c, v);
    store_f(out + r * 2 * H + H + c, x0[idx]);
  }
}

__global__ void __launch_bounds__(256) scale_rows_kernel(float* __restrict__ x, long long n, float factor) {
  for (long long idx = static_cast<long long>(blockIdx.x) * 256 + threadIdx.x; idx < n; idx += static_cast<long long>(gridDim.x) * 256)
    x[idx] *= factor;
}

// x <- cap * tanh(x / cap): values far below the cap pass almost unchanged, none leaves (-cap, cap)
__global__ void __launch_bounds__(256) softcap_rows_kernel(float* __restrict__ x, long long n, float cap) {
  const float inv = 1.0f / cap;
  for (long long idx = static_cast<long long>(blockIdx.x) * 256 + threadIdx.x; idx < n; idx += static_cast<long long>(gridDim.x) * 256)
    x[idx] = cap * tanhf(x[idx] * inv);
}

template <class T>
__global__ void __launch_bounds__(256)
    head_gate_kernel(T* __restrict__ o, int ldo, const float* __restrict__ gate, int ldg, long long n, int heads, int dv,
                     int per_element) {
  const int per_row = heads * dv;
  for (long long idx = static_cast<long long>(blockIdx.x) * 256 + threadIdx.x; idx < n; idx += static_cast<long long>(gridDim.x) * 256) {
    const long long r = idx / per_row;
    const int c = static_cast<int>(idx % per_row);
    const float g = 1.0f / (1.0f + expf(-gate[r * ldg + (per_element ? c : c / dv)]));
    T* p = o + r * ldo + c;
    store_f(p, load_f(p) * g);
  }
}

// one wave per (row, group); out null: in place, else out[row, g * size + i] in TO
template <class TO>
__global__ void __launch_bounds__(256)
    rms_groups_kernel(float* __restrict__ x, int ld, int col0, int size, int groups, const float* __restrict__ w, float eps,
                      TO* __restrict__ out, int ldo, long long items) {
  const long long item = static_cast<long long>(blockIdx.x) * (256 / kWave) + threadIdx.x / kWave;
  if (item >= items) return;
  const int lane = threadIdx.x % kWave;
  float* p = x + (item / groups) * ld + col0 + (item % groups) * size;
  TO* q = out ? out + (item / groups) * ldo + (item % groups) * size : nullptr;
  constexpr int kHeld = 16;      // values a lane keeps: groups of up to 1,024 are read once, all loads on their way together
  if (size <= kHeld * kWave) {
    float v[kHeld];
#pragma unroll
    for (int j = 0; j < kHeld; ++j) {
      const int i = lane + j * kWave;
      v[j] = i < size ? p[i] : 0.f;
    }
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < kHeld; ++j) ss = fmaf(v[j], v[j], ss);      // (the same order of sums as the loop below: lane, then j)
    ss = wave_sum(ss);
    const float inv = 1.0f / sqrtf(ss / float(size) + eps);
#pragma unroll
    for (int j = 0; j < kHeld; ++j) {
      const int i = lane + j * kWave;
      if (i >= size) break;
      const float y = v[j] * inv * w[i];
      if (q) store_f(q + i, y);
      else p[i] = y;
    }
    return;
  }
  float ss = 0.f;
  for (int i = lane; i < size; i += kWave) ss = fmaf(p[i], p[i], ss);
  ss = wave_sum(ss);
  const float inv = 1.0f / sqrtf(ss / float(size) + eps);
  if (q) {
    for (int i = lane; i < size; i += kWave) store_f(q + i, p[i] * inv * w[i]);
  } else {
    for (int i = lane; i < size; i += kWave) p[i] = p[i] * inv * w[i];
  }
}

inline unsigned grid_for(long long n) {
  const long long blocks = (n + 255) / 256;
  return static_cast<unsigned>(blocks < 1 ? 1 : (blocks > 16384 ? 16384 : blocks));
}

}  // namespace kvcm

using namespace kvcm;

extern "C" {

// x [T, H] 32-bit; a, b [T, H] 32-bit or null; a may be the un-added slices of a split product, [a_splits][T][H] with
// a_stride floats between slices (a_splits 1: finished); rows: source rows of the R outputs (null: row r, and then
// x <- x + a + b is written back when write_back is set); use_x 0: the sum starts from zero (x is only written).
// out1 / out2 [R, H] in out_dtype, each with its weight, bias and factor, or null.
int kvcm_dyt_norm(float* x, int use_x, const float* a, int a_splits, long long a_stride, const float* b, const int* rows, int write_back, const float* w1,
                  const float* b1, float alpha1, void* out1, const float* w2, const float* b2, float alpha2, void* out2,
                  int out_dtype, int R, int H, hipStream_t s) {
  if (R == 0) return 0;
  KVCM_REQUIRE(R > 0 && H > 0 && x != nullptr, "dyt_norm: bad sizes R=%d H=%d", R, H);
  KVCM_REQUIRE(!(rows && write_back), "dyt_norm: gathered rows are not written back");
  KVCM_REQUIRE(use_x || a, "dyt_norm: nothing to norm");
  KVCM_REQUIRE(a_splits >= 1 && a_stride >= 0, "dyt_norm: an addition has at least one slice");
  KVCM_REQUIRE((!out1 || (w1 && b1)) && (!out2 || (w2 && b2)), "dyt_norm: an output needs its weight and bias");
  KVCM_REQUIRE(out1 || out2 || write_back, "dyt_norm: nothing to do");
  const long long n = static_cast<long long>(R) * H;
  if (out_dtype == kF32)
    dyt_norm_kernel<float><<<grid_for(n), 256, 0, s>>>(x, use_x, a, a_splits, a_stride, b, rows, write_back, w1, b1, alpha1, static_cast<float*>(out1),
                                                       w2, b2, alpha2, static_cast<float*>(out2), n, H);
  else if (out_dtype == kBF16)
    dyt_norm_kernel<bf16_t><<<grid_for(n), 256, 0, s>>>(x, use_x, a, a_splits, a_stride, b, rows, write_back, w1, b1, alpha1, static_cast<bf16_t*>(out1),
                                                        w2, b2, alpha2, static_cast<bf16_t*>(out2), n, H);
  else KVCM_REQUIRE(false, "dyt_norm: unknown output dtype %d", out_dtype);
  return launch_status("dyt_norm");
}

// out [T, 2H] = [x + a + b | x0]
int kvcm_stream_pack(const float* x, const float* a, const float* b, const float* x0, void* out, int out_dtype, int T, int H,
                     hipStream_t s) {
  if (T == 0) return 0;
  KVCM_REQUIRE(T > 0 && H > 0 && x && x0 && out, "stream_pack: bad arguments");
  const long long n = static_cast<long long>(T) * H;
  if (out_dtype == kF32) stream_pack_kernel<float><<<grid_for(n), 256, 0, s>>>(x, a, b, x0, static_cast<float*>(out), n, H);
  else if (out_dtype == kBF16) stream_pack_kernel<bf16_t><<<grid_for(n), 256, 0, s>>>(x, a, b, x0, static_cast<bf16_t*>(out), n, H);
  else KVCM_REQUIRE(false, "stream_pack: unknown output dtype %d", out_dtype);
  return launch_status("stream_pack");
}

int kvcm_scale_rows(float* x, long long n, float factor, hipStream_t s) {
  if (n == 0) return 0;
  KVCM_REQUIRE(n > 0 && x, "scale_rows: bad arguments");
  scale_rows_kernel<<<grid_for(n), 256, 0, s>>>(x, n, factor);
  return launch_status("scale_rows");
}

int kvcm_softcap_rows(float* x, long long n, float cap, hipStream_t s) {
  if (n == 0) return 0;
  KVCM_REQUIRE(n > 0 && x && cap > 0.f, "softcap_rows: bad arguments (a positive cap)");
  softcap_rows_kernel<<<grid_for(n), 256, 0, s>>>(x, n, cap);
  return launch_status("softcap_rows");
}

// o [T, heads*dv] (dtype) *= sigmoid(gate[T, heads]) per head, or (per_element) sigmoid(gate[T, heads*dv]) per element
int kvcm_head_gate(void* o, int dtype, int ldo, const float* gate, int ldg, int T, int heads, int dv, int per_element, hipStream_t s) {
  if (T == 0) return 0;
  KVCM_REQUIRE(T > 0 && heads > 0 && dv > 0 && o && gate, "head_gate: bad sizes");
  KVCM_REQUIRE(ldo >= heads * dv && ldg >= (per_element ? heads * dv : heads), "head_gate: row strides too small");
  const long long n = static_cast<long long>(T) * heads * dv;
  if (dtype == kF32) head_gate_kernel<float><<<grid_for(n), 256, 0, s>>>(static_cast<float*>(o), ldo, gate, ldg, n, heads, dv, per_element);
  else if (dtype == kBF16) head_gate_kernel<bf16_t><<<grid_for(n), 256, 0, s>>>(static_cast<bf16_t*>(o), ldo, gate, ldg, n, heads, dv, per_element);
  else KVCM_REQUIRE(false, "head_gate: unknown dtype %d", dtype);
  return launch_status("head_gate");
}

// x [T, ld]: columns col0 + g*size .. + size, g < groups, each <- n(.) * w[0..size); with out: x stays and
// out [T, ldo] (out_dtype) receives the groups side by side from its column 0
int kvcm_rms_groups(float* x, int ld, int col0, int size, int groups, const float* w, float eps, void* out, int out_dtype, int ldo,
                    int T, hipStream_t s) {
  if (T == 0) return 0;
  KVCM_REQUIRE(T > 0 && size > 0 && groups > 0 && col0 >= 0 && x && w, "rms_groups: bad sizes");
  KVCM_REQUIRE(ld >= col0 + size * groups, "rms_groups: the groups do not fit the rows");
  KVCM_REQUIRE(!out || ldo >= size * groups, "rms_groups: the groups do not fit the output's rows");
  const long long items = static_cast<long long>(T) * groups;
  const long long blocks = (items + 3) / 4;
  KVCM_REQUIRE(blocks < (1ll << 31), "rms_groups: too many rows");
  if (!out || out_dtype == kF32)
    rms_groups_kernel<float><<<static_cast<unsigned>(blocks), 256, 0, s>>>(x, ld, col0, size, groups, w, eps, static_cast<float*>(out), ldo, items);
  else if (out_dtype == kBF16)
    rms_groups_kernel<bf16_t><<<static_cast<unsigned>(blocks), 256, 0, s>>>(x, ld, col0, size, groups, w, eps, static_cast<bf16_t*>(out), ldo, items);
  else KVCM_REQUIRE(false, "rms_groups: unknown output dtype %d", out_dtype);
  return launch_status("rms_groups");
}

}  // extern "C"
