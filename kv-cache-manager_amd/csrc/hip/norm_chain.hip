// RMS norms whose arithmetic is 32-bit from end to end, chained along a row in one launch.
//
// A layer that norms a sublayer's output before adding it to the residual stream, and norms the
// stream again for the next sublayer, does per row
//     m = c * (n(a) * wa + n(b) * wb)      (only where two branches are combined; else m = a)
//     x += n(m) * w_post                   (only where a sublayer's output is added)
//     out = n(x) * w_pre                   (only where somebody reads the normed stream; without w_pre: out = x, for
//                                           sublayers that read the stream as it is)
// with n(v) = v / sqrt(mean(v^2) + eps).  Every stage needs the whole row of the stage before, and
// nothing else: one workgroup per row runs all of them, so a layer boundary costs one launch instead
// of up to four, and the branches' outputs are read once.  Sums of squares are added in a tree whose
// shape depends on the row length only; a row's result does not depend on the other rows.
#include "common.h"
#include "kvcm_hip.h"

namespace kvcm {

constexpr int kChainThreads = 256;

template <class TO>
__global__ void __launch_bounds__(kChainThreads)
    rmsnorm_chain_kernel(float* __restrict__ x, const float* __restrict__ a, int a_splits, const float* __restrict__ b,
                         int b_splits, size_t split_stride, const float* __restrict__ wa, const float* __restrict__ wb,
                         float combine,
                         const float* __restrict__ w_post, const int* __restrict__ rows,
                         const float* __restrict__ w_pre, TO* __restrict__ out, int H, float eps, int write_back) {
  __shared__ float scratch[kChainThreads / kWave + 1];
  const int r = blockIdx.x;
  const int src = rows ? rows[r] : r;
  float* xr = x + size_t(src) * H;
  const float* ar = a ? a + size_t(src) * H : nullptr;
  const float* br = b ? b + size_t(src) * H : nullptr;
  const float inv_h = 1.0f / float(H);
  // a branch is a finished tensor (splits 1) or the slices of a product that was split along K and not added up yet
  // ([splits][T][H] floats): then the slices are added here, in their order
  auto part = [&](const float* p, int splits, int i) {
    float v = p[i];
    for (int sl = 1; sl < splits; ++sl) v += p[size_t(sl) * split_stride + i];
    return v;
  };

  float inv_a = 0.f, inv_b = 0.f;
  if (br) {
    float sa = 0.f, sb = 0.f;
    for (int i = threadIdx.x; i < H; i += kChainThreads) {
      const float u = part(ar, a_splits, i), v = part(br, b_splits, i);
      sa = fmaf(u, u, sa);
      sb = fmaf(v, v, sb);
    }
    sa = block_sum<kChainThreads>(sa, scratch);
    sb = block_sum<kChainThreads>(sb, scratch);
    inv_a = 1.0f / sqrtf(sa * inv_h + eps);
    inv_b = 1.0f / sqrtf(sb * inv_h + eps);
  }
  auto branch = [&](int i) {
    return br ? combine * (part(ar, a_splits, i) * inv_a * wa[i] + part(br, b_splits, i) * inv_b * wb[i]) : part(ar, a_splits, i);
  };
  float inv_m = 0.f;
  if (ar) {
    float sm = 0.f;
    for (int i = threadIdx.x; i < H; i += kChainThreads) {
      const float m = branch(i);
      sm = fmaf(m, m, sm);
    }
    sm = block_sum<kChainThreads>(sm, scratch);
    inv_m = 1.0f / sqrtf(sm * inv_h + eps);
  }
  auto stream = [&](int i) { return ar ? xr[i] + branch(i) * inv_m * w_post[i] : xr[i]; };
  if (!out) {
    for (int i = threadIdx.x; i < H; i += kChainThreads) xr[i] = stream(i);
    return;
  }
  float inv_x = 1.f;
  if (w_pre) {
    float sx = 0.f;
    for (int i = threadIdx.x; i < H; i += kChainThreads) {
      const float v = stream(i);
      sx = fmaf(v, v, sx);
    }
    sx = block_sum<kChainThreads>(sx, scratch);
    inv_x = 1.0f / sqrtf(sx * inv_h + eps);
  }
  TO* o = out + size_t(r) * H;
  for (int i = threadIdx.x; i < H; i += kChainThreads) {
    const float v = stream(i);
    if (ar && write_back) xr[i] = v;      // each element is read and written by one thread only
    store_f(o + i, w_pre ? v * inv_x * w_pre[i] : v);
  }
}

// The same chain for rows whose length is a multiple of 4 and at most 1024 * G (G groups of four values a thread):
// the branches' and the stream's values of a row are read once, 16 bytes a load, and stay in registers through all
// stages, so the row costs one trip to memory instead of one per stage.  A branch that is still the slices of a split
// product is added up as it is read, slice after slice.  Which of the two kernels runs depends on the row length only,
// never on the batch.
template <class TO, int G>
__global__ void __launch_bounds__(kChainThreads)
    rmsnorm_chain_rows_kernel(float* __restrict__ x, const float* __restrict__ a, int a_splits, const float* __restrict__ b,
                              int b_splits, size_t split_stride,
                              const float* __restrict__ wa, const float* __restrict__ wb, float combine,
                              const float* __restrict__ w_post, const int* __restrict__ rows,
                              const float* __restrict__ w_pre, TO* __restrict__ out, int H, float eps, int write_back) {
  __shared__ float scratch[kChainThreads / kWave + 1];
  const int r = blockIdx.x;
  const int src = rows ? rows[r] : r;
  float* xr = x + size_t(src) * H;
  const float inv_h = 1.0f / float(H);
  float xv[G][4], av[G][4], bv[G][4];
  bool in[G];
#pragma unroll
  for (int g = 0; g < G; ++g) {
    const int i = (g * kChainThreads + threadIdx.x) * 4;
    in[g] = i < H;
    const int ic = in[g] ? i : 0;
    const float4 vx = *reinterpret_cast<const float4*>(xr + ic);
    xv[g][0] = vx.x; xv[g][1] = vx.y; xv[g][2] = vx.z; xv[g][3] = vx.w;
    if (a) {
      const float* p = a + size_t(src) * H + ic;
      float4 va = *reinterpret_cast<const float4*>(p);
#pragma unroll 4
      for (int sl = 1; sl < a_splits; ++sl) {
        const float4 t = *reinterpret_cast<const float4*>(p + size_t(sl) * split_stride);
        va.x += t.x; va.y += t.y; va.z += t.z; va.w += t.w;
      }
      av[g][0] = va.x; av[g][1] = va.y; av[g][2] = va.z; av[g][3] = va.w;
    }
    if (b) {
      const float* p = b + size_t(src) * H + ic;
      float4 vb = *reinterpret_cast<const float4*>(p);
#pragma unroll 4
      for (int sl = 1; sl < b_splits; ++sl) {
        const float4 t = *reinterpret_cast<const float4*>(p + size_t(sl) * split_stride);
        vb.x += t.x; vb.y += t.y; vb.z += t.z; vb.w += t.w;
      }
      bv[g][0] = vb.x; bv[g][1] = vb.y; bv[g][2] = vb.z; bv[g][3] = vb.w;
    }
  }
  if (b) {
    float sa = 0.f, sb = 0.f;
#pragma unroll
    for (int g = 0; g < G; ++g)
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (in[g]) {
          sa = fmaf(av[g][e], av[g][e], sa);
          sb = fmaf(bv[g][e], bv[g][e], sb);
        }
    sa = block_sum<kChainThreads>(sa, scratch);
    sb = block_sum<kChainThreads>(sb, scratch);
    const float inv_a = 1.0f / sqrtf(sa * inv_h + eps), inv_b = 1.0f / sqrtf(sb * inv_h + eps);
#pragma unroll
    for (int g = 0; g < G; ++g) {
      const int i = in[g] ? (g * kChainThreads + threadIdx.x) * 4 : 0;
#pragma unroll
      for (int e = 0; e < 4; ++e) av[g][e] = combine * (av[g][e] * inv_a * wa[i + e] + bv[g][e] * inv_b * wb[i + e]);
    }
  }
  if (a) {
    float sm = 0.f;
#pragma unroll
    for (int g = 0; g < G; ++g)
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (in[g]) sm = fmaf(av[g][e], av[g][e], sm);
    sm = block_sum<kChainThreads>(sm, scratch);
    const float inv_m = 1.0f / sqrtf(sm * inv_h + eps);
#pragma unroll
    for (int g = 0; g < G; ++g) {
      const int i = in[g] ? (g * kChainThreads + threadIdx.x) * 4 : 0;
#pragma unroll
      for (int e = 0; e < 4; ++e) xv[g][e] += av[g][e] * inv_m * w_post[i + e];
      if (in[g] && write_back) *reinterpret_cast<float4*>(xr + i) = float4{xv[g][0], xv[g][1], xv[g][2], xv[g][3]};
    }
  }
  if (!out) return;
  float inv_x = 1.f;
  if (w_pre) {
    float sx = 0.f;
#pragma unroll
    for (int g = 0; g < G; ++g)
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (in[g]) sx = fmaf(xv[g][e], xv[g][e], sx);
    sx = block_sum<kChainThreads>(sx, scratch);
    inv_x = 1.0f / sqrtf(sx * inv_h + eps);
  }
  TO* o = out + size_t(r) * H;
#pragma unroll
  for (int g = 0; g < G; ++g) {
    if (!in[g]) continue;
    const int i = (g * kChainThreads + threadIdx.x) * 4;
#pragma unroll
    for (int e = 0; e < 4; ++e) store_f(o + i + e, w_pre ? xv[g][e] * inv_x * w_pre[i + e] : xv[g][e]);
  }
}

// out[r, h, :] = n(o[r, h, :]) * w[h, :] * sigmoid(g[r, h, :]): the norm of every head on its own, a
// plain weight over all heads, and a gate.  One wave per (row, head).
template <class TO>
__global__ void __launch_bounds__(256)
    head_norm_gate_kernel(const float* __restrict__ o, int ldo, const float* __restrict__ g, int ldg,
                          const float* __restrict__ w, TO* __restrict__ out, int ldout, long long items, int heads,
                          int d, float eps) {
  const long long item = static_cast<long long>(blockIdx.x) * (256 / kWave) + threadIdx.x / kWave;
  if (item >= items) return;
  const int lane = threadIdx.x % kWave;
  const int row = static_cast<int>(item / heads), head = static_cast<int>(item % heads);
  const float* orow = o + size_t(row) * ldo + size_t(head) * d;
  const float* grow = g + size_t(row) * ldg + size_t(head) * d;
  float ss = 0.f;
  for (int i = lane; i < d; i += kWave) ss = fmaf(orow[i], orow[i], ss);
  ss = wave_sum(ss);
  const float inv = 1.0f / sqrtf(ss / float(d) + eps);
  TO* dst = out + size_t(row) * ldout + size_t(head) * d;
  for (int i = lane; i < d; i += kWave) {
    const float gate = 1.0f / (1.0f + expf(-grow[i]));
    store_f(dst + i, orow[i] * inv * w[size_t(head) * d + i] * gate);
  }
}

}  // namespace kvcm

using namespace kvcm;

extern "C" {

// a, b: the branches [T, H] (b null: one branch, taken as it is; a null: nothing is added), each finished (splits 1) or
// the un-added slices of a split product, [splits][T][H] with split_stride = T * H floats between slices.  rows: source
// rows of the R outputs (null: row r).  out null: only the addition.  The stream is updated in place
// unless rows are gathered.
int kvcm_rmsnorm_chain(float* x, const float* a, int a_splits, const float* b, int b_splits, long long split_stride,
                       const float* wa, const float* wb, float combine, const float* w_post, const int* rows,
                       const float* w_pre, void* out, int out_dtype, int R, int H, float eps, hipStream_t s) {
  if (R == 0) return 0;
  KVCM_REQUIRE(R > 0 && H > 0 && x != nullptr, "rmsnorm_chain: bad sizes R=%d H=%d", R, H);
  KVCM_REQUIRE(!b || (a && wa && wb), "rmsnorm_chain: two branches need both outputs and both weights");
  KVCM_REQUIRE(!a || w_post, "rmsnorm_chain: an added output needs the weight of its norm");
  KVCM_REQUIRE(out || (a && !rows), "rmsnorm_chain: nothing to do");
  KVCM_REQUIRE(a_splits >= 1 && b_splits >= 1 && split_stride >= 0, "rmsnorm_chain: a branch has at least one slice");
  const int wb_flag = rows ? 0 : 1;
  KVCM_REQUIRE(!out || out_dtype == kF32 || out_dtype == kBF16, "rmsnorm_chain: unknown output dtype %d", out_dtype);
  const bool f32 = !out || out_dtype == kF32;
  auto aligned = [](const void* p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; };
  if (H % 4 == 0 && H <= 8192 && aligned(x) && aligned(a) && aligned(b)) {      // slices lie split_stride = T * H floats apart
#define KVCM_CHAIN_ROWS(TO, G)                                                                                     \
  rmsnorm_chain_rows_kernel<TO, G><<<R, kChainThreads, 0, s>>>(x, a, a_splits, b, b_splits,                         \
                                                               static_cast<size_t>(split_stride), wa, wb, combine, \
                                                               w_post, rows, w_pre, static_cast<TO*>(out), H, eps, wb_flag)
    if (H <= 2048) { if (f32) KVCM_CHAIN_ROWS(float, 2); else KVCM_CHAIN_ROWS(bf16_t, 2); }
    else if (H <= 4096) { if (f32) KVCM_CHAIN_ROWS(float, 4); else KVCM_CHAIN_ROWS(bf16_t, 4); }
    else { if (f32) KVCM_CHAIN_ROWS(float, 8); else KVCM_CHAIN_ROWS(bf16_t, 8); }
#undef KVCM_CHAIN_ROWS
    return launch_status("rmsnorm_chain");
  }
  if (f32)
    rmsnorm_chain_kernel<float><<<R, kChainThreads, 0, s>>>(x, a, a_splits, b, b_splits, static_cast<size_t>(split_stride), wa, wb,
                                                             combine, w_post, rows, w_pre, static_cast<float*>(out), H, eps, wb_flag);
  else
    rmsnorm_chain_kernel<bf16_t><<<R, kChainThreads, 0, s>>>(x, a, a_splits, b, b_splits, static_cast<size_t>(split_stride), wa, wb,
                                                              combine, w_post, rows, w_pre, static_cast<bf16_t*>(out), H, eps, wb_flag);
  return launch_status("rmsnorm_chain");
}

int kvcm_head_norm_gate(const float* o, int ldo, const float* g, int ldg, const float* w, void* out, int out_dtype,
                        int ldout, int T, int heads, int d, float eps, hipStream_t s) {
  if (T == 0) return 0;
  KVCM_REQUIRE(T > 0 && heads > 0 && d > 0, "head_norm_gate: bad sizes T=%d heads=%d d=%d", T, heads, d);
  KVCM_REQUIRE(ldo >= heads * d && ldg >= heads * d && ldout >= heads * d, "head_norm_gate: row strides too small");
  const long long items = static_cast<long long>(T) * heads;
  const long long blocks = (items + 3) / 4;
  KVCM_REQUIRE(blocks < (1ll << 31), "head_norm_gate: too many rows");
  if (out_dtype == kF32)
    head_norm_gate_kernel<float><<<static_cast<unsigned>(blocks), 256, 0, s>>>(o, ldo, g, ldg, w, static_cast<float*>(out),
                                                                                ldout, items, heads, d, eps);
  else if (out_dtype == kBF16)
    head_norm_gate_kernel<bf16_t><<<static_cast<unsigned>(blocks), 256, 0, s>>>(o, ldo, g, ldg, w, static_cast<bf16_t*>(out),
                                                                                 ldout, items, heads, d, eps);
  else KVCM_REQUIRE(false, "head_norm_gate: unknown output dtype %d", out_dtype);
  return launch_status("head_norm_gate");
}

}  // extern "C"
