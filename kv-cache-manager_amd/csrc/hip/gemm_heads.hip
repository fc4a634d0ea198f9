// One small product per head in one launch: Y[m, h*N + n] = sum_k X[m, h*K + k] * W[h, n, k], for a stack of matrices
// W [heads, N, K] that each act on their own stretch of the rows (a latent attention's values: every head's output over
// the cached latent, size K, is taken to the head's value size N by that head's matrix).  The result may be multiplied
// element by element with sigmoid(gate[m, h*N + n]) (32-bit gate logits) before it is stored.
//
// bfloat16: v_mfma_f32_16x16x32_bf16 on tiles of 64 columns and 64 rows (four waves, a 32 x 32 quadrant each) or, for
// steps of up to 16 rows, 16 rows (a wave per 16 columns); K advanced 32 at a time through LDS; rows, columns and k
// outside the matrices are staged as zeros.  float32: plain FMA, every output element one chain over k = 0 .. K-1 in
// ascending order, whatever else the launch holds.
#include "common.h"
#include "kvcm_hip.h"

namespace kvcm {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4;

constexpr int kHeadsBN = 64, kHeadsBK = 32, kHeadsPitch = kHeadsBK + 8;

// eight consecutive values of a row from k on, zeros beyond K or outside the rows
__device__ __forceinline__ uint4 heads_piece(const uint16_t* row_base, bool row_ok, int k, int K, bool wide) {
  uint4 v = {0u, 0u, 0u, 0u};
  if (!row_ok || k >= K) return v;
  if (wide && k + 8 <= K) return *reinterpret_cast<const uint4*>(row_base + k);
  uint32_t half[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) half[i] = (k + i < K) ? row_base[k + i] : 0u;
  return uint4{half[0] | (half[1] << 16), half[2] | (half[3] << 16), half[4] | (half[5] << 16), half[6] | (half[7] << 16)};
}

template <class TO, int BM>      // BM 64 or 16 rows a workgroup
__global__ void __launch_bounds__(256)
    gemm_heads_bf16_kernel(const uint16_t* __restrict__ X, int ldx, const uint16_t* __restrict__ W, TO* __restrict__ Y, int ldy,
                           const float* __restrict__ gate, int ldg, int M, int N, int K, int wide) {
  constexpr int TI = BM == 64 ? 2 : 1, TJ = BM == 64 ? 2 : 1;
  __shared__ __attribute__((aligned(16))) uint16_t Xs[BM][kHeadsPitch];
  __shared__ __attribute__((aligned(16))) uint16_t Ws[kHeadsBN][kHeadsPitch];
  const int tid = threadIdx.x, wave = tid / kWave, lane = tid % kWave;
  const int head = blockIdx.z, m0 = blockIdx.y * BM, n0 = blockIdx.x * kHeadsBN;
  const int row_off = BM == 64 ? (wave / 2) * 32 : 0, col_off = BM == 64 ? (wave % 2) * 32 : wave * 16;
  const uint16_t* xh = X + size_t(head) * K;
  const uint16_t* wh = W + size_t(head) * N * K;
  const int piece_row = tid / 4, piece_k = (tid % 4) * 8;
  const int frag_row = lane % 16, frag_k = (lane / 16) * 8;
  f32x4 acc[TI][TJ];
#pragma unroll
  for (int i = 0; i < TI; ++i)
#pragma unroll
    for (int j = 0; j < TJ; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
  for (int k0 = 0; k0 < K; k0 += kHeadsBK) {
    const uint4 wv = heads_piece(wh + size_t(n0 + piece_row) * K, n0 + piece_row < N, k0 + piece_k, K, wide);
    uint4 xv = {0u, 0u, 0u, 0u};
    if (piece_row < BM) xv = heads_piece(xh + size_t(m0 + piece_row) * ldx, m0 + piece_row < M, k0 + piece_k, K, wide);
    __syncthreads();      // the step before is done with the tiles
    *reinterpret_cast<uint4*>(&Ws[piece_row][piece_k]) = wv;
    if (piece_row < BM) *reinterpret_cast<uint4*>(&Xs[piece_row][piece_k]) = xv;
    __syncthreads();
    bf16x8 a[TI], b[TJ];
#pragma unroll
    for (int i = 0; i < TI; ++i) a[i] = *reinterpret_cast<const bf16x8*>(&Xs[row_off + i * 16 + frag_row][frag_k]);
#pragma unroll
    for (int j = 0; j < TJ; ++j) b[j] = *reinterpret_cast<const bf16x8*>(&Ws[col_off + j * 16 + frag_row][frag_k]);
#pragma unroll
    for (int i = 0; i < TI; ++i)
#pragma unroll
      for (int j = 0; j < TJ; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[i], b[j], acc[i][j], 0, 0, 0);
  }
  // a lane holds column lane % 16 and rows 4 * (lane / 16) .. + 4 of each 16 x 16 tile
#pragma unroll
  for (int i = 0; i < TI; ++i)
#pragma unroll
    for (int j = 0; j < TJ; ++j) {
      const int n = n0 + col_off + j * 16 + lane % 16;
      if (n >= N) continue;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int m = m0 + row_off + i * 16 + (lane / 16) * 4 + e;
        if (m >= M) continue;
        float v = acc[i][j][e];
        if (gate) v *= 1.0f / (1.0f + expf(-gate[size_t(m) * ldg + size_t(head) * N + n]));
        store_f(Y + size_t(m) * ldy + size_t(head) * N + n, v);
      }
    }
}

// a thread per output element: 64 columns x 4 rows a workgroup
__global__ void __launch_bounds__(256)
    gemm_heads_f32_kernel(const float* __restrict__ X, int ldx, const float* __restrict__ W, float* __restrict__ Y, int ldy,
                          const float* __restrict__ gate, int ldg, int M, int N, int K) {
  const int head = blockIdx.z;
  const int n = blockIdx.x * 64 + threadIdx.x % 64, m = blockIdx.y * 4 + threadIdx.x / 64;
  if (n >= N || m >= M) return;
  const float* x = X + size_t(m) * ldx + size_t(head) * K;
  const float* w = W + (size_t(head) * N + n) * K;
  float acc = 0.f;
  for (int k = 0; k < K; ++k) acc = fmaf(x[k], w[k], acc);
  if (gate) acc *= 1.0f / (1.0f + expf(-gate[size_t(m) * ldg + size_t(head) * N + n]));
  Y[size_t(m) * ldy + size_t(head) * N + n] = acc;
}

}  // namespace kvcm

using namespace kvcm;

// X [M, >= heads*K] and W [heads, N, K] contiguous in in_dtype; Y [M, >= heads*N] in out_dtype (float32 operands give a
// float32 result); gate: 32-bit rows [M, >= heads*N] or null.
extern "C" int kvcm_gemm_heads(const void* X, int in_dtype, int ldx, const void* W, void* Y, int out_dtype, int ldy,
                               const float* gate, int ldg, int M, int heads, int N, int K, hipStream_t s) {
  if (M == 0) return 0;
  KVCM_REQUIRE(M > 0 && heads > 0 && N > 0 && K > 0 && X && W && Y, "gemm_heads: bad sizes M=%d heads=%d N=%d K=%d", M, heads, N, K);
  KVCM_REQUIRE(ldx >= heads * K && ldy >= heads * N && (!gate || ldg >= heads * N), "gemm_heads: row strides too small");
  KVCM_REQUIRE(heads <= 65535, "gemm_heads: too many heads for one launch (%d)", heads);
  if (in_dtype == kF32) {
    KVCM_REQUIRE(out_dtype == kF32, "gemm_heads: float32 operands give a float32 result");
    const dim3 grid((N + 63) / 64, (M + 3) / 4, heads);
    KVCM_REQUIRE(grid.y <= 65535, "gemm_heads: too many rows for one launch (%d)", M);
    gemm_heads_f32_kernel<<<grid, 256, 0, s>>>(static_cast<const float*>(X), ldx, static_cast<const float*>(W), static_cast<float*>(Y),
                                               ldy, gate, ldg, M, N, K);
    return launch_status("gemm_heads");
  }
  KVCM_REQUIRE(in_dtype == kBF16 && (out_dtype == kBF16 || out_dtype == kF32), "gemm_heads: unknown dtypes %d -> %d", in_dtype, out_dtype);
  const int wide = K % 8 == 0 && ldx % 8 == 0 && reinterpret_cast<uintptr_t>(X) % 16 == 0 && reinterpret_cast<uintptr_t>(W) % 16 == 0;
  const uint16_t* x = static_cast<const uint16_t*>(X);
  const uint16_t* w = static_cast<const uint16_t*>(W);
  const int bm = M <= 16 ? 16 : 64;
  const dim3 grid((N + kHeadsBN - 1) / kHeadsBN, (M + bm - 1) / bm, heads);
  KVCM_REQUIRE(grid.y <= 65535, "gemm_heads: too many rows for one launch (%d)", M);
#define KVCM_HEADS(TO, BM) \
  gemm_heads_bf16_kernel<TO, BM><<<grid, 256, 0, s>>>(x, ldx, w, static_cast<TO*>(Y), ldy, gate, ldg, M, N, K, wide)
  if (bm == 16) { if (out_dtype == kBF16) KVCM_HEADS(bf16_t, 16); else KVCM_HEADS(float, 16); }
  else { if (out_dtype == kBF16) KVCM_HEADS(bf16_t, 64); else KVCM_HEADS(float, 64); }
#undef KVCM_HEADS
  return launch_status("gemm_heads");
}
