// The routed feed-forward for steps with many rows (bfloat16): the (row, slot) pairs are grouped by their expert and
// every expert's group is multiplied with that expert's matrices in tiles on the matrix cores, so that an expert's
// weights are read once per tile of 128 pairs and not once per pair.
//
//   moe_group      pairs p = row * top + slot, grouped by chosen[p]: order[] lists the pairs expert by expert, tiles[]
//                  lists (expert, first place in order, pairs) for every stretch of up to 128 pairs of one expert, with
//                  the number of tiles in front.  One workgroup; places inside a group are handed out by an atomic
//                  counter in LDS, so the order inside a group may differ from run to run, which changes no result: a
//                  pair's row of a tile is computed from that row alone.
//   moe_grouped    UP:   act[place, :] = square(relu(W_up[e] h[row of the pair]))           (bfloat16, in grouped order)
//                  GATED UP: act[place, :] = silu(W_gate[e] h) * (W_up[e] h); the two matrices of an expert are stored as
//                        one of 2F rows, interleaved sixteen at a time (gate 0..15, up 0..15, gate 16..31, ...), so that a
//                        lane's neighbouring 16 x 16 tiles hold the gate and the up value of one column
//                  DOWN: y[pair, :]   = weight[pair] * W_down[e] act[place, :]               (32-bit, by pair)
//                  Tile 128 pairs x 128 columns per workgroup of four waves (64 x 64 each: 4 x 4 matrix instructions of
//                  16 x 16 x 32), K advanced 64 at a time through LDS, the next 64 on their way in registers meanwhile.
//   moe_combine    out[row, :] = (add[row, :] +) sum over the row's slots, in slot order, of y[row * top + slot, :]
#include "common.h"
#include "kvcm_hip.h"

namespace kvcm {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4;

constexpr int kGM = 128, kGN = 128, kGK = 64, kGPitch = kGK + 8;      // a row pitch of 144 bytes: 16 rows meet no bank twice

__global__ void __launch_bounds__(1024)
    moe_group_kernel(const int* __restrict__ chosen, int n, int E, int* __restrict__ order, int* __restrict__ tiles, int max_tiles) {
  extern __shared__ int sh[];      // count / cursor [E], base [E]
  int* cnt = sh;
  int* base = sh + E;
  for (int e = threadIdx.x; e < E; e += blockDim.x) cnt[e] = 0;
  __syncthreads();
  for (int p = threadIdx.x; p < n; p += blockDim.x) {
    const int e = chosen[p];
    if (e >= 0 && e < E) atomicAdd(&cnt[e], 1);
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int at = 0, nt = 0;
    for (int e = 0; e < E; ++e) {
      base[e] = at;
      for (int r = 0; r < cnt[e] && nt < max_tiles; r += kGM) {
        tiles[1 + 3 * nt] = e;
        tiles[2 + 3 * nt] = at + r;
        tiles[3 + 3 * nt] = cnt[e] - r < kGM ? cnt[e] - r : kGM;
        ++nt;
      }
      at += cnt[e];
      cnt[e] = 0;
    }
    tiles[0] = nt;
  }
  __syncthreads();
  for (int p = threadIdx.x; p < n; p += blockDim.x) {
    const int e = chosen[p];
    if (e >= 0 && e < E) order[base[e] + atomicAdd(&cnt[e], 1)] = p;
  }
}

enum : int { kDown = 0, kUp = 1, kUpGated = 2 };

// N: rows of an expert's matrix (2F for the gated form); the output has N columns (F for the gated form)
template <int MODE>
__global__ void __launch_bounds__(256)
    moe_grouped_kernel(const uint16_t* __restrict__ A, int lda, const uint16_t* __restrict__ W, const int* __restrict__ order,
                       const int* __restrict__ tiles, int top, void* __restrict__ out, const float* __restrict__ weight, int N,
                       int K, int col_blocks) {
  __shared__ __attribute__((aligned(16))) uint16_t staged[2][kGM][kGPitch];      // both operands; the down form's results pass through it too
  uint16_t (*As)[kGPitch] = staged[0];
  uint16_t (*Bs)[kGPitch] = staged[1];
  __shared__ int pair_of[kGM];
  // The chip hands consecutive workgroups to its eight XCDs in turn, each with an L2 of its own.  Workgroup L goes to
  // XCD L % 8; it takes a column block that is congruent to its XCD and walks the tiles in order, so that the tiles of
  // one expert (neighbours in the list) meet the same blocks of that expert's matrix in the same L2.
  const int col_slots = (col_blocks + 7) / 8;
  const int xcd = blockIdx.x % 8, turn = blockIdx.x / 8;
  const int tile = turn / col_slots, col_block = (turn % col_slots) * 8 + xcd;
  if (col_block >= col_blocks || tile >= tiles[0]) return;
  const int e = tiles[1 + 3 * tile], p0 = tiles[2 + 3 * tile], rows = tiles[3 + 3 * tile];
  const int n0 = col_block * kGN;
  const int tid = threadIdx.x, wave = tid / kWave, lane = tid % kWave;
  if (tid < kGM) pair_of[tid] = order[p0 + (tid < rows ? tid : 0)];
  __syncthreads();
  // the four 16-byte pieces a thread stages of each operand: rows tid / 8 + 32 q, k offset (tid % 8) * 8
  const int kk = (tid % 8) * 8;
  const uint16_t* arow[4];
  const uint16_t* brow[4];
  bool aok[4], bok[4];
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const int r = tid / 8 + 32 * q;
    aok[q] = r < rows;
    const long long src = MODE != kDown ? pair_of[r] / top : p0 + (aok[q] ? r : 0);
    arow[q] = A + src * lda;
    const int c = n0 + r;
    bok[q] = c < N;
    brow[q] = W + (static_cast<long long>(e) * N + (bok[q] ? c : N - 1)) * K;
  }
  uint4 areg[4], breg[4];
  auto request = [&](int k0) {      // unconditional loads from clamped places, masked afterwards
    const bool kin = k0 + kk < K;      // K is a multiple of 8: a piece lies inside or outside
    const int off = kin ? k0 + kk : 0;      // (a piece outside is read from the row's start: nothing beyond a row is touched)
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const uint4 a = *reinterpret_cast<const uint4*>(arow[q] + off);
      const uint4 b = *reinterpret_cast<const uint4*>(brow[q] + off);
      areg[q] = (kin && aok[q]) ? a : uint4{0u, 0u, 0u, 0u};
      breg[q] = (kin && bok[q]) ? b : uint4{0u, 0u, 0u, 0u};
    }
  };
  f32x4 acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
  const int wm = wave / 2, wn = wave % 2;
  const int frow = lane % 16, fk = (lane / 16) * 8;
  request(0);
  for (int k0 = 0; k0 < K; k0 += kGK) {
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      *reinterpret_cast<uint4*>(&As[tid / 8 + 32 * q][kk]) = areg[q];
      *reinterpret_cast<uint4*>(&Bs[tid / 8 + 32 * q][kk]) = breg[q];
    }
    __syncthreads();
    if (k0 + kGK < K) request(k0 + kGK);
#pragma unroll
    for (int ks = 0; ks < kGK / 32; ++ks) {
      bf16x8 a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = *reinterpret_cast<const bf16x8*>(&As[wm * 64 + i * 16 + frow][ks * 32 + fk]);
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j] = *reinterpret_cast<const bf16x8*>(&Bs[wn * 64 + j * 16 + frow][ks * 32 + fk]);
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[i], b[j], acc[i][j], 0, 0, 0);
    }
    __syncthreads();
  }
  // accumulator layout: a lane holds column lane % 16 and rows 4 * (lane / 16) + r of each 16 x 16 tile
  if constexpr (MODE == kDown) {
    // 32-bit results by pair: stored from the accumulators a wave's store would write 64-byte pieces of four rows.  Each
    // wave passes its 64 x 64 results through LDS instead, 32 rows at a time, and writes whole 256-byte stretches of
    // a row, 16 bytes a lane.  The operands' space is free by now (the loop ended with a barrier).
    constexpr int kPitch = 68;      // floats; 4 waves x 32 rows x 68 fit the operands' 9,216 floats
    static_assert(4 * 32 * kPitch * sizeof(float) <= sizeof(staged), "the results of half a tile must fit the operands' space");
    float* mine = reinterpret_cast<float*>(&staged[0][0][0]) + wave * 32 * kPitch;
#pragma unroll
    for (int half = 0; half < 2; ++half) {
#pragma unroll
      for (int ii = 0; ii < 2; ++ii)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
          for (int r = 0; r < 4; ++r)
            mine[(ii * 16 + (lane / 16) * 4 + r) * kPitch + j * 16 + lane % 16] = acc[half * 2 + ii][j][r];
      __syncthreads();
#pragma unroll
      for (int it = 0; it < 8; ++it) {
        const int idx = it * kWave + lane, rl = idx / 16, c4 = (idx % 16) * 4;
        const int m = wm * 64 + half * 32 + rl;
        const int c = n0 + wn * 64 + c4;
        if (m >= rows || c >= N) continue;
        const int pair = pair_of[m];
        const float g = weight[pair];
        const float4 v = *reinterpret_cast<const float4*>(mine + rl * kPitch + c4);
        float* dst = static_cast<float*>(out) + static_cast<long long>(pair) * N + c;
        if (c + 3 < N && N % 4 == 0) {
          *reinterpret_cast<float4*>(dst) = float4{g * v.x, g * v.y, g * v.z, g * v.w};
        } else {
          const float e4[4] = {v.x, v.y, v.z, v.w};
          for (int q = 0; q < 4 && c + q < N; ++q) dst[q] = g * e4[q];
        }
      }
      __syncthreads();
    }
    return;
  }
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int m = wm * 64 + i * 16 + (lane / 16) * 4 + r;
      if (m >= rows) continue;
      const int pair = pair_of[m];
      const float g = MODE != kDown ? 1.f : weight[pair];
      if constexpr (MODE == kUpGated) {
#pragma unroll
        for (int j = 0; j < 4; j += 2) {      // tile j: sixteen gate columns, tile j + 1: the same sixteen up columns
          const int c = n0 + wn * 64 + j * 16 + lane % 16;
          if (c >= N) continue;
          const int col = (n0 + wn * 64 + j * 16) / 2 + lane % 16;
          static_cast<uint16_t*>(out)[static_cast<long long>(p0 + m) * (N / 2) + col] =
              float_to_bf16_bits(silu<bf16_t>(acc[i][j][r]) * acc[i][j + 1][r]);
        }
      } else {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int c = n0 + wn * 64 + j * 16 + lane % 16;
          if (c >= N) continue;
          const float v = acc[i][j][r];
          if (MODE == kUp) {
            const float z = fmaxf(v, 0.f);
            static_cast<uint16_t*>(out)[static_cast<long long>(p0 + m) * N + c] = float_to_bf16_bits(z * z);
          } else {
            static_cast<float*>(out)[static_cast<long long>(pair) * N + c] = g * v;
          }
        }
      }
    }
}

__global__ void __launch_bounds__(256)
    moe_combine_kernel(const float* __restrict__ y, const float* __restrict__ add, float* __restrict__ out, long long n, int H,
                       int top) {
  for (long long idx = static_cast<long long>(blockIdx.x) * 256 + threadIdx.x; idx < n; idx += static_cast<long long>(gridDim.x) * 256) {
    const long long row = idx / H;
    const int c = static_cast<int>(idx % H);
    float acc = 0.f;
    for (int s = 0; s < top; ++s) acc += y[(row * top + s) * H + c];
    out[idx] = add ? add[idx] + acc : acc;
  }
}

}  // namespace kvcm

using namespace kvcm;

extern "C" {

// Does the grouped form take these sizes?  (bfloat16; rows of 16-byte pieces)
int kvcm_moe_grouped_supported(int K, int F, int E) { return K > 0 && F > 0 && K % 8 == 0 && F % 8 == 0 && E > 0 && E <= 4096; }

// Tiles a step of n pairs over E experts can have at most.
int kvcm_moe_grouped_max_tiles(int n, int E) { return (n + kGM - 1) / kGM + E; }

// h [T, K] bfloat16; w_up [E, F, K], w_down [E, H, F] bfloat16; chosen [T * top], weight [T * top]; work memory:
// order [T * top] and tiles [3 * max_tiles + 1] (int32), act [T * top, F] (bfloat16), y [T * top, H] (32-bit); out [T, H] 32-bit.
// gated: w_up [E, 2F, K] (gate and up rows interleaved sixteen at a time), act = silu(gate) * up.  add [T, H] 32-bit or
// null: out = add + the experts' sum.
int kvcm_moe_grouped(const void* h, int ldh, const void* w_up, const void* w_down, const int* chosen, const float* weight,
                     int* order, int* tiles, void* act, float* y, const float* add, float* out, int T, int K, int F, int H,
                     int top, int E, int gated, hipStream_t s) {
  if (T == 0) return 0;
  KVCM_REQUIRE(T > 0 && top > 0 && H > 0 && ldh >= K, "moe_grouped: bad sizes");
  KVCM_REQUIRE(kvcm_moe_grouped_supported(K, F, E), "moe_grouped: sizes K=%d F=%d experts=%d are not supported", K, F, E);
  KVCM_REQUIRE(static_cast<long long>(T) * top < (1ll << 30), "moe_grouped: too many rows");
  KVCM_REQUIRE(ldh % 8 == 0 && reinterpret_cast<uintptr_t>(h) % 16 == 0 && reinterpret_cast<uintptr_t>(w_up) % 16 == 0 &&
                   reinterpret_cast<uintptr_t>(w_down) % 16 == 0 && reinterpret_cast<uintptr_t>(act) % 16 == 0,
               "moe_grouped: operands must be 16-byte aligned");
  const int n = T * top, max_tiles = kvcm_moe_grouped_max_tiles(n, E);
  KVCM_REQUIRE(!gated || F % 16 == 0, "moe_grouped: gated experts of %d columns are not supported (a multiple of 16)", F);
  const int up_rows = gated ? 2 * F : F;
  const int up_blocks = (up_rows + kGN - 1) / kGN, down_blocks = (H + kGN - 1) / kGN;
  const long long up_grid = static_cast<long long>(max_tiles) * ((up_blocks + 7) / 8) * 8;
  const long long down_grid = static_cast<long long>(max_tiles) * ((down_blocks + 7) / 8) * 8;
  KVCM_REQUIRE(up_grid < (1ll << 31) && down_grid < (1ll << 31), "moe_grouped: too many tiles");
  moe_group_kernel<<<1, 1024, 2 * E * sizeof(int), s>>>(chosen, n, E, order, tiles, max_tiles);
  if (gated)
    moe_grouped_kernel<kUpGated><<<static_cast<unsigned>(up_grid), 256, 0, s>>>(
        static_cast<const uint16_t*>(h), ldh, static_cast<const uint16_t*>(w_up), order, tiles, top, act, nullptr, up_rows, K, up_blocks);
  else
    moe_grouped_kernel<kUp><<<static_cast<unsigned>(up_grid), 256, 0, s>>>(
        static_cast<const uint16_t*>(h), ldh, static_cast<const uint16_t*>(w_up), order, tiles, top, act, nullptr, F, K, up_blocks);
  moe_grouped_kernel<kDown><<<static_cast<unsigned>(down_grid), 256, 0, s>>>(
      static_cast<const uint16_t*>(act), F, static_cast<const uint16_t*>(w_down), order, tiles, top, y, weight, H, F, down_blocks);
  const long long total = static_cast<long long>(T) * H;
  const long long blocks = (total + 255) / 256;
  moe_combine_kernel<<<static_cast<unsigned>(blocks > 16384 ? 16384 : blocks), 256, 0, s>>>(y, add, out, total, H, top);
  return launch_status("moe_grouped");
}

}  // extern "C"
