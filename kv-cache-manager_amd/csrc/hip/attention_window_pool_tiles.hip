// The attention over a window and pooled blocks (attention_window_pool.hip) for runs of consecutive
// positions, on the matrix cores: a workgroup of four waves takes 64 consecutive rows of one run and one
// query head, walks the keys those rows can see 64 at a time (first the pooled blocks from block 0, then the
// tokens in chunks that start at absolute multiples of 64), stages each chunk's keys and values once in LDS
// as bfloat16 and multiplies with v_mfma_f32_16x16x32_bf16: S = Q K^T (a wave: 16 rows x 64 keys), the
// mask and a running-maximum softmax in 32-bit on the accumulators, P rounded to bfloat16 and handed over
// through LDS as the next product's first operand, O += P V.  Which keys a row sees is decided per score
// (window, causality, blocks wholly before the window), so a chunk that some rows of the tile do not see
// costs them nothing but zeros; a row's chunks and their order depend on its own position only.  The first
// keep_first tokens of a sequence may stay visible beyond the window (chunks of their own, from token 0), and the
// scores may be capped, score <- c tanh(score / c), and a bias that grows with the distance may be taken off them,
// score <- score - slope_h * (i - j) with a slope per query head (tokens only: not beside pooled blocks); the output may be
// multiplied element by element with sigmoid(gate) before it is stored.
// bfloat16 storage only; sizes d and dv in multiples of 8, pages whose size is a multiple of 8 and divides 64.
#include <cfloat>

#include "common.h"
#include "kvcm_hip.h"

namespace kvcm {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4;

constexpr int kTileRows = 64, kChunk = 64, kVtPitch = kChunk + 8;
constexpr float kMasked = -1.0e30f;

__device__ __forceinline__ uint32_t pack_bf16(float a, float b) {
  return uint32_t(float_to_bf16_bits(a)) | (uint32_t(float_to_bf16_bits(b)) << 16);
}

// DP: key size padded to a multiple of 32; DVT: tiles of 16 value columns
template <int DP, int DVT>
__global__ void __launch_bounds__(256)
    attention_window_pool_tiles_kernel(const uint16_t* __restrict__ q, int ldq, uint16_t* __restrict__ out, int ldo,
                                       const uint16_t* __restrict__ kcache, const uint16_t* __restrict__ vcache,
                                       const float* __restrict__ pk, const float* __restrict__ pv,
                                       const int* __restrict__ tables, int table_stride, const int* __restrict__ run_start,
                                       const int* __restrict__ seq_start, const float* __restrict__ head_scale,
                                       const float* __restrict__ dist_slope, const float* __restrict__ gate, int ldg, int tiles_per_seq,
                                       int nh, int nkv, int d, int dv, int B, float scale, int window, int P, int E,
                                       int keep_first, float softcap) {
  constexpr int KP = DP + 8, KS = DP / 32, DVP = DVT * 16;
  __shared__ __attribute__((aligned(16))) uint16_t Ks[kChunk][KP];
  __shared__ __attribute__((aligned(16))) uint16_t Vt[DVP][kVtPitch];
  __shared__ __attribute__((aligned(16))) uint16_t Ps[4][16][kVtPitch];
  const int s = blockIdx.x / tiles_per_seq, tile = blockIdx.x % tiles_per_seq, head = blockIdx.y;
  const int run0 = run_start[s], run_len = run_start[s + 1] - run0;
  if (tile * kTileRows >= run_len) return;
  const int r0 = run0 + tile * kTileRows;
  const int nrows = run_len - tile * kTileRows < kTileRows ? run_len - tile * kTileRows : kTileRows;
  const int p0 = seq_start[s] + tile * kTileRows, p_last = p0 + nrows - 1;
  const int kvh = head / (nh / nkv);
  const int* table = tables + size_t(s) * table_stride;
  const int tid = threadIdx.x, wave = tid / kWave, lane = tid % kWave;
  const int col = lane % 16, quad = lane / 16;
  // scores are kept in units of log 2 (the factor rides along with the scale), so that the exponentials are the
  // hardware's exp2: a bfloat16 probability keeps 8 bits of it
  // (with a cap c on the scores, score <- c tanh(score / c): f then brings the product to score / c and the capped
  // value is scaled to units of log 2 afterwards)
  constexpr float kLog2e = 1.44269504088896341f;
  const float f = (head_scale ? scale * head_scale[head] : scale) * (softcap > 0.f ? 1.0f / softcap : kLog2e);
  const float cap2 = softcap * kLog2e;
  const float slope2 = dist_slope ? dist_slope[head] * kLog2e : 0.f;      // the bias in units of log 2, like the scores

  // this wave's 16 query rows as first operands (row = lane % 16, k = 8 * (lane / 16) .. + 8 of every 32)
  bf16x8 qf[KS];
  {
    const int row = wave * 16 + col;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int k = ks * 32 + quad * 8;
      uint4 v = {0u, 0u, 0u, 0u};
      if (row < nrows && k < d) v = *reinterpret_cast<const uint4*>(q + size_t(r0 + row) * ldq + size_t(head) * d + k);
      qf[ks] = __builtin_bit_cast(bf16x8, v);
    }
  }
  // the four rows whose scores this lane holds: 4 * quad + i of the wave's 16
  int pos[4], seen_blocks[4];
  float m[4], lsum[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int row = wave * 16 + quad * 4 + i;
    pos[i] = row < nrows ? p0 + row : -1;
    seen_blocks[i] = (P > 0 && window > 0 && pos[i] + 1 > window) ? (pos[i] + 1 - window) / P : 0;
    m[i] = kMasked;
    lsum[i] = 0.f;
  }
  f32x4 o[DVT];
#pragma unroll
  for (int vt = 0; vt < DVT; ++vt) o[vt] = f32x4{0.f, 0.f, 0.f, 0.f};

  const int blocks = (P > 0 && window > 0 && p_last + 1 > window) ? (p_last + 1 - window) / P : 0;      // of the tile's last row
  const int t_lo = (window > 0 && p0 + 1 > window) ? p0 + 1 - window : 0;
  const int block_chunks = (blocks + kChunk - 1) / kChunk;
  // the sequence's first tokens that stay visible beyond the window: those before the tile's first seen token get chunks
  // of their own, from token 0, between the blocks and the window (every row of the tile sees all of them)
  const int kept = keep_first < t_lo ? keep_first : t_lo;
  const int head_chunks = block_chunks + (kept + kChunk - 1) / kChunk;
  const int first_token_chunk = t_lo / kChunk, last_token_chunk = p_last / kChunk;
  const int chunks = head_chunks + (last_token_chunk - first_token_chunk + 1);
  auto chunk_start = [&](int c) {
    return c < block_chunks ? c * kChunk : c < head_chunks ? (c - block_chunks) * kChunk : (first_token_chunk + (c - head_chunks)) * kChunk;
  };

  // A chunk of tokens on its way from the pages to LDS, held in registers meanwhile: the next chunk is requested
  // before the current one is multiplied.  Loads are unconditional, from places clamped into the sequence, and
  // masked afterwards (a branch around a load would make each wait for the one before).
  constexpr int KQ = (kChunk * (DP / 8) + 255) / 256, VQ = (DVP * (kChunk / 8) + 255) / 256;
  uint4 kreg[KQ], vreg[VQ];
  // a chunk of tokens c0 .. c0 + 63 of which the stretch [lo, hi] may be read (the window up to the newest token, or the
  // kept first tokens)
  auto request_tokens = [&](int c0, int lo, int hi) {
#pragma unroll
    for (int qq = 0; qq < KQ; ++qq) {
      const int e = tid + qq * 256;
      const int key = (e / (DP / 8)) % kChunk, k = (e % (DP / 8)) * 8, t = c0 + key;
      // (pages that the window has passed may have been given back: nothing outside the stretch is read)
      const int tl = t < lo ? lo : t;
      const int tc = tl <= hi ? tl : hi, kc = k < d ? k : d - 8;
      const uint4 v = *reinterpret_cast<const uint4*>(kcache + ((size_t(table[tc / B]) * nkv + kvh) * B + tc % B) * d + kc);
      kreg[qq] = (t <= hi && k < d) ? v : uint4{0u, 0u, 0u, 0u};
    }
#pragma unroll
    for (int qq = 0; qq < VQ; ++qq) {
      const int e = tid + qq * 256;
      const int cc = (e / (kChunk / 8)) % DVP, piece = e % (kChunk / 8), t = c0 + piece * 8;
      const int tl = t < (lo / 8) * 8 ? (lo / 8) * 8 : t;
      const int tc = tl <= hi ? tl : (hi / 8) * 8, ccl = cc < dv ? cc : dv - 1;
      uint4 v = *reinterpret_cast<const uint4*>(vcache + ((size_t(table[tc / B]) * nkv + kvh) * dv + ccl) * B + tc % B);
      v = keep_first_bf16(v, hi + 1 - tc < 8 ? hi + 1 - tc : 8);      // beyond the stretch: whatever was there (counted from the piece that was read)
      vreg[qq] = cc < dv ? v : uint4{0u, 0u, 0u, 0u};
    }
  };
  auto request_chunk = [&](int c) {      // c >= block_chunks
    if (c < head_chunks) request_tokens(chunk_start(c), 0, kept - 1);
    else request_tokens(chunk_start(c), t_lo, p_last);
  };
  auto stage_tokens = [&]() {
#pragma unroll
    for (int qq = 0; qq < KQ; ++qq) {
      const int e = tid + qq * 256;
      if (e < kChunk * (DP / 8)) *reinterpret_cast<uint4*>(&Ks[e / (DP / 8)][(e % (DP / 8)) * 8]) = kreg[qq];
    }
#pragma unroll
    for (int qq = 0; qq < VQ; ++qq) {
      const int e = tid + qq * 256;
      if (e < DVP * (kChunk / 8)) *reinterpret_cast<uint4*>(&Vt[e / (kChunk / 8)][(e % (kChunk / 8)) * 8]) = vreg[qq];
    }
  };

  for (int c = 0; c < chunks; ++c) {
    const bool pooled = c < block_chunks, early = !pooled && c < head_chunks;
    const int c0 = chunk_start(c);
    if (!pooled && c == block_chunks) request_chunk(c);      // the first chunk of tokens: nobody asked for it yet
    __syncthreads();      // the chunk before is done with Ks, Vt and Ps
    if (pooled) {
      for (int e = tid; e < kChunk * (DP / 8); e += 256) {
        const int key = e / (DP / 8), k = (e % (DP / 8)) * 8, b = c0 + key;
        uint4 v = {0u, 0u, 0u, 0u};
        if (b < blocks && k < d) {
          const int pgi = (b * P + P - 1) / B;
          const float* src = pk + ((size_t(table[pgi]) * nkv + kvh) * E + (b - (pgi * B) / P)) * d + k;
          const float4 x = *reinterpret_cast<const float4*>(src), y = *reinterpret_cast<const float4*>(src + 4);
          v = uint4{pack_bf16(x.x, x.y), pack_bf16(x.z, x.w), pack_bf16(y.x, y.y), pack_bf16(y.z, y.w)};
        }
        *reinterpret_cast<uint4*>(&Ks[key][k]) = v;
      }
      for (int e = tid; e < kChunk * DVP; e += 256) {
        const int key = e / DVP, cc = e % DVP, b = c0 + key;
        float x = 0.f;
        if (b < blocks && cc < dv) {
          const int pgi = (b * P + P - 1) / B;
          x = pv[((size_t(table[pgi]) * nkv + kvh) * E + (b - (pgi * B) / P)) * dv + cc];
        }
        Vt[cc][key] = float_to_bf16_bits(x);
      }
    } else {
      stage_tokens();
    }
    __syncthreads();
    if (!pooled && c + 1 < chunks) request_chunk(c + 1);      // on its way while this chunk is multiplied

    // scores of 16 rows x 64 keys: four column tiles
    f32x4 sc[4];
#pragma unroll
    for (int ct = 0; ct < 4; ++ct) {
      sc[ct] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const bf16x8 kf = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(&Ks[ct * 16 + col][ks * 32 + quad * 8]));
        sc[ct] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qf[ks], kf, sc[ct], 0, 0, 0);
      }
    }
    float alpha[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      float mx = kMasked;
      bool vis[4];
#pragma unroll
      for (int ct = 0; ct < 4; ++ct) {
        const int key = c0 + ct * 16 + col;
        vis[ct] = pooled ? key < seen_blocks[i]
                  : early ? (key < kept && pos[i] >= 0)
                          : (key >= t_lo && key <= pos[i] && (window == 0 || key > pos[i] - window || key < keep_first));
        float sv = sc[ct][i] * f;
        if (softcap > 0.f) sv = cap2 * tanhf(sv);
        if (dist_slope) sv = fmaf(-slope2, float(pos[i] - key), sv);
        sv = vis[ct] ? sv : kMasked;
        sc[ct][i] = sv;
        mx = fmaxf(mx, sv);
      }
      mx = group_max<16>(mx);
      const float m_new = fmaxf(m[i], mx);
      alpha[i] = __builtin_amdgcn_exp2f(m[i] - m_new);
      float add = 0.f;
#pragma unroll
      for (int ct = 0; ct < 4; ++ct) {
        const float p = vis[ct] ? __builtin_amdgcn_exp2f(sc[ct][i] - m_new) : 0.f;
        const uint16_t pb = float_to_bf16_bits(p);
        Ps[wave][quad * 4 + i][ct * 16 + col] = pb;
        add += bf16_bits_to_float(pb);      // the sum of what is multiplied, so that the weights add up to one
      }
      lsum[i] = lsum[i] * alpha[i] + add;
      m[i] = m_new;
    }
#pragma unroll
    for (int vt = 0; vt < DVT; ++vt)
#pragma unroll
      for (int i = 0; i < 4; ++i) o[vt][i] *= alpha[i];
    __syncthreads();      // Ps written by other lanes of the wave
#pragma unroll
    for (int ks = 0; ks < kChunk / 32; ++ks) {
      const bf16x8 pf = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(&Ps[wave][col][ks * 32 + quad * 8]));
#pragma unroll
      for (int vt = 0; vt < DVT; ++vt) {
        const bf16x8 vf = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(&Vt[vt * 16 + col][ks * 32 + quad * 8]));
        o[vt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pf, vf, o[vt], 0, 0, 0);
      }
    }
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const float l = group_sum<16>(lsum[i]);
    const int row = wave * 16 + quad * 4 + i;
    if (row < nrows) {
      const float inv = 1.0f / l;
#pragma unroll
      for (int vt = 0; vt < DVT; ++vt) {
        const int cc = vt * 16 + col;
        if (cc < dv) {
          float res = o[vt][i] * inv;
          if (gate) res *= 1.0f / (1.0f + expf(-gate[size_t(r0 + row) * ldg + size_t(head) * dv + cc]));      // a gate per element
          out[size_t(r0 + row) * ldo + size_t(head) * dv + cc] = float_to_bf16_bits(res);
        }
      }
    }
  }
}

template <int DP>
int launch_tiles(int dvt, dim3 grid, hipStream_t s, const uint16_t* q, int ldq, uint16_t* out, int ldo, const uint16_t* kc,
                 const uint16_t* vc, const float* pk, const float* pv, const int* tables, int table_stride, const int* run_start,
                 const int* seq_start, const float* head_scale, const float* dist_slope, const float* gate, int ldg, int tiles_per_seq,
                 int nh, int nkv, int d, int dv, int B, float scale, int window, int P, int E, int keep_first, float softcap) {
#define KVCM_TILES(DVT)                                                                                                     \
  attention_window_pool_tiles_kernel<DP, DVT><<<grid, 256, 0, s>>>(q, ldq, out, ldo, kc, vc, pk, pv, tables, table_stride,   \
                                                                   run_start, seq_start, head_scale, dist_slope, gate, ldg, tiles_per_seq, \
                                                                   nh, nkv, d, dv, B, scale, window, P, E, keep_first, softcap)
  if (dvt <= 2) KVCM_TILES(2);
  else if (dvt <= 4) KVCM_TILES(4);
  else if (dvt <= 8) KVCM_TILES(8);
  else KVCM_TILES(16);
#undef KVCM_TILES
  return launch_status("attention_window_pool_tiles");
}

}  // namespace kvcm

using namespace kvcm;

extern "C" {

int kvcm_attention_window_pool_tiles_supported(int d, int dv, int B) {
  return d > 0 && d % 8 == 0 && d <= 128 && dv > 0 && dv % 8 == 0 && dv <= 256 && B % 8 == 0 && B > 0 && kChunk % B == 0;
}

// q, out, pages: bfloat16; pooled entries: 32-bit.  S sequences with runs of up to max_run rows.
int kvcm_attention_window_pool_tiles(const void* q, int ldq, void* out, int ldo, const void* kcache, const void* vcache,
                                     const float* pk, const float* pv, const int* tables, int table_stride,
                                     const int* run_start, const int* seq_start, const float* head_scale, const float* dist_slope,
                                     const float* gate, int ldg, int S, int max_run, int nh, int nkv, int d, int dv, int B, float scale, int window, int P,
                                     int E, int keep_first, float softcap, hipStream_t s) {
  if (S == 0 || max_run == 0) return 0;
  KVCM_REQUIRE(S > 0 && max_run > 0 && nh > 0 && nkv > 0 && nh % nkv == 0, "attention_window_pool_tiles: bad sizes");
  KVCM_REQUIRE(kvcm_attention_window_pool_tiles_supported(d, dv, B),
               "attention_window_pool_tiles: key size %d, value size %d, pages of %d are not supported", d, dv, B);
  KVCM_REQUIRE(ldq >= nh * d && ldo >= nh * dv && ldq % 8 == 0 && reinterpret_cast<uintptr_t>(q) % 16 == 0,
               "attention_window_pool_tiles: q rows must be 16-byte aligned and long enough");
  KVCM_REQUIRE(window >= 0 && P >= 0 && (P == 0 || (pk && pv && E == (B + P - 1) / P)),
               "attention_window_pool_tiles: pooled blocks need their entries");
  KVCM_REQUIRE(P == 0 || d % 8 == 0, "attention_window_pool_tiles: pooled keys are read eight at a time");
  KVCM_REQUIRE(keep_first >= 0 && softcap >= 0.f, "attention_window_pool_tiles: negative count of kept tokens or score cap");
  KVCM_REQUIRE(!dist_slope || P == 0, "attention_window_pool_tiles: a distance bias beside pooled blocks is not supported");
  KVCM_REQUIRE(!gate || ldg >= nh * dv, "attention_window_pool_tiles: the gate's rows are too short");
  const int tiles_per_seq = (max_run + kTileRows - 1) / kTileRows;
  KVCM_REQUIRE(static_cast<long long>(S) * tiles_per_seq < (1ll << 31) && nh <= 65535, "attention_window_pool_tiles: too many rows");
  const dim3 grid(S * tiles_per_seq, nh);
  const int dvt = (dv + 15) / 16;
  const uint16_t* qq = static_cast<const uint16_t*>(q);
  uint16_t* oo = static_cast<uint16_t*>(out);
  const uint16_t* kc = static_cast<const uint16_t*>(kcache);
  const uint16_t* vc = static_cast<const uint16_t*>(vcache);
  if (d <= 32)
    return launch_tiles<32>(dvt, grid, s, qq, ldq, oo, ldo, kc, vc, pk, pv, tables, table_stride, run_start, seq_start, head_scale,
                            dist_slope, gate, ldg, tiles_per_seq, nh, nkv, d, dv, B, scale, window, P, E, keep_first, softcap);
  if (d <= 64)
    return launch_tiles<64>(dvt, grid, s, qq, ldq, oo, ldo, kc, vc, pk, pv, tables, table_stride, run_start, seq_start, head_scale,
                            dist_slope, gate, ldg, tiles_per_seq, nh, nkv, d, dv, B, scale, window, P, E, keep_first, softcap);
  return launch_tiles<128>(dvt, grid, s, qq, ldq, oo, ldo, kc, vc, pk, pv, tables, table_stride, run_start, seq_start, head_scale,
                           dist_slope, gate, ldg, tiles_per_seq, nh, nkv, d, dv, B, scale, window, P, E, keep_first, softcap);
}

}  // extern "C"
