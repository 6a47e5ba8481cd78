// Score-driven block masks ("SSTA" style): every query block attends to a diagonal band of key blocks, to the first key
// blocks of the sequence, and to the top-k key blocks ranked by <mean of the query block's rows, mean of the key block's
// rows>.  Three HBM-bound kernels: block means of Q and K, then scores + top-k + union into the bool block mask the
// compaction kernel consumes, and the (un)permutation of a video latent grid into contiguous tiles.
#include "fba_kernels.h"

namespace fba {

namespace {

constexpr int kD = 128;

__device__ __forceinline__ float bf16_lo(uint32_t u) { return __uint_as_float(u << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t u) { return __uint_as_float(u & 0xffff0000u); }

// out[g, :] = mean over rows [g*block, (g+1)*block) of x, x [n_blocks*block, 128] bf16, out fp32.
// One work-group per block: 16 lanes cover one 256-byte row, the 16 row groups of the work-group stride through the
// block, then add up through LDS in a fixed order (the result does not depend on scheduling).
__global__ __attribute__((amdgpu_flat_work_group_size(256, 256))) void block_mean_kernel(
    const __bf16* __restrict__ x, float* __restrict__ out, int block, float inv_block) {
  __shared__ float red[16][kD + 4];
  const int tid = threadIdx.x, c = tid & 15, r0 = tid >> 4;
  const uint4* src = reinterpret_cast<const uint4*>(x + (size_t)blockIdx.x * block * kD);
  float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  int r = r0;
  for (; r + 48 < block; r += 64) {
    uint4 u[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) u[i] = src[(size_t)(r + 16 * i) * 16 + c];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      acc[0] += bf16_lo(u[i].x); acc[1] += bf16_hi(u[i].x); acc[2] += bf16_lo(u[i].y); acc[3] += bf16_hi(u[i].y);
      acc[4] += bf16_lo(u[i].z); acc[5] += bf16_hi(u[i].z); acc[6] += bf16_lo(u[i].w); acc[7] += bf16_hi(u[i].w);
    }
  }
  for (; r < block; r += 16) {
    const uint4 u = src[(size_t)r * 16 + c];
    acc[0] += bf16_lo(u.x); acc[1] += bf16_hi(u.x); acc[2] += bf16_lo(u.y); acc[3] += bf16_hi(u.y);
    acc[4] += bf16_lo(u.z); acc[5] += bf16_hi(u.z); acc[6] += bf16_lo(u.w); acc[7] += bf16_hi(u.w);
  }
#pragma unroll
  for (int e = 0; e < 8; ++e) red[r0][c * 8 + e] = acc[e];
  __syncthreads();
  if (tid < kD) {
    float s = 0.f;
#pragma unroll
    for (int g = 0; g < 16; ++g) s += red[g][tid];
    out[(size_t)blockIdx.x * kD + tid] = s * inv_block;
  }
}

constexpr int kQPerWave = 2;
constexpr int kQPerGroup = 8;      // query blocks per work-group (4 waves x 2)
constexpr int kChunk = 64;         // key blocks per LDS chunk: one per lane
constexpr int kRowStride = kD + 1; // floats; lane-per-row reads hit 64 different banks
constexpr int kChunksSmall = 16;   // nK <= 1024: 32 score registers per lane
constexpr int kChunksLarge = 64;   // nK <= 4096: 128 score registers per lane

// mask[bh, i, j] = (j among the topk largest <q_mean[bh,i], k_mean[kv(bh),j]>, ties to the lower j)
//                  || |j - (i*q_block)/k_block| <= band || j < sink || base[i, j]   (base: optional [nQ, nK] mask).
// A wave ranks two query blocks; lane l holds the scores of key blocks l, l+64, ... (kMaxChunks of them) in registers.
template <int kMaxChunks>
__global__ __attribute__((amdgpu_flat_work_group_size(256, 256))) void ssta_mask_kernel(
    const float* __restrict__ q_mean, const float* __restrict__ k_mean, const uint8_t* __restrict__ base,
    uint8_t* __restrict__ mask, int Hq, int Hkv, int nQ, int nK, int q_block, int k_block, int topk, int band, int sink) {
  __shared__ float k_lds[kChunk * kRowStride];
  __shared__ float q_lds[kQPerGroup * kD];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int64_t bh = blockIdx.y;
  const int64_t kv_seq = (bh / Hq) * Hkv + (bh % Hq) / (Hq / Hkv);
  const int i0 = blockIdx.x * kQPerGroup;
  for (int idx = tid; idx < kQPerGroup * kD; idx += 256) {
    const int i = i0 + (idx >> 7);
    q_lds[idx] = i < nQ ? q_mean[((size_t)(bh * nQ + i) << 7) + (idx & 127)] : 0.f;
  }
  const float ninf = -__builtin_inff();
  float sc[kQPerWave][kMaxChunks];
  const int n_chunks = (nK + kChunk - 1) / kChunk;
#pragma unroll
  for (int t = 0; t < kMaxChunks; ++t) {
    sc[0][t] = ninf;
    sc[1][t] = ninf;
    if (t < n_chunks) {  // uniform over the work-group
      __syncthreads();
      for (int idx = tid; idx < kChunk * kD; idx += 256) {
        const int r = idx >> 7, j = t * kChunk + r;
        k_lds[r * kRowStride + (idx & 127)] = j < nK ? k_mean[((size_t)(kv_seq * nK + j) << 7) + (idx & 127)] : 0.f;
      }
      __syncthreads();
      float s0 = 0.f, s1 = 0.f;
      const float* kr = k_lds + lane * kRowStride;
      const float* q0 = q_lds + (wave * kQPerWave) * kD;
#pragma unroll 8
      for (int d = 0; d < kD; ++d) {
        const float kv = kr[d];
        s0 += q0[d] * kv;
        s1 += q0[kD + d] * kv;
      }
      if (t * kChunk + lane < nK) {
        sc[0][t] = s0;
        sc[1][t] = s1;
      }
    }
  }
#pragma unroll
  for (int qq = 0; qq < kQPerWave; ++qq) {
    const int i = i0 + wave * kQPerWave + qq;
    if (i >= nQ) break;  // uniform over the wave
    uint64_t sel = 0;
    for (int round = 0; round < topk; ++round) {
      float best = ninf;
      int bt = -1;
#pragma unroll
      for (int t = 0; t < kMaxChunks; ++t)
        if (!((sel >> t) & 1u) && sc[qq][t] > best) {
          best = sc[qq][t];
          bt = t;
        }
      int j = bt < 0 ? 0x7fffffff : bt * kChunk + lane;
#pragma unroll
      for (int off = 32; off >= 1; off >>= 1) {
        const float ob = __shfl_xor(best, off, 64);
        const int oj = __shfl_xor(j, off, 64);
        if (ob > best || (ob == best && oj < j)) {
          best = ob;
          j = oj;
        }
      }
      if (j == 0x7fffffff) break;  // nothing left to pick: every lane sees the same j
      if ((j & 63) == lane) sel |= 1ull << (j >> 6);
    }
    const int diag = (int)(((int64_t)i * q_block) / k_block);
    uint8_t* row = mask + (size_t)(bh * nQ + i) * nK;
#pragma unroll
    for (int t = 0; t < kMaxChunks; ++t) {
      const int j = t * kChunk + lane;
      if (j < nK) {
        const int dist = j > diag ? j - diag : diag - j;
        const uint32_t keep = base ? (base[(size_t)i * nK + j] != 0) : 0u;
        row[j] = (uint8_t)((uint32_t)((sel >> t) & 1u) | (dist <= band) | (j < sink) | keep);
      }
    }
  }
}

// Gather of 256-byte token rows between the raster order of a (T, H, W) grid and tile order, in which the tT x tH x tW
// tokens of one tile are consecutive (tiles in raster order of the tile grid, tokens in raster order inside the tile).
// to_tiles = 1: out[tile order] = x[raster order]; 0: the inverse.  16 lanes move one row.
__global__ __attribute__((amdgpu_flat_work_group_size(256, 256))) void tile_permute_kernel(
    const uint4* __restrict__ x, uint4* __restrict__ out, int64_t n_seq, int T, int H, int W, int tT, int tH, int tW,
    int to_tiles) {
  const int64_t S = (int64_t)T * H * W;
  const int64_t row = (int64_t)blockIdx.x * 16 + (threadIdx.x >> 4);
  if (row >= n_seq * S) return;
  const int c = threadIdx.x & 15;
  const int64_t seq = row / S;
  int64_t p = row - seq * S;  // position in tile order
  const int tile_sz = tT * tH * tW, nH = H / tH, nW = W / tW;
  const int tile = (int)(p / tile_sz), in = (int)(p - (int64_t)tile * tile_sz);
  const int bt = tile / (nH * nW), bh = (tile / nW) % nH, bw = tile % nW;
  const int it = in / (tH * tW), ih = (in / tW) % tH, iw = in % tW;
  const int64_t raster = ((int64_t)(bt * tT + it) * H + (bh * tH + ih)) * W + (bw * tW + iw);
  const int64_t a = (seq * S + raster) * 16 + c, b = row * 16 + c;
  if (to_tiles) out[b] = x[a];
  else out[a] = x[b];
}

}  // namespace

hipError_t launch_block_mean(const __bf16* x, float* out, int64_t n_blocks, int block, hipStream_t stream) {
  if (n_blocks <= 0) return hipSuccess;
  if (n_blocks > 0x7fffffffLL) return hipErrorInvalidValue;
  hipLaunchKernelGGL(block_mean_kernel, dim3((unsigned)n_blocks), dim3(256), 0, stream, x, out, block, 1.0f / (float)block);
  return hipGetLastError();
}

hipError_t launch_ssta_mask(const float* q_mean, const float* k_mean, const uint8_t* base, uint8_t* mask, int64_t BH, int Hq, int Hkv, int nQ,
                            int nK, int q_block, int k_block, int topk, int band, int sink, hipStream_t stream) {
  if (BH <= 0 || BH > 65535 || nK > kChunk * kChunksLarge) return hipErrorInvalidValue;
  void (*fn)(const float*, const float*, const uint8_t*, uint8_t*, int, int, int, int, int, int, int, int, int) =
      nK <= kChunk * kChunksSmall ? &ssta_mask_kernel<kChunksSmall> : &ssta_mask_kernel<kChunksLarge>;
  hipLaunchKernelGGL(fn, dim3((unsigned)((nQ + kQPerGroup - 1) / kQPerGroup), (unsigned)BH), dim3(256), 0,
                     stream, q_mean, k_mean, base, mask, Hq, Hkv, nQ, nK, q_block, k_block, topk, band, sink);
  return hipGetLastError();
}

hipError_t launch_tile_permute(const void* x, void* out, int64_t n_seq, int T, int H, int W, int tT, int tH, int tW,
                               int to_tiles, hipStream_t stream) {
  const int64_t rows = n_seq * T * H * W;
  const int64_t blocks = (rows + 15) / 16;
  if (blocks <= 0) return hipSuccess;
  if (blocks > 0x7fffffffLL) return hipErrorInvalidValue;
  hipLaunchKernelGGL(tile_permute_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, (const uint4*)x, (uint4*)out, n_seq,
                     T, H, W, tT, tH, tW, to_tiles);
  return hipGetLastError();
}

}  // namespace fba
