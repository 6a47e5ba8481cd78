// Mask compaction: bool block mask [mask_bh, nQ, nK] -> ascending active-index lists in both orientations.
//
// The reference never materialises such lists: every CTA rescans its mask row in the tile loop
// (flex_block_attn_h100.cu:134-135, :247-248) and the backward pass needs a transposed copy of the mask
// (flex_block_attn_interface.py:85-86; scan at flex_block_attn_h100.cu:672, :738).  Here one launch emits
//   q_cnt[m, i], q_idx[m, i, 0..q_cnt) = { j : mask[m, i, j] }   ascending, padded with -1 to nK entries
//   k_cnt[m, j], k_idx[m, j, 0..k_cnt) = { i : mask[m, i, j] }   ascending, padded with -1 to nQ entries
// One wave per output row: 64 mask bytes per step, ballot + prefix popcount gives each active lane its slot, so the
// output order is the index order and the result is independent of scheduling (bit-exact, no atomics).
#include "fba_common.h"
#include "fba_kernels.h"

namespace fba {

__global__ __attribute__((amdgpu_flat_work_group_size(256, 256))) void mask_compact_kernel(
    const uint8_t* __restrict__ mask, int64_t mask_bh, int nQ, int nK, int32_t* __restrict__ q_cnt,
    int32_t* __restrict__ q_idx, int32_t* __restrict__ k_cnt, int32_t* __restrict__ k_idx) {
  const int lane = threadIdx.x & 63;
  const int64_t w = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int64_t n_qrows = mask_bh * nQ, n_krows = mask_bh * nK;
  if (w >= n_qrows + n_krows) return;

  const bool row_pass = w < n_qrows;
  const int64_t r = row_pass ? w : w - n_qrows;
  const int len = row_pass ? nK : nQ;           // entries per output row
  const int64_t m = r / (row_pass ? nQ : nK);   // which (batch, head) mask
  const int self = (int)(r - m * (row_pass ? nQ : nK));
  const uint8_t* base = mask + m * (int64_t)nQ * nK;
  // element t of this output row's source: row pass mask[self, t]; column pass mask[t, self]
  const int64_t stride = row_pass ? 1 : nK;
  const uint8_t* src = base + (row_pass ? (int64_t)self * nK : (int64_t)self);
  int32_t* out = (row_pass ? q_idx : k_idx) + r * (int64_t)len;

  int cnt = 0;
  for (int t0 = 0; t0 < len; t0 += 64) {
    const int t = t0 + lane;
    const bool on = t < len && src[(int64_t)t * stride] != 0;
    const unsigned long long bal = __ballot(on);
    if (on) out[cnt + __popcll(bal & ((1ull << lane) - 1ull))] = t;
    cnt += __popcll(bal);
  }
  for (int t = cnt + lane; t < len; t += 64) out[t] = -1;
  if (lane == 0) (row_pass ? q_cnt : k_cnt)[r] = cnt;
}

hipError_t launch_mask_compact(const uint8_t* mask, int64_t mask_bh, int nQ, int nK, int32_t* q_cnt, int32_t* q_idx,
                               int32_t* k_cnt, int32_t* k_idx, hipStream_t stream) {
  const int64_t waves = mask_bh * ((int64_t)nQ + nK);
  const int64_t blocks = (waves + 3) / 4;
  if (blocks <= 0) return hipSuccess;
  if (blocks > 0x7fffffffLL) return hipErrorInvalidValue;
  hipLaunchKernelGGL(mask_compact_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, mask, mask_bh, nQ, nK, q_cnt,
                     q_idx, k_cnt, k_idx);
  return hipGetLastError();
}

// Tile lists for block sizes that do not align with the kernels' 128-row tiles (q_block or k_block not a multiple of
// 128).  The attention kernels then work on 128-row tiles that straddle mask blocks, so every list entry carries a
// predicate per 16-row group (query side) or per (wave, 16-row half-slab) pair (key side):
//   qt_ent[m, T, 0..qt_cnt) = (J << 8) | bits, ascending J: key block J is selected by at least one of the eight 16-row
//       groups of query tile T; bit g is mask[m, (128 T + 16 g) / q_block, J].                       (forward, dQ)
//   kt_ent[m, U, 0..kt_cnt) = (s << 8) | bits, ascending s: 32-row query slab s touches key tile U; bit 2w + f is
//       mask[m, (32 s + 16 f) / q_block, (128 U + 32 w) / k_block], w = wave (32 keys), f = half of the slab.  (dK/dV)
// One wave per output row, same ballot / prefix-popcount compaction as above; unused entries are -1.
__global__ __attribute__((amdgpu_flat_work_group_size(256, 256))) void tile_lists_kernel(
    const uint8_t* __restrict__ mask, int64_t mask_bh, int nQ, int nK, int q_block, int k_block, int n_qt, int n_kt,
    int n_qs, int32_t* __restrict__ qt_cnt, int32_t* __restrict__ qt_ent, int32_t* __restrict__ kt_cnt,
    int32_t* __restrict__ kt_ent) {
  const int lane = threadIdx.x & 63;
  const int64_t w = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int64_t n_qrows = mask_bh * n_qt, n_krows = mask_bh * n_kt;
  if (w >= n_qrows + n_krows) return;
  const bool q_pass = w < n_qrows;
  const int64_t r = q_pass ? w : w - n_qrows;
  const int per = q_pass ? n_qt : n_kt;
  const int64_t m = r / per;
  const int tile = (int)(r - m * per);
  const uint8_t* base = mask + m * (int64_t)nQ * nK;
  const int len = q_pass ? nK : n_qs;
  int32_t* out = (q_pass ? qt_ent : kt_ent) + r * (int64_t)len;

  int cnt = 0;
  for (int t0 = 0; t0 < len; t0 += 64) {
    const int t = t0 + lane;
    int bits = 0;
    if (t < len) {
      if (q_pass) {
#pragma unroll
        for (int g = 0; g < 8; ++g) bits |= (base[(int64_t)((128 * tile + 16 * g) / q_block) * nK + t] != 0) << g;
      } else {
#pragma unroll
        for (int wv = 0; wv < 4; ++wv)
#pragma unroll
          for (int f = 0; f < 2; ++f)
            bits |= (base[(int64_t)((32 * t + 16 * f) / q_block) * nK + (128 * tile + 32 * wv) / k_block] != 0) << (2 * wv + f);
      }
    }
    const bool on = bits != 0;
    const unsigned long long bal = __ballot(on);
    if (on) out[cnt + __popcll(bal & ((1ull << lane) - 1ull))] = (t << 8) | bits;
    cnt += __popcll(bal);
  }
  for (int t = cnt + lane; t < len; t += 64) out[t] = -1;
  if (lane == 0) (q_pass ? qt_cnt : kt_cnt)[r] = cnt;
}

hipError_t launch_tile_lists(const uint8_t* mask, int64_t mask_bh, int nQ, int nK, int q_block, int k_block, int n_qt,
                             int n_kt, int n_qs, int32_t* qt_cnt, int32_t* qt_ent, int32_t* kt_cnt, int32_t* kt_ent,
                             hipStream_t stream) {
  const int64_t waves = mask_bh * ((int64_t)n_qt + n_kt);
  const int64_t blocks = (waves + 3) / 4;
  if (blocks <= 0) return hipSuccess;
  if (blocks > 0x7fffffffLL) return hipErrorInvalidValue;
  hipLaunchKernelGGL(tile_lists_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, mask, mask_bh, nQ, nK, q_block, k_block,
                     n_qt, n_kt, n_qs, qt_cnt, qt_ent, kt_cnt, kt_ent);
  return hipGetLastError();
}

// Pair numbering for the dS hand-over of backward.  Every selected (query block, key block) pair gets a number in
// key-major list order: pair_base = exclusive prefix sum of k_cnt over the flattened (m, J) rows (the last entry is the
// total), pair (m, J, e) = pair_base[m, J] + e.  q_slot gives the same numbers in query-major list order, so that the
// query-major kernel finds what the key-major kernel stored: for J = q_idx[m, I, e], q_slot[m, I, e] = pair_base[m, J] +
// position of I in the ascending row k_idx[m, J, :] (binary search).  Integer work, independent of scheduling.
__global__ __attribute__((amdgpu_flat_work_group_size(1024, 1024))) void pair_base_kernel(const int32_t* __restrict__ k_cnt, int64_t n,
                                                                                          int32_t* __restrict__ pair_base) {
  __shared__ int32_t wave_sum[16];
  __shared__ int32_t carry_s;
  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  if (tid == 0) carry_s = 0;
  __syncthreads();
  for (int64_t t0 = 0; t0 < n; t0 += 1024) {
    const int64_t t = t0 + tid;
    const int32_t x = t < n ? k_cnt[t] : 0;
    int32_t incl = x;  // inclusive scan inside the wave
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      const int32_t y = __shfl_up(incl, d);
      if (lane >= d) incl += y;
    }
    if (lane == 63) wave_sum[wv] = incl;
    __syncthreads();
    int32_t before = carry_s;
    for (int w = 0; w < wv; ++w) before += wave_sum[w];
    if (t < n) pair_base[t] = before + incl - x;
    __syncthreads();
    if (tid == 1023) carry_s = before + incl;
    __syncthreads();
  }
  if (tid == 0) pair_base[n] = carry_s;
}

__global__ __attribute__((amdgpu_flat_work_group_size(256, 256))) void q_slot_kernel(
    const int32_t* __restrict__ q_cnt, const int32_t* __restrict__ q_idx, const int32_t* __restrict__ k_cnt,
    const int32_t* __restrict__ k_idx, const int32_t* __restrict__ pair_base, int64_t mask_bh, int nQ, int nK,
    int32_t* __restrict__ q_slot) {
  const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (t >= mask_bh * nQ * nK) return;
  const int e = (int)(t % nK);
  const int64_t row = t / nK;  // m * nQ + I
  const int I = (int)(row % nQ);
  const int64_t m = row / nQ;
  int32_t out = -1;
  if (e < q_cnt[row]) {
    const int J = q_idx[t];
    const int64_t krow = m * nK + J;
    const int32_t* list = k_idx + krow * nQ;
    int lo = 0, hi = k_cnt[krow] - 1;
    while (lo < hi) {  // I is in the list: the two orientations describe one mask
      const int mid = (lo + hi) >> 1;
      if (list[mid] < I) lo = mid + 1; else hi = mid;
    }
    out = pair_base[krow] + lo;
  }
  q_slot[t] = out;
}

hipError_t launch_pair_slots(const int32_t* q_cnt, const int32_t* q_idx, const int32_t* k_cnt, const int32_t* k_idx, int64_t mask_bh,
                             int nQ, int nK, int32_t* pair_base, int32_t* q_slot, hipStream_t stream) {
  const int64_t n = mask_bh * nK, entries = mask_bh * nQ * nK;
  if (n <= 0 || entries <= 0) return hipSuccess;
  const int64_t blocks = (entries + 255) / 256;
  if (blocks > 0x7fffffffLL) return hipErrorInvalidValue;
  hipLaunchKernelGGL(pair_base_kernel, dim3(1), dim3(1024), 0, stream, k_cnt, n, pair_base);
  hipLaunchKernelGGL(q_slot_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, q_cnt, q_idx, k_cnt, k_idx, pair_base, mask_bh, nQ, nK, q_slot);
  return hipGetLastError();
}

// Tile-pair numbering for the dS hand-over on tile lists.  The unit of the workspace is a (128-row query tile T, 128-key
// tile U) pair, listed when some 32-row slab of T appears in kt_ent[m, U, :]; pairs are numbered in key-major order:
// pair_base = exclusive prefix sum of the listed pairs per (m, U) row (last entry = total), pair (m, U, r) =
// pair_base[m, U] + r for the r-th distinct query tile of the ascending row.  kt_slot gives every kt_ent entry the number
// of its pair (what the key-major kernel needs, next to the entry); slot_table [m, T, U] gives the query-major kernel
// the same number by position (-1 where nothing is listed).  One wave per row; integer work, independent of scheduling.
__global__ __attribute__((amdgpu_flat_work_group_size(256, 256))) void tile_pair_count_kernel(
    const int32_t* __restrict__ kt_cnt, const int32_t* __restrict__ kt_ent, int64_t rows, int n_qs, int32_t* __restrict__ row_cnt) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const int cnt = kt_cnt[row];
  const int32_t* list = kt_ent + row * n_qs;
  int total = 0;
  for (int t0 = 0; t0 < cnt; t0 += 64) {
    const int e = t0 + lane;
    const bool first = e < cnt && (e == 0 || (list[e] >> 10) != (list[e - 1] >> 10));  // entry = slab << 8 | bits, tile = slab / 4
    total += __popcll(__ballot(first));
  }
  if (lane == 0) row_cnt[row] = total;
}

__global__ __attribute__((amdgpu_flat_work_group_size(256, 256))) void fill_i32_kernel(int32_t* __restrict__ out, int64_t n, int32_t value) {
  for (int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x; t < n; t += (int64_t)gridDim.x * 256) out[t] = value;
}

__global__ __attribute__((amdgpu_flat_work_group_size(256, 256))) void tile_slots_kernel(
    const int32_t* __restrict__ kt_cnt, const int32_t* __restrict__ kt_ent, const int32_t* __restrict__ pair_base, int64_t rows,
    int n_qt, int n_kt, int n_qs, int32_t* __restrict__ kt_slot, int32_t* __restrict__ slot_table) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const int64_t m = row / n_kt;
  const int U = (int)(row - m * n_kt);
  const int cnt = kt_cnt[row];
  const int32_t* list = kt_ent + row * n_qs;
  const int32_t base = pair_base[row];
  int seen = 0;  // distinct query tiles before this chunk
  for (int t0 = 0; t0 < n_qs; t0 += 64) {
    const int e = t0 + lane;
    const bool in = e < cnt;
    const int T = in ? list[e] >> 10 : 0;
    const bool first = in && (e == 0 || (list[e - 1] >> 10) != T);
    const unsigned long long bal = __ballot(first);
    const int32_t slot = base + seen + __popcll(bal & (~0ull >> (63 - lane))) - 1;  // firsts up to and including this lane
    if (e < n_qs) kt_slot[row * n_qs + e] = in ? slot : -1;
    if (first) slot_table[(m * n_qt + T) * n_kt + U] = slot;
    seen += __popcll(bal);
  }
}

hipError_t launch_tile_slots(const int32_t* kt_cnt, const int32_t* kt_ent, int64_t mask_bh, int n_qt, int n_kt, int n_qs,
                             int32_t* pair_base, int32_t* kt_slot, int32_t* slot_table, hipStream_t stream) {
  const int64_t rows = mask_bh * n_kt, table = mask_bh * n_qt * n_kt;
  if (rows <= 0 || table <= 0 || n_qs <= 0) return hipSuccess;
  const int64_t blocks = (rows + 3) / 4;
  if (blocks > 0x7fffffffLL) return hipErrorInvalidValue;
  // the per-row counts rest in the first `rows` entries of kt_slot (which has rows * n_qs >= rows entries) until the
  // prefix sum has read them
  hipLaunchKernelGGL(tile_pair_count_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, kt_cnt, kt_ent, rows, n_qs, kt_slot);
  hipLaunchKernelGGL(pair_base_kernel, dim3(1), dim3(1024), 0, stream, kt_slot, rows, pair_base);
  const int64_t fill_blocks = (table + 255) / 256;
  hipLaunchKernelGGL(fill_i32_kernel, dim3((unsigned)(fill_blocks < 4096 ? fill_blocks : 4096)), dim3(256), 0, stream, slot_table, table, -1);
  hipLaunchKernelGGL(tile_slots_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, kt_cnt, kt_ent, pair_base, rows, n_qt, n_kt, n_qs,
                     kt_slot, slot_table);
  return hipGetLastError();
}

// Backward statistics, one pass over O and dO: stats[r] = lse[r] * log2(e) and stats[rows + r] = -delta[r] =
// -sum_c dO[r, c] * O[r, c] in fp32 (reference: bwd_attend_prep_ker, flex_block_attn_h100.cu:375-379).  The backward
// kernels exponentiate in base 2, hence the pre-scaled LSE; they start the dP accumulators from the second plane, so that
// the matrix instructions themselves form dP - delta (the reference preloads its accumulator the same way,
// flex_block_attn_h100.cu:445-467), hence the sign.  16 lanes per row (16 bytes of each operand per lane).
__global__ __attribute__((amdgpu_flat_work_group_size(256, 256))) void bwd_stats_kernel(const __bf16* __restrict__ o,
                                                                                        const __bf16* __restrict__ d_o,
                                                                                        const float* __restrict__ lse,
                                                                                        float* __restrict__ stats, int64_t rows) {
  const int sub = threadIdx.x & 15;
  for (int64_t r = (int64_t)blockIdx.x * 16 + (threadIdx.x >> 4); r < rows; r += (int64_t)gridDim.x * 16) {
    const bf16x8 a = *reinterpret_cast<const bf16x8*>(o + r * kHeadDim + sub * 8);
    const bf16x8 b = *reinterpret_cast<const bf16x8*>(d_o + r * kHeadDim + sub * 8);
    float acc = 0.f;
#pragma unroll
    for (int t = 0; t < 8; ++t) acc += (float)a[t] * (float)b[t];
    acc += __shfl_xor(acc, 8);
    acc += __shfl_xor(acc, 4);
    acc += __shfl_xor(acc, 2);
    acc += __shfl_xor(acc, 1);
    if (sub == 0) {
      stats[r] = lse[r] * 1.4426950408889634f;
      stats[rows + r] = -acc;
    }
  }
}

hipError_t launch_bwd_stats(const __bf16* o, const __bf16* d_o, const float* lse, float* stats, int64_t rows, hipStream_t stream) {
  if (rows <= 0) return hipSuccess;
  int64_t blocks = (rows + 15) / 16;
  if (blocks > 65536) blocks = 65536;
  hipLaunchKernelGGL(bwd_stats_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, o, d_o, lse, stats, rows);
  return hipGetLastError();
}

}  // namespace fba
