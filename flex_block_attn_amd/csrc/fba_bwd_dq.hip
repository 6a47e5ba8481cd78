// Backward, dQ: gfx950, head_dim 128, bf16 in / fp32 accumulate / bf16 out, no atomics.
//
// With P = exp(S/sqrt(D) - LSE), delta = rowsum(dO o O), dP = dO V^T, dS = P o (dP - delta) / sqrt(D):
//   dQ = dS K                                   (reference: flex_block_attn_h100.cu:498-529, :750-753)
// The reference forms dQ inside its key-major kernel and adds it into an fp32 buffer with reducing stores
// (:707-708).  Here a query-major kernel owns its dQ rows: it walks the per-query-block lists exactly like the forward
// kernel and recomputes S and dP.
//
// Work-group = 128 query rows, wave = 32 rows, lane = query row (everything transposed, as in the forward kernel):
//   S^T = K Q^T, dP^T = V dO^T         A = K / V slab rows from LDS (128-bit fetches), B = Q / dO in registers
//   dS^T = exp2(c S^T - lse2) o (dP^T - delta)
//   dQ^T += K^T dS^T                   A = K slab through transposing LDS fetches, B = dS^T packed to bf16
// Every step handles one 32-key slab: scores, dS, dQ update.  Two waves per SIMD overlap each other (one wave's matrix
// instructions cover the other's exponentials).  K and V slabs travel global -> LDS directly into a ring of four
// (K | V) buffers; slab t+4 is requested when slab t is dead, three steps before its first use.
#include <type_traits>

#include "fba_common.h"
#include "fba_kernels.h"

namespace fba {

namespace {

constexpr int kSlab = 32;
constexpr int kSlabBytes = kSlab * kRowBytes;  // 8 KiB
constexpr int kPairBytes = 2 * kSlabBytes;     // K slab | V slab
constexpr int kRing = 4;

template <int N>
using IC = std::integral_constant<int, N>;

}  // namespace

// kTiled: see the forward kernel (tile lists with a predicate per 16-row group instead of block lists).
template <bool kTiled>
__global__ __attribute__((amdgpu_flat_work_group_size(256, 256), amdgpu_waves_per_eu(2, 2))) void dq_kernel(const BwdParams p) {
  extern __shared__ __attribute__((aligned(16))) char smem[];  // ring [4] of (K slab | V slab)
  constexpr int TQ = 128;

  const int tid = threadIdx.x, lane = tid & 63, l32 = lane & 31, h = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  // whole items first (dealt to the XCDs in contiguous spans), then the parts of the split items
  int item, part = 0, parts = 1;
  if ((int)blockIdx.x < p.split.main_wgs) {
    item = xcd_remap(blockIdx.x, p.items_per_xcd);
    if (item >= p.split.first) return;
  } else {
    const int s = blockIdx.x - p.split.main_wgs;
    item = p.split.first + s / p.split.parts;
    part = s - (item - p.split.first) * p.split.parts;
    parts = p.split.parts;
  }
  const int tiles_per_head = p.Sq / TQ;
  const int bh = item / tiles_per_head;
  const int qt = item - bh * tiles_per_head;
  const int b = bh / p.Hq, hq = bh - b * p.Hq;
  const int hkv = hq / (p.Hq / p.Hkv);

  const int64_t qrow0 = (int64_t)bh * p.Sq + (int64_t)qt * TQ + wave * 32;
  const char* kp = reinterpret_cast<const char*>(p.k + ((int64_t)(b * p.Hkv + hkv) * p.Skv) * kHeadDim);
  const char* vp = reinterpret_cast<const char*>(p.v + ((int64_t)(b * p.Hkv + hkv) * p.Skv) * kHeadDim);

  const int64_t mrow = (p.mask_bh == 1 ? 0 : (int64_t)bh) * (kTiled ? tiles_per_head : p.nQ) + (kTiled ? qt : (qt * TQ) / p.q_block);
  const int cnt = p.q_cnt[mrow];
  const ConstIdx idx = const_idx(p.q_idx + mrow * p.nK);
  auto key_block = [&](int e) -> int { return kTiled ? idx[e] >> 8 : idx[e]; };
  const int group_bit = 1 << (2 * wave + (l32 >> 4));  // this lane's 16-row group in a tile-list entry
  const int wave_bits = 3 << (2 * wave);               // both groups of this wave
  const int nsub = p.k_block / kSlab;
  // this work-group's range of 32-key steps of the list: all of it, or part `part` of `parts` (even boundaries)
  const int steps_all = cnt * nsub;
  const int t_begin = parts == 1 ? 0 : 2 * (int)(((int64_t)(steps_all / 2) * part) / parts);
  const int nsteps = (parts == 1 ? steps_all : 2 * (int)(((int64_t)(steps_all / 2) * (part + 1)) / parts)) - t_begin;
  const int e_begin = t_begin / nsub, sub_begin = t_begin - e_begin * nsub;

  // Q and dO as B operands: lane holds row l32, d = 16 ks + 8 h .. +7
  bf16x8 qreg[8], doreg[8];
#pragma unroll
  for (int ks = 0; ks < 8; ++ks) {
    qreg[ks] = *reinterpret_cast<const bf16x8*>(p.q + (qrow0 + l32) * kHeadDim + 16 * ks + 8 * h);
    doreg[ks] = *reinterpret_cast<const bf16x8*>(p.d_o + (qrow0 + l32) * kHeadDim + 16 * ks + 8 * h);
  }
  const int64_t rows_total = (int64_t)p.B * p.Hq * p.Sq;
  const float lse2 = p.stats[qrow0 + l32];
  const float neg_dlt = p.stats[rows_total + qrow0 + l32];  // -delta of this lane's row
  const float c = p.scale_log2e;

  RowMajorOffsets rm;
  rm.init(lane);
  TransposedOffsets tr;
  tr.init(lane);
  SlabDma dma;
  dma.init(wave, lane);
  const uint32_t ring_dst = lds_addr(smem);

  f32x16 acc[4];
#pragma unroll
  for (int mb = 0; mb < 4; ++mb)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[mb][r] = 0.f;

  // slab source offsets in list order; the list entry of the following key block is read one block ahead
  const int64_t block_bytes = (int64_t)p.k_block * kRowBytes;
  int e_next = e_begin + 1, rem = nsub - sub_begin;
  int64_t src_off = nsteps > 0 ? key_block(e_begin) * block_bytes + (int64_t)sub_begin * kSlabBytes : 0;
  int blk_next = e_next < cnt ? key_block(e_next) : 0;
  auto next_off = [&]() -> int64_t {  // past the end of the list: offsets of some listed slab
    const int64_t off = src_off;
    if (--rem == 0) {
      rem = nsub;
      src_off = blk_next * block_bytes;
      ++e_next;
      blk_next = e_next < cnt ? key_block(e_next) : 0;
    } else {
      src_off += kSlabBytes;
    }
    return off;
  };
  auto copy_next = [&](int ring) {
    const int64_t off = next_off();
    dma.copy(ring_dst + ring * kPairBytes, kp + off);
    dma.copy(ring_dst + ring * kPairBytes + kSlabBytes, vp + off);
  };

  // S^T and dP^T of one slab: 16 MFMAs, the two chains interleaved.  `between(ks)` runs behind the matrix instructions
  // of operand step ks: the place for the global -> LDS copies a step owes, which take a wave tens of cycles each to issue.
  auto scores = [&](const char* pair, f32x16& s, f32x16& dp, auto between) {
#pragma unroll
    for (int r = 0; r < 16; ++r) { s[r] = 0.f; dp[r] = 0.f; }
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) {
      s = mfma32(lds_read_b128(pair, rm.rd[ks]), qreg[ks], s);
      dp = mfma32(lds_read_b128(pair + kSlabBytes, rm.rd[ks]), doreg[ks], dp);
      between(ks);
    }
  };

  if (nsteps > 0) {
#pragma unroll
    for (int j = 0; j < 4; ++j)
      if (j < nsteps) copy_next(j);
    wait_vmem<0>();
    __syncthreads();
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) { pin(qreg[ks]); pin(doreg[ks]); }

    int e_cmp = 0, rem_cmp = nsub;  // list entry of the slab being computed (tile lists: its predicate bits)
    int bits_cmp = kTiled ? idx[0] & 255 : 255;

    // The copies a step requests (K and V slab t+4 into the buffer of slab t, free behind the step's barrier) are issued
    // by the following step, with block lists in between its first matrix instructions.  Every step requests them, so
    // that the counter of copies in flight means the same thing at every wait; past the end of the list they repeat a
    // listed slab into a buffer that nobody reads any more.
    uint32_t owed_dst = 0;
    int64_t owed_off = 0;

    // step t (t % 4 == R): S_t, dP_t | dS_t | dQ += K_t^T dS_t
    auto step = [&](auto ring_c, auto first_c, int t) {
      constexpr int R = decltype(ring_c)::value;
      constexpr bool kOwed = !decltype(first_c)::value;  // the first step owes nothing
      const bool active = !kTiled || (bits_cmp & group_bit) != 0;
      if constexpr (kTiled && kOwed) {
        dma.copy(owed_dst, kp + owed_off);
        dma.copy(owed_dst + kSlabBytes, vp + owed_off);
      }
      // a wave whose two 16-row groups are both switched off for this slab has nothing to add (wave-uniform branch)
      if (!kTiled || (bits_cmp & wave_bits) != 0) {
        f32x16 s_cur, dp_cur;
        scores(smem + R * kPairBytes, s_cur, dp_cur, [&](int ks) {
          if constexpr (!kTiled && kOwed) {
            if (ks == 0) dma.copy_piece(0, owed_dst, kp + owed_off);
            if (ks == 1) dma.copy_piece(1, owed_dst, kp + owed_off);
            if (ks == 2) dma.copy_piece(0, owed_dst + kSlabBytes, vp + owed_off);
            if (ks == 3) dma.copy_piece(1, owed_dst + kSlabBytes, vp + owed_off);
          }
        });
        bf16x8 dsk[2];
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          float pv = fast_exp2(__builtin_fmaf(s_cur[r], c, -lse2));
          if constexpr (kTiled) pv = active ? pv : 0.f;  // a select, so that inf or NaN of a masked row is discarded
          s_cur[r] = pv * (dp_cur[r] + neg_dlt);
        }
#pragma unroll
        for (int j = 0; j < 2; ++j)
          dsk[j] = pack8(s_cur[8 * j + 0], s_cur[8 * j + 1], s_cur[8 * j + 2], s_cur[8 * j + 3], s_cur[8 * j + 4],
                         s_cur[8 * j + 5], s_cur[8 * j + 6], s_cur[8 * j + 7]);
        const char* k_t = smem + R * kPairBytes;
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
          for (int mb = 0; mb < 4; ++mb) {
            const int roff = 16 * j * kRowBytes;
            const bf16x8 a = cat(lds_read_tr(k_t, tr.rd[mb][0] + roff), lds_read_tr(k_t, tr.rd[mb][1] + roff));
            acc[mb] = mfma32(a, dsk[j], acc[mb]);
          }
      }
      if constexpr (kTiled) {
        if (--rem_cmp == 0) {
          rem_cmp = nsub;
          ++e_cmp;
          bits_cmp = e_cmp < cnt ? idx[e_cmp] & 255 : 0;
        }
      }
      // slab t+2 must have landed; the four copies of slab t+3 may still fly
      wait_vmem<4>();
      __syncthreads();
      owed_dst = ring_dst + R * kPairBytes;
      owed_off = next_off();
    };
    step(IC<0>{}, std::true_type{}, 0);
    step(IC<1>{}, std::false_type{}, 1);
    for (int t = 2; t < nsteps; t += 4) {  // nsteps is even
      step(IC<2>{}, std::false_type{}, t);
      step(IC<3>{}, std::false_type{}, t + 1);
      if (t + 2 >= nsteps) break;
      step(IC<0>{}, std::false_type{}, t + 2);
      step(IC<1>{}, std::false_type{}, t + 3);
    }
    wait_vmem<0>();  // no copy may still be writing LDS when the work-group gives it back
  }

  if (parts > 1) {  // part of a split item: unscaled fp32 partial sums go to the workspace
    float* prow = p.split.ws + ((int64_t)(item - p.split.first) * parts + part) * (TQ * kHeadDim) + (wave * 32 + l32) * kHeadDim;
#pragma unroll
    for (int mb = 0; mb < 4; ++mb)
#pragma unroll
      for (int g = 0; g < 4; ++g)
        *reinterpret_cast<f32x4*>(prow + 32 * mb + 8 * g + 4 * h) = (f32x4){acc[mb][4 * g + 0], acc[mb][4 * g + 1], acc[mb][4 * g + 2], acc[mb][4 * g + 3]};
    return;
  }
  __bf16* orow = p.dq + (qrow0 + l32) * kHeadDim;
#pragma unroll
  for (int mb = 0; mb < 4; ++mb)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const bf16x4 ov = pack4(acc[mb][4 * g + 0] * p.scale, acc[mb][4 * g + 1] * p.scale, acc[mb][4 * g + 2] * p.scale,
                              acc[mb][4 * g + 3] * p.scale);
      *reinterpret_cast<bf16x4*>(orow + 32 * mb + 8 * g + 4 * h) = ov;
    }
}

hipError_t launch_bwd_dq(BwdParams p, hipStream_t stream) {
  constexpr int kSmem = kRing * kPairBytes;
  p.num_items = p.B * p.Hq * (p.Sq / 128);
  // tail splitting on block lists (two work-groups per compute unit); a part stores a 128 x 128 fp32 tile
  p.split = plan_split(p.num_items, 2, 128 * kHeadDim * 4, p.tiled ? nullptr : p.split.ws, p.split_ws_bytes);
  plan_xcd_mapping(p.B * p.Hq, p.split.first, p.items_per_xcd, p.split.main_wgs);
  const int split_items = p.num_items - p.split.first;
  void (*fn)(const BwdParams) = p.tiled ? &dq_kernel<true> : &dq_kernel<false>;
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(fn), hipFuncAttributeMaxDynamicSharedMemorySize, kSmem);
  if (e != hipSuccess) return e;
  hipLaunchKernelGGL(fn, dim3(p.split.main_wgs + split_items * p.split.parts), dim3(256), kSmem, stream, p);
  if (split_items > 0)
    return launch_partial_sum(p.split.ws, p.split.parts, 128 * kHeadDim, p.dq, (int64_t)p.split.first * 128, split_items, p.scale, stream);
  return hipGetLastError();
}

}  // namespace fba
