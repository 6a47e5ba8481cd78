// Backward, dQ from handed-over dS: gfx950, head_dim 128, bf16 in / fp32 accumulate / bf16 out, no atomics.
//
//   dQ = dS K                                   (reference: flex_block_attn_h100.cu:750-753)
// The reference forms dS and dQ in one key-major kernel and adds dQ into an fp32 buffer with reducing stores
// (:707-708).  Here the key-major kernel (dkdv_kernel with kHandOver) stores the bf16 dS of every selected block pair
// once, and this query-major kernel reads it back: two products per pair instead of the six of dq_kernel, which
// recomputes S and dP.  Every dQ element is still written exactly once, by the work-group that owns its row.
//
// Work-group = 128 query rows, wave = 32 rows, lane = query row:
//   dQ^T += K^T dS^T                   A = K slab through transposing LDS fetches, B = dS^T through transposing LDS
//                                      fetches of the wave's own dS unit (layout: fba_common.h)
// The kernel does 8 MFMAs per 16 KiB it reads, so it runs at the speed of memory: K slabs (8 KiB, shared by the four
// waves, mostly L2 hits) and dS units (2 KiB per wave, each read exactly once from HBM) travel global -> LDS directly
// into a ring of four stages; stage t+4 is requested when stage t is dead.
#include <type_traits>

#include "fba_common.h"
#include "fba_kernels.h"

namespace fba {

namespace {

constexpr int kSlab = 32;
constexpr int kSlabBytes = kSlab * kRowBytes;        // 8 KiB: one K slab, or the four dS units of a step
constexpr int kStageBytes = 2 * kSlabBytes;          // K slab | dS units
constexpr int kRing = 4;

template <int N>
using IC = std::integral_constant<int, N>;

}  // namespace

__global__ __attribute__((amdgpu_flat_work_group_size(256, 256), amdgpu_waves_per_eu(2, 2))) void dq_from_ds_kernel(const BwdParams p) {
  extern __shared__ __attribute__((aligned(16))) char smem[];  // ring [4] of (K slab | dS units)
  constexpr int TQ = 128;

  const int tid = threadIdx.x, lane = tid & 63, l32 = lane & 31, h = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int item = xcd_remap(blockIdx.x, p.items_per_xcd);
  if (item >= p.num_items) return;
  const int tiles_per_head = p.Sq / TQ;
  const int bh = item / tiles_per_head;
  const int qt = item - bh * tiles_per_head;
  const int b = bh / p.Hq, hq = bh - b * p.Hq;
  const int hkv = hq / (p.Hq / p.Hkv);

  const int64_t qrow0 = (int64_t)bh * p.Sq + (int64_t)qt * TQ + wave * 32;
  const char* kp = reinterpret_cast<const char*>(p.k + ((int64_t)(b * p.Hkv + hkv) * p.Skv) * kHeadDim);

  const int qblk = (qt * TQ) / p.q_block;
  const int tq = (qt * TQ - qblk * p.q_block) / TQ;  // this tile's position inside its query block
  const int64_t mrow = (p.mask_bh == 1 ? 0 : (int64_t)bh) * p.nQ + qblk;
  const int cnt = p.q_cnt[mrow];
  const ConstIdx idx = const_idx(p.q_idx + mrow * p.nK);
  const ConstIdx slot = const_idx(p.q_slot + mrow * p.nK);
  const int nsub = p.k_block / kSlab;
  const int nsteps = cnt * nsub;
  const int64_t pair_bytes = (int64_t)p.q_block * p.k_block * 2;
  // dS of this wave's 32 rows: pair base + (tq * nsub + t) * 4 units + wave, t = 32-key slab inside the key block
  const int64_t head_pairs = p.mask_bh == 1 ? (int64_t)bh * const_idx(p.pair_base)[p.nK] : 0;
  const char* ds_base = reinterpret_cast<const char*>(p.ds_ws) + head_pairs * pair_bytes + ((int64_t)tq * nsub * 4 + wave) * kDsUnitBytes;

  TransposedOffsets tr;
  tr.init(lane);
  SlabDma dma;
  dma.init(wave, lane);
  const uint32_t ring_dst = lds_addr(smem);
  // Transposing fetches of the B operand from the wave's unit.  Group G = lane / 16 of the wave serves query rows
  // 16 (G % 2) .. +15 and the key half 4 (G / 2) .. +3 of each 8 keys; source lane s = lane % 16 addresses the slot of
  // key (16 jj + 8 rr + 4 (G / 2) + s / 4) and query group 4 (G % 2) + s % 4.
  int ds_off[2][2];
#pragma unroll
  for (int jj = 0; jj < 2; ++jj)
#pragma unroll
    for (int rr = 0; rr < 2; ++rr) {
      const int G = lane >> 4, s = lane & 15;
      ds_off[jj][rr] = kSlabBytes + wave * kDsUnitBytes + ds_unit_slot_off(16 * jj + 8 * rr + 4 * (G >> 1) + (s >> 2), 4 * (G & 1) + (s & 3));
    }

  f32x16 acc[4];
#pragma unroll
  for (int mb = 0; mb < 4; ++mb)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[mb][r] = 0.f;

  // sources of the next stage to request, in list order; the following list entry is read one block ahead
  const int64_t block_bytes = (int64_t)p.k_block * kRowBytes;
  int e_next = 1, rem = nsub;
  int64_t k_off = cnt > 0 ? idx[0] * block_bytes : 0;
  int64_t ds_off_g = cnt > 0 ? slot[0] * pair_bytes : 0;
  int blk_next = cnt > 1 ? idx[1] : 0;
  int slot_next = cnt > 1 ? slot[1] : 0;
  const uint32_t lane16 = (uint32_t)lane * 16;
  auto copy_next = [&](int ring) {
    const uint32_t dst = ring_dst + ring * kStageBytes;
    dma.copy(dst, kp + k_off);
    dma16_stream(dst + kSlabBytes + wave * kDsUnitBytes, ds_base + ds_off_g, lane16);
    dma16_stream(dst + kSlabBytes + wave * kDsUnitBytes + 1024, ds_base + ds_off_g, lane16 + 1024);
    if (--rem == 0) {
      rem = nsub;
      k_off = blk_next * block_bytes;
      ds_off_g = slot_next * pair_bytes;
      ++e_next;
      blk_next = e_next < cnt ? idx[e_next] : 0;
      slot_next = e_next < cnt ? slot[e_next] : 0;
    } else {
      k_off += kSlabBytes;
      ds_off_g += 4 * kDsUnitBytes;
    }
  };

  if (nsteps > 0) {
#pragma unroll
    for (int j = 0; j < 4; ++j)
      if (j < nsteps) copy_next(j);
    wait_vmem<0>();
    __syncthreads();

    // step t (t % 4 == R): dQ += K_t^T dS_t
    auto step = [&](auto ring_c, int t) {
      constexpr int R = decltype(ring_c)::value;
      const char* stage = smem + R * kStageBytes;
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const bf16x8 dsk = cat(lds_read_tr(stage, ds_off[j][0]), lds_read_tr(stage, ds_off[j][1]));
#pragma unroll
        for (int mb = 0; mb < 4; ++mb) {
          const int roff = 16 * j * kRowBytes;
          const bf16x8 a = cat(lds_read_tr(stage, tr.rd[mb][0] + roff), lds_read_tr(stage, tr.rd[mb][1] + roff));
          acc[mb] = mfma32(a, dsk, acc[mb]);
        }
      }
      // stage t+1 must have landed (first read in step t+1); the copies of stages t+2 and t+3 (4 each) may still fly
      if (t + 3 < nsteps) wait_vmem<8>(); else if (t + 2 < nsteps) wait_vmem<4>(); else wait_vmem<0>();
      __syncthreads();
      if (t + 4 < nsteps) copy_next(R);
    };
    for (int t = 0; t < nsteps; t += 4) {  // nsteps is a multiple of 4
      step(IC<0>{}, t);
      step(IC<1>{}, t + 1);
      step(IC<2>{}, t + 2);
      step(IC<3>{}, t + 3);
    }
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

hipError_t launch_bwd_dq_from_ds(BwdParams p, hipStream_t stream) {
  constexpr int kSmem = kRing * kStageBytes;
  if (p.tiled || p.ds_ws == nullptr) return hipErrorInvalidValue;
  p.num_items = p.B * p.Hq * (p.Sq / 128);
  p.items_per_xcd = (p.num_items + kNumXcd - 1) / kNumXcd;
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&dq_from_ds_kernel), hipFuncAttributeMaxDynamicSharedMemorySize, kSmem);
  if (e != hipSuccess) return e;
  hipLaunchKernelGGL(dq_from_ds_kernel, dim3(p.items_per_xcd * kNumXcd), dim3(256), kSmem, stream, p);
  return hipGetLastError();
}

}  // namespace fba
