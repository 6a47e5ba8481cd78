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
//
// kTiled: tile lists.  The workspace is divided into (128-row query tile, 128-key tile) pairs of 16 units; the list of the
// work-group's query tile names key blocks with a predicate per 16 rows.  A wave whose rows do not select a key block has
// no unit there (the key-major kernel stored none): it copies 2 KiB of zeros instead, so that every wave issues the same
// number of copies per stage, and leaves the matrix work of those steps out.
#include <mutex>
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

template <bool kTiled>
__global__ __attribute__((amdgpu_flat_work_group_size(256, 256), amdgpu_waves_per_eu(2, 2))) void dq_from_ds_kernel(const BwdParams p) {
  extern __shared__ __attribute__((aligned(16))) char smem[];  // ring [4] of (K slab | dS units)
  constexpr int TQ = 128;

  if (!workspace_holds_lists(p)) return;  // the launcher's last launch reports it
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

  const int qblk = (qt * TQ) / p.q_block;
  const int tq = kTiled ? 0 : (qt * TQ - qblk * p.q_block) / TQ;  // this tile's position inside its query block
  const int n_kt = p.Skv / 128;
  const int64_t mrow = (p.mask_bh == 1 ? 0 : (int64_t)bh) * (kTiled ? tiles_per_head : p.nQ) + (kTiled ? qt : qblk);
  const int cnt = p.q_cnt[mrow];
  const ConstIdx idx = const_idx(p.q_idx + mrow * p.nK);
  // block lists: pair number per list entry; tile lists: pair number per key tile, for this query tile
  const ConstIdx slot = const_idx(p.q_slot + mrow * (kTiled ? n_kt : p.nK));
  const int nsub = p.k_block / kSlab;
  // this work-group's range of 32-key steps of the list: all of it, or part `part` of `parts` (boundaries on whole rings)
  const int steps_all = cnt * nsub;
  const int t_begin = parts == 1 ? 0 : 4 * (int)(((int64_t)(steps_all / 4) * part) / parts);
  const int t_end = parts == 1 ? steps_all : 4 * (int)(((int64_t)(steps_all / 4) * (part + 1)) / parts);
  const int nsteps = t_end - t_begin;
  const int e_begin = t_begin / nsub, sub_begin = t_begin - e_begin * nsub;
  const int64_t pair_bytes = kTiled ? 16 * kDsUnitBytes : (int64_t)p.q_block * p.k_block * 2;
  // dS of this wave's 32 rows: pair base + (tq * nsub + t) * 4 units + wave, t = 32-key slab inside the key block (inside
  // the key tile with tile lists)
  const int64_t head_pairs = p.mask_bh == 1 ? (int64_t)bh * const_idx(p.pair_base)[kTiled ? n_kt : p.nK] : 0;
  const char* ds_base = reinterpret_cast<const char*>(p.ds_ws) + head_pairs * pair_bytes + ((int64_t)tq * nsub * 4 + wave) * kDsUnitBytes;
  auto key_block = [&](int e) -> int { return kTiled ? idx[e] >> 8 : idx[e]; };
  const int wave_bits = 3 << (2 * wave);  // predicate bits of this wave's two 16-row groups in a tile-list entry

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
  int e_next = e_begin + 1, rem = nsub - sub_begin;
  int64_t k_off = nsteps > 0 ? key_block(e_begin) * block_bytes + (int64_t)sub_begin * kSlabBytes : 0;
  int64_t ds_off_g = nsteps > 0 && !kTiled ? slot[e_begin] * pair_bytes + (int64_t)sub_begin * (4 * kDsUnitBytes) : 0;
  int blk_next = e_next < cnt ? key_block(e_next) : 0;
  int slot_next = e_next < cnt && !kTiled ? slot[e_next] : 0;
  // tile lists: predicate bits of the entry being requested and of the next one; pair number of the key tile that the
  // next stage's slab lies in, read one stage ahead
  int bits_req = kTiled && cnt > 0 ? idx[0] & 255 : 0;
  int bits_req_next = kTiled && cnt > 1 ? idx[1] & 255 : 0;
  int tile_slot = kTiled && cnt > 0 ? slot[(int)(k_off >> 15)] : 0;  // 32 KiB of K rows per key tile
  const uint32_t lane16 = (uint32_t)lane * 16;
  auto copy_next = [&](int ring) {
    const uint32_t dst = ring_dst + ring * kStageBytes;
    dma.copy(dst, kp + k_off);
    const char* src = ds_base + ds_off_g;
    if constexpr (kTiled) {
      const int t = (int)(k_off >> 13) & 3;  // 32-key slab inside its key tile
      src = (bits_req & wave_bits) != 0 ? ds_base + (int64_t)tile_slot * pair_bytes + t * (4 * kDsUnitBytes) : p.zero_unit;
    }
    dma16_stream(dst + kSlabBytes + wave * kDsUnitBytes, src, lane16);
    dma16_stream(dst + kSlabBytes + wave * kDsUnitBytes + 1024, src, lane16 + 1024);
    if (--rem == 0) {
      rem = nsub;
      k_off = blk_next * block_bytes;
      ds_off_g = slot_next * pair_bytes;
      bits_req = bits_req_next;
      ++e_next;
      blk_next = e_next < cnt ? key_block(e_next) : 0;
      if constexpr (kTiled) bits_req_next = e_next < cnt ? idx[e_next] & 255 : 0;
      else slot_next = e_next < cnt ? slot[e_next] : 0;
    } else {
      k_off += kSlabBytes;
      ds_off_g += 4 * kDsUnitBytes;
    }
    if constexpr (kTiled) tile_slot = slot[(int)(k_off >> 15)];  // past the last stage: some listed tile's number, unused
  };

  if (nsteps > 0) {
#pragma unroll
    for (int j = 0; j < 4; ++j)
      if (j < nsteps) copy_next(j);
    wait_vmem<0>();
    __syncthreads();

    // tile lists: predicate bits of the entry whose slab is worked on (a second walk over the list)
    int e_cmp = 0, rem_cmp = nsub;
    int bits_cmp = kTiled ? idx[0] & 255 : 255;
    int bits_ahead = kTiled && cnt > 1 ? idx[1] & 255 : 0;

    // step t (t % 4 == R): dQ += K_t^T dS_t
    auto step = [&](auto ring_c, int t) {
      constexpr int R = decltype(ring_c)::value;
      const char* stage = smem + R * kStageBytes;
      if (!kTiled || (bits_cmp & wave_bits) != 0) {
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
      }
      if constexpr (kTiled) {
        if (--rem_cmp == 0) {
          rem_cmp = nsub;
          ++e_cmp;
          bits_cmp = bits_ahead;
          bits_ahead = e_cmp + 1 < cnt ? idx[e_cmp + 1] & 255 : 0;
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

namespace {

// What a wave copies in place of a dS unit that nobody stored (tile lists).  Part of the library's device image and never
// written; host code reaches it only through the address hipGetSymbolAddress returns for the current device.
__device__ __attribute__((aligned(256))) char g_zero_unit[kDsUnitBytes];

hipError_t zero_unit_address(const char** out) {
  constexpr int kMaxDevices = 64;
  static std::mutex mu;
  static const char* cache[kMaxDevices] = {};
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  if (dev < 0 || dev >= kMaxDevices) return hipErrorInvalidDevice;
  std::lock_guard<std::mutex> lock(mu);
  if (cache[dev] == nullptr) {
    void* ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(g_zero_unit));
    if (e != hipSuccess) return e;
    cache[dev] = static_cast<const char*>(ptr);
  }
  *out = cache[dev];
  return hipSuccess;
}

}  // namespace

// Sums the fp32 partial tiles of the split items in part order: out = scale * sum_p partial_p, as bf16.  One thread per
// four columns; `rows_per_slot` rows of 128 columns per part, `sections` consecutive outputs per slot (dK/dV: two).
__global__ __attribute__((amdgpu_flat_work_group_size(256, 256))) void partial_sum_kernel(const float* ws, int parts, int64_t slot_floats,
                                                                                          __bf16* out, int64_t out_row0, float scale) {
  const int tid = threadIdx.x;
  const int64_t row = (int64_t)blockIdx.x * 8 + (tid >> 5);  // row among 128 * (split items) rows
  const int c4 = (tid & 31) * 4;
  const int64_t it = row >> 7;
  const int r = (int)(row & 127);
  const float* src = ws + it * parts * slot_floats + r * kHeadDim + c4;
  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  for (int q = 0; q < parts; ++q) acc += *reinterpret_cast<const f32x4*>(src + q * slot_floats);
  *reinterpret_cast<bf16x4*>(out + (out_row0 + row) * kHeadDim + c4) = pack4(acc[0] * scale, acc[1] * scale, acc[2] * scale, acc[3] * scale);
}

hipError_t launch_partial_sum(const float* ws, int parts, int64_t slot_floats, __bf16* out, int64_t out_row0, int n_items, float scale,
                              hipStream_t stream) {
  hipLaunchKernelGGL(partial_sum_kernel, dim3(n_items * 16), dim3(256), 0, stream, ws, parts, slot_floats, out, out_row0, scale);
  return hipGetLastError();
}

__global__ __attribute__((amdgpu_flat_work_group_size(256, 256))) void poison_unless_fit_kernel(const BwdParams p, __bf16* __restrict__ out_a, __bf16* __restrict__ out_b, int64_t n) {
  if (workspace_holds_lists(p)) return;
  const __bf16 nan = (__bf16)__builtin_nanf("");
  for (int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x; t < n; t += (int64_t)gridDim.x * 256) {
    out_a[t] = nan;
    if (out_b) out_b[t] = nan;
  }
}

hipError_t launch_poison_unless_fit(const BwdParams& p, __bf16* out_a, __bf16* out_b, int64_t n, hipStream_t stream) {
  if (n <= 0) return hipSuccess;
  const int64_t blocks = (n + 255) / 256;
  hipLaunchKernelGGL(poison_unless_fit_kernel, dim3((unsigned)(blocks < 64 ? blocks : 64)), dim3(256), 0, stream, p, out_a, out_b, n);
  return hipGetLastError();
}

hipError_t launch_bwd_dq_from_ds(BwdParams p, hipStream_t stream) {
  constexpr int kSmem = kRing * kStageBytes;
  if (p.ds_ws == nullptr) return hipErrorInvalidValue;
  p.num_items = p.B * p.Hq * (p.Sq / 128);
  // tail splitting on block lists (two work-groups per compute unit); a part stores a 128 x 128 fp32 tile
  p.split = plan_split(p.num_items, 2, 128 * kHeadDim * 4, p.tiled ? nullptr : p.split.ws, p.split_ws_bytes);
  plan_xcd_mapping(p.B * p.Hq, p.split.first, p.items_per_xcd, p.split.main_wgs);
  const int split_items = p.num_items - p.split.first;
  void (*fn)(const BwdParams) = p.tiled ? &dq_from_ds_kernel<true> : &dq_from_ds_kernel<false>;
  hipError_t e = hipSuccess;
  if (p.tiled && (e = zero_unit_address(&p.zero_unit)) != hipSuccess) return e;
  e = hipFuncSetAttribute(reinterpret_cast<const void*>(fn), hipFuncAttributeMaxDynamicSharedMemorySize, kSmem);
  if (e != hipSuccess) return e;
  hipLaunchKernelGGL(fn, dim3(p.split.main_wgs + split_items * p.split.parts), dim3(256), kSmem, stream, p);
  if (split_items > 0) {
    e = launch_partial_sum(p.split.ws, p.split.parts, 128 * kHeadDim, p.dq, (int64_t)p.split.first * 128, split_items, p.scale, stream);
    if (e != hipSuccess) return e;
  }
  return launch_poison_unless_fit(p, p.dq, nullptr, (int64_t)p.B * p.Hq * p.Sq * kHeadDim, stream);
}

}  // namespace fba
