// Backward kernels for gfx950, head_dim 128, bf16 in / fp32 accumulate / bf16 out, no atomics.
//
// With P = exp(S/sqrt(D) - LSE), delta = rowsum(dO o O), dP = dO V^T, dS = P o (dP - delta) / sqrt(D):
//   dV = P^T dO,  dK = dS^T Q,  dQ = dS K      (reference: flex_block_attn_h100.cu:498-537, :750-753)
// The reference forms all three in one key-major kernel and adds dQ (and dK, dV) into fp32 buffers with reducing
// stores (:556, :566, :707-708).  Here two kernels each own their output rows and recompute S and dP:
//   * dq_kernel walks the per-query-block lists (same traversal as the forward kernel);
//   * dkdv_kernel walks the per-key-block lists and loops over the query heads of a GQA group.
// Which operand sits in registers is chosen so that the summed index of the second product is the register index
// of the first product's accumulator; the operand that has to be read "column-wise" comes through the
// transposing LDS fetch.
#include "fba_common.h"
#include "fba_kernels.h"

namespace fba {

// ------------------------------------------------------------------------------------------------------------------
// dQ: work-group = 128 query rows, wave = 32 rows.  Per 64-key slab:
//   S^T = K Q^T, dP^T = V dO^T         (A = K / V slab rows, B = Q / dO in registers; lane = query row)
//   dS^T = exp2(c S^T - lse2) o (dP^T - delta)
//   dQ^T += K^T dS^T                   (A = K slab through transposing fetches, B = dS^T packed)
// ------------------------------------------------------------------------------------------------------------------
__global__ __attribute__((amdgpu_flat_work_group_size(256, 256))) void dq_kernel(const BwdParams p) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  constexpr int TQ = 128;
  constexpr int kSlab = 64;
  constexpr int kTileBytes = kSlab * kRowBytes;

  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, l32 = lane & 31, h = lane >> 5;
  const int item = xcd_remap(blockIdx.x, p.items_per_xcd);
  if (item >= p.num_items) return;
  const int tiles_per_head = p.Sq / TQ;
  const int bh = item / tiles_per_head;
  const int qt = item - bh * tiles_per_head;
  const int b = bh / p.Hq, hq = bh - b * p.Hq;
  const int hkv = hq / (p.Hq / p.Hkv);

  const int64_t qrow0 = (int64_t)bh * p.Sq + (int64_t)qt * TQ + wave * 32;
  const __bf16* qp = p.q + qrow0 * kHeadDim;
  const __bf16* dop = p.d_o + qrow0 * kHeadDim;
  const __bf16* kp = p.k + ((int64_t)(b * p.Hkv + hkv) * p.Skv) * kHeadDim;
  const __bf16* vp = p.v + ((int64_t)(b * p.Hkv + hkv) * p.Skv) * kHeadDim;

  const int qblk = (qt * TQ) / p.q_block;
  const int64_t mrow = (p.mask_bh == 1 ? 0 : (int64_t)bh) * p.nQ + qblk;
  const int cnt = p.q_cnt[mrow];
  const int32_t* __restrict__ idx = p.q_idx + mrow * p.nK;
  const int nsub = p.k_block / kSlab;
  const int nsteps = cnt * nsub;

  bf16x8 qreg[8], doreg[8];
#pragma unroll
  for (int ks = 0; ks < 8; ++ks) {
    qreg[ks] = *reinterpret_cast<const bf16x8*>(qp + (int64_t)l32 * kHeadDim + 16 * ks + 8 * h);
    doreg[ks] = *reinterpret_cast<const bf16x8*>(dop + (int64_t)l32 * kHeadDim + 16 * ks + 8 * h);
  }
  const float lse2 = p.lse[qrow0 + l32] * 1.4426950408889634f;
  const float dlt = p.delta[qrow0 + l32];

  RowMajorOffsets rm;
  rm.init(lane);
  TransposedOffsets tr;
  tr.init(lane);
  const int wr_off = tile_off(tid >> 4, tid & 15);
  const float c = p.scale_log2e;

  f32x16 acc[4];
#pragma unroll
  for (int mb = 0; mb < 4; ++mb)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[mb][r] = 0.f;

  TileCopy<kSlab> kc, vc;
  int e_next = 0, s_next = 0;
  auto fetch = [&]() {
    const int64_t row0 = (int64_t)idx[e_next] * p.k_block + s_next * kSlab;
    kc.load(kp + row0 * kHeadDim, tid);
    vc.load(vp + row0 * kHeadDim, tid);
    if (++s_next == nsub) { s_next = 0; ++e_next; }
  };
  if (nsteps > 0) {
    fetch();
    kc.store(smem, wr_off);
    vc.store(smem + kTileBytes, wr_off);
  }
  __syncthreads();
  // all loads so far must have landed: inside the loop the vector-memory counter is for the slab prefetch only
  wait_vmem_all();
#pragma unroll
  for (int ks = 0; ks < 8; ++ks) { pin(qreg[ks]); pin(doreg[ks]); }

  for (int step = 0; step < nsteps; ++step) {
    const char* ks_lds = smem + (step & 1) * 2 * kTileBytes;
    const char* vs_lds = ks_lds + kTileBytes;
    char* nxt = smem + ((step + 1) & 1) * 2 * kTileBytes;
    const bool more = step + 1 < nsteps;
    if (more) fetch();

    f32x16 s[2], dp[2];
#pragma unroll
    for (int m2 = 0; m2 < 2; ++m2)
#pragma unroll
      for (int r = 0; r < 16; ++r) { s[m2][r] = 0.f; dp[m2][r] = 0.f; }
#pragma unroll
    for (int m2 = 0; m2 < 2; ++m2)
#pragma unroll
      for (int ks = 0; ks < 8; ++ks) {
        const bf16x8 ak = lds_read_b128(ks_lds, rm.rd[ks] + m2 * 32 * kRowBytes);
        s[m2] = mfma32(ak, qreg[ks], s[m2]);
        const bf16x8 av = lds_read_b128(vs_lds, rm.rd[ks] + m2 * 32 * kRowBytes);
        dp[m2] = mfma32(av, doreg[ks], dp[m2]);
      }

    bf16x8 dsk[2][2];
#pragma unroll
    for (int m2 = 0; m2 < 2; ++m2) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const float pv = fast_exp2(__builtin_fmaf(s[m2][r], c, -lse2));
        s[m2][r] = pv * (dp[m2][r] - dlt);
      }
#pragma unroll
      for (int j = 0; j < 2; ++j)
        dsk[m2][j] = pack8(s[m2][8 * j + 0], s[m2][8 * j + 1], s[m2][8 * j + 2], s[m2][8 * j + 3], s[m2][8 * j + 4],
                           s[m2][8 * j + 5], s[m2][8 * j + 6], s[m2][8 * j + 7]);
    }

#pragma unroll
    for (int mb = 0; mb < 4; ++mb)
#pragma unroll
      for (int m2 = 0; m2 < 2; ++m2)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          const int roff = (32 * m2 + 16 * j) * kRowBytes;
          const bf16x8 a = cat(lds_read_tr(ks_lds, tr.rd[mb][0] + roff), lds_read_tr(ks_lds, tr.rd[mb][1] + roff));
          acc[mb] = mfma32(a, dsk[m2][j], acc[mb]);
        }

    if (more) {
      kc.store(nxt, wr_off);
      vc.store(nxt + kTileBytes, wr_off);
    }
    __syncthreads();
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

// ------------------------------------------------------------------------------------------------------------------
// dK, dV: work-group = 128 key rows of one (batch, kv head), wave = 32 keys.  For every query head of the GQA group
// and every query block in the key block's list, per 64-query slab (Q, dO, lse2, delta staged in LDS):
//   S = Q K^T, dP = dO V^T             (A = Q / dO slab rows, B = K / V in registers; lane = key, registers = query)
//   P = exp2(c S - lse2[q]),  dS = P o (dP - delta[q])
//   dV^T += dO^T P,  dK^T += Q^T dS    (A = dO / Q slab through transposing fetches, B = P / dS packed)
// ------------------------------------------------------------------------------------------------------------------
__global__ __attribute__((amdgpu_flat_work_group_size(256, 256))) void dkdv_kernel(const BwdParams p) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  constexpr int TK = 128;
  constexpr int kSlab = 64;
  constexpr int kTileBytes = kSlab * kRowBytes;
  constexpr int kStageBytes = 2 * kTileBytes + 2 * kSlab * 4;  // Q, dO, lse2, delta

  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, l32 = lane & 31, h = lane >> 5;
  const int item = xcd_remap(blockIdx.x, p.items_per_xcd);
  if (item >= p.num_items) return;
  const int tiles_per_head = p.Skv / TK;
  const int bhk = item / tiles_per_head;
  const int kt = item - bhk * tiles_per_head;
  const int b = bhk / p.Hkv, hkv = bhk - b * p.Hkv;
  const int group = p.Hq / p.Hkv;
  const int kblk = (kt * TK) / p.k_block;

  const int64_t krow0 = (int64_t)bhk * p.Skv + (int64_t)kt * TK + wave * 32;
  bf16x8 kreg[8], vreg[8];
#pragma unroll
  for (int ks = 0; ks < 8; ++ks) {
    kreg[ks] = *reinterpret_cast<const bf16x8*>(p.k + (krow0 + l32) * kHeadDim + 16 * ks + 8 * h);
    vreg[ks] = *reinterpret_cast<const bf16x8*>(p.v + (krow0 + l32) * kHeadDim + 16 * ks + 8 * h);
  }

  const int nsub = p.q_block / kSlab;
  auto list_row = [&](int g) -> int64_t {
    const int64_t bh = (int64_t)b * p.Hq + hkv * group + g;
    return (p.mask_bh == 1 ? 0 : bh) * p.nK + kblk;
  };
  int nsteps = 0;
  for (int g = 0; g < group; ++g) nsteps += p.k_cnt[list_row(g)];
  nsteps *= nsub;

  RowMajorOffsets rm;
  rm.init(lane);
  TransposedOffsets tr;
  tr.init(lane);
  const int wr_off = tile_off(tid >> 4, tid & 15);
  const float c = p.scale_log2e;

  f32x16 acc_k[4], acc_v[4];
#pragma unroll
  for (int mb = 0; mb < 4; ++mb)
#pragma unroll
    for (int r = 0; r < 16; ++r) { acc_k[mb][r] = 0.f; acc_v[mb][r] = 0.f; }

  TileCopy<kSlab> qc, dc;
  float stat = 0.f;  // thread t < 64: lse2[t]; 64 <= t < 128: delta[t - 64]
  int g_next = 0, e_next = 0, s_next = 0;
  int cur_cnt = nsteps > 0 ? p.k_cnt[list_row(0)] : 0;
  auto fetch = [&]() {
    while (e_next >= cur_cnt) {
      ++g_next;
      e_next = 0;
      cur_cnt = p.k_cnt[list_row(g_next)];
    }
    const int64_t bh = (int64_t)b * p.Hq + hkv * group + g_next;
    const int qb = p.k_idx[list_row(g_next) * p.nQ + e_next];
    const int64_t row0 = bh * p.Sq + (int64_t)qb * p.q_block + s_next * kSlab;
    qc.load(p.q + row0 * kHeadDim, tid);
    dc.load(p.d_o + row0 * kHeadDim, tid);
    if (tid < 64) stat = p.lse[row0 + tid] * 1.4426950408889634f;
    else if (tid < 128) stat = p.delta[row0 + tid - 64];
    if (++s_next == nsub) { s_next = 0; ++e_next; }
  };
  auto stash = [&](char* stage) {
    qc.store(stage, wr_off);
    dc.store(stage + kTileBytes, wr_off);
    if (tid < 128) reinterpret_cast<float*>(stage + 2 * kTileBytes)[tid] = stat;
  };

  if (nsteps > 0) {
    fetch();
    stash(smem);
  }
  __syncthreads();
  // all loads so far must have landed: inside the loop the vector-memory counter is for the slab prefetch only
  wait_vmem_all();
#pragma unroll
  for (int ks = 0; ks < 8; ++ks) { pin(kreg[ks]); pin(vreg[ks]); }

  for (int step = 0; step < nsteps; ++step) {
    const char* q_lds = smem + (step & 1) * kStageBytes;
    const char* do_lds = q_lds + kTileBytes;
    const float* st_lds = reinterpret_cast<const float*>(q_lds + 2 * kTileBytes);
    char* nxt = smem + ((step + 1) & 1) * kStageBytes;
    const bool more = step + 1 < nsteps;
    if (more) fetch();

    f32x16 s[2], dp[2];
#pragma unroll
    for (int m2 = 0; m2 < 2; ++m2)
#pragma unroll
      for (int r = 0; r < 16; ++r) { s[m2][r] = 0.f; dp[m2][r] = 0.f; }
#pragma unroll
    for (int m2 = 0; m2 < 2; ++m2)
#pragma unroll
      for (int ks = 0; ks < 8; ++ks) {
        const bf16x8 aq = lds_read_b128(q_lds, rm.rd[ks] + m2 * 32 * kRowBytes);
        s[m2] = mfma32(aq, kreg[ks], s[m2]);
        const bf16x8 ad = lds_read_b128(do_lds, rm.rd[ks] + m2 * 32 * kRowBytes);
        dp[m2] = mfma32(ad, vreg[ks], dp[m2]);
      }

    bf16x8 pk[2][2], dsk[2][2];
#pragma unroll
    for (int m2 = 0; m2 < 2; ++m2) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const f32x4 l4 = *reinterpret_cast<const f32x4*>(st_lds + 32 * m2 + 8 * g + 4 * h);
        const f32x4 d4 = *reinterpret_cast<const f32x4*>(st_lds + kSlab + 32 * m2 + 8 * g + 4 * h);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const float pv = fast_exp2(__builtin_fmaf(s[m2][4 * g + e], c, -l4[e]));
          s[m2][4 * g + e] = pv;
          dp[m2][4 * g + e] = pv * (dp[m2][4 * g + e] - d4[e]);
        }
      }
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        pk[m2][j] = pack8(s[m2][8 * j + 0], s[m2][8 * j + 1], s[m2][8 * j + 2], s[m2][8 * j + 3], s[m2][8 * j + 4],
                          s[m2][8 * j + 5], s[m2][8 * j + 6], s[m2][8 * j + 7]);
        dsk[m2][j] = pack8(dp[m2][8 * j + 0], dp[m2][8 * j + 1], dp[m2][8 * j + 2], dp[m2][8 * j + 3], dp[m2][8 * j + 4],
                           dp[m2][8 * j + 5], dp[m2][8 * j + 6], dp[m2][8 * j + 7]);
      }
    }

#pragma unroll
    for (int mb = 0; mb < 4; ++mb)
#pragma unroll
      for (int m2 = 0; m2 < 2; ++m2)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          const int roff = (32 * m2 + 16 * j) * kRowBytes;
          const bf16x8 adv = cat(lds_read_tr(do_lds, tr.rd[mb][0] + roff), lds_read_tr(do_lds, tr.rd[mb][1] + roff));
          acc_v[mb] = mfma32(adv, pk[m2][j], acc_v[mb]);
          const bf16x8 adk = cat(lds_read_tr(q_lds, tr.rd[mb][0] + roff), lds_read_tr(q_lds, tr.rd[mb][1] + roff));
          acc_k[mb] = mfma32(adk, dsk[m2][j], acc_k[mb]);
        }

    if (more) stash(nxt);
    __syncthreads();
  }

  __bf16* dkrow = p.dk + (krow0 + l32) * kHeadDim;
  __bf16* dvrow = p.dv + (krow0 + l32) * kHeadDim;
#pragma unroll
  for (int mb = 0; mb < 4; ++mb)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const bf16x4 kv = pack4(acc_k[mb][4 * g + 0] * p.scale, acc_k[mb][4 * g + 1] * p.scale, acc_k[mb][4 * g + 2] * p.scale,
                              acc_k[mb][4 * g + 3] * p.scale);
      const bf16x4 vv = pack4(acc_v[mb][4 * g + 0], acc_v[mb][4 * g + 1], acc_v[mb][4 * g + 2], acc_v[mb][4 * g + 3]);
      *reinterpret_cast<bf16x4*>(dkrow + 32 * mb + 8 * g + 4 * h) = kv;
      *reinterpret_cast<bf16x4*>(dvrow + 32 * mb + 8 * g + 4 * h) = vv;
    }
}

hipError_t launch_bwd_dq(BwdParams p, hipStream_t stream) {
  constexpr int kSmem = 2 * 2 * 64 * kRowBytes;
  p.num_items = p.B * p.Hq * (p.Sq / 128);
  p.items_per_xcd = (p.num_items + kNumXcd - 1) / kNumXcd;
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&dq_kernel), hipFuncAttributeMaxDynamicSharedMemorySize, kSmem);
  if (e != hipSuccess) return e;
  hipLaunchKernelGGL(dq_kernel, dim3(p.items_per_xcd * kNumXcd), dim3(256), kSmem, stream, p);
  return hipGetLastError();
}

hipError_t launch_bwd_dkdv(BwdParams p, hipStream_t stream) {
  constexpr int kSmem = 2 * (2 * 64 * kRowBytes + 2 * 64 * 4);
  p.num_items = p.B * p.Hkv * (p.Skv / 128);
  p.items_per_xcd = (p.num_items + kNumXcd - 1) / kNumXcd;
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&dkdv_kernel), hipFuncAttributeMaxDynamicSharedMemorySize, kSmem);
  if (e != hipSuccess) return e;
  hipLaunchKernelGGL(dkdv_kernel, dim3(p.items_per_xcd * kNumXcd), dim3(256), kSmem, stream, p);
  return hipGetLastError();
}

}  // namespace fba
