// Backward, dK and dV: gfx950, head_dim 128, bf16 in / fp32 accumulate / bf16 out, no atomics.
//
// With P = exp(S/sqrt(D) - LSE), delta = rowsum(dO o O), dP = dO V^T, dS = P o (dP - delta) / sqrt(D):
//   dV = P^T dO,  dK = dS^T Q                   (reference: flex_block_attn_h100.cu:498-537)
// The reference accumulates dK and dV per CTA and adds them into fp32 buffers with reducing stores (:556, :566).  Here a
// key-major kernel owns its dK / dV rows: it walks the per-key-block lists of every query head of the GQA group and
// writes each output element once.
//
// Work-group = 128 key rows of one (batch, kv head), wave = 32 keys, lane = key:
//   S = Q K^T, dP = dO V^T             A = Q / dO slab rows from LDS (128-bit fetches), B = K / V in registers
//   P = exp2(c S - lse2[q]),  dS = P o (dP - delta[q])          (lse2, delta per accumulator row, read from LDS)
//   dV^T += dO^T P,  dK^T += Q^T dS    A = dO / Q slab through transposing LDS fetches, B = P / dS packed to bf16
// Software pipeline over 32-query slabs: while the VALU turns (S_t, dP_t) into P_t and dS_t, the matrix pipe computes
// S_{t+1} and dP_{t+1}; the dV / dK updates of slab t follow.  Q, dO and the two statistics travel global -> LDS
// directly into a ring of four (Q | dO | lse2 | delta) buffers; slab t+4 is requested when slab t is dead.
#include <type_traits>

#include "fba_common.h"
#include "fba_kernels.h"

namespace fba {

namespace {

constexpr int kSlab = 32;
constexpr int kSlabBytes = kSlab * kRowBytes;       // 8 KiB
constexpr int kStatBytes = 2 * kSlab * 4;           // lse2[32] | delta[32]
constexpr int kStageBytes = 2 * kSlabBytes + kStatBytes;
constexpr int kRing = 4;

template <int N>
using IC = std::integral_constant<int, N>;

// ring slot of a step: a compile-time constant in the unrolled loop, a run-time value in the rolled one
template <int N>
FBA_DEVICE constexpr int ring_of(IC<N>) { return N; }
FBA_DEVICE int ring_of(int r) { return r; }

}  // namespace

// kTiled = false: q_block and k_block are multiples of 128; list entries are query blocks, expanded to q_block/32 slabs.
// kTiled = true: tile lists; list entries are 32-row query slabs with a predicate per (wave, 16-row half-slab).
template <bool kTiled>
__global__ __attribute__((amdgpu_flat_work_group_size(256, 256))) void dkdv_kernel(const BwdParams p) {
  extern __shared__ __attribute__((aligned(16))) char smem[];  // ring [4] of (Q slab | dO slab | lse2 | delta)
  constexpr int TK = 128;

  const int tid = threadIdx.x, lane = tid & 63, l32 = lane & 31, h = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int item = xcd_remap(blockIdx.x, p.items_per_xcd);
  if (item >= p.num_items) return;
  const int tiles_per_head = p.Skv / TK;
  const int bhk = item / tiles_per_head;
  const int kt = item - bhk * tiles_per_head;
  const int b = bhk / p.Hkv, hkv = bhk - b * p.Hkv;
  const int group = p.Hq / p.Hkv;
  const int kblk = (kt * TK) / p.k_block;

  // K and V as B operands: lane holds key row l32, d = 16 ks + 8 h .. +7
  const int64_t krow0 = (int64_t)bhk * p.Skv + (int64_t)kt * TK + wave * 32;
  bf16x8 kreg[8], vreg[8];
#pragma unroll
  for (int ks = 0; ks < 8; ++ks) {
    kreg[ks] = *reinterpret_cast<const bf16x8*>(p.k + (krow0 + l32) * kHeadDim + 16 * ks + 8 * h);
    vreg[ks] = *reinterpret_cast<const bf16x8*>(p.v + (krow0 + l32) * kHeadDim + 16 * ks + 8 * h);
  }

  const int nsub = kTiled ? 1 : p.q_block / kSlab;
  const int row_len = kTiled ? p.Sq / kSlab : p.nQ;  // entries per list row
  auto list_row = [&](int g) -> int64_t {
    const int64_t bh = (int64_t)b * p.Hq + hkv * group + g;
    return (p.mask_bh == 1 ? 0 : bh) * (kTiled ? tiles_per_head : p.nK) + (kTiled ? kt : kblk);
  };
  const ConstIdx k_cnt = const_idx(p.k_cnt);
  int nsteps = 0;
  for (int g = 0; g < group; ++g) nsteps += k_cnt[list_row(g)];
  nsteps *= nsub;

  RowMajorOffsets rm;
  rm.init(lane);
  TransposedOffsets tr;
  tr.init(lane);
  SlabDma dma;
  dma.init(wave, lane);
  const uint32_t ring_dst = lds_addr(smem);
  const int64_t rows_total = (int64_t)p.B * p.Hq * p.Sq;
  // statistics copy: lanes 0..31 fetch lse2[row0 + l], lanes 32..63 fetch delta[row0 + l - 32]
  const uint32_t stat_off = (uint32_t)((lane >> 5) * rows_total * 4 + (lane & 31) * 4);
  const float c = p.scale_log2e;

  f32x16 acc_k[4], acc_v[4];
#pragma unroll
  for (int mb = 0; mb < 4; ++mb)
#pragma unroll
    for (int r = 0; r < 16; ++r) { acc_k[mb][r] = 0.f; acc_v[mb][r] = 0.f; }

  // Cursor over (query head of the group, list entry, slab): first query row of the next slab to request.
  const char* qbase = reinterpret_cast<const char*>(p.q);
  const char* dobase = reinterpret_cast<const char*>(p.d_o);
  const char* stbase = reinterpret_cast<const char*>(p.stats);
  int g_cur = -1, e_cur = 0, cnt_cur = 0, rem = 1;
  bool more = true;  // false once every listed slab has been requested; row_next then stays on the last one
  ConstIdx idx_cur = nullptr;
  int64_t row_next = 0, head_row0 = 0;
  auto next_block = [&]() {  // position row_next on the first row of the next listed query block, if any
    ++e_cur;
    while (e_cur >= cnt_cur) {
      if (++g_cur >= group) { more = false; return; }
      const int64_t lr = list_row(g_cur);
      cnt_cur = k_cnt[lr];
      idx_cur = const_idx(p.k_idx + lr * row_len);
      head_row0 = ((int64_t)b * p.Hq + hkv * group + g_cur) * p.Sq;
      e_cur = 0;
    }
    row_next = head_row0 + (kTiled ? (int64_t)(idx_cur[e_cur] >> 8) * kSlab : (int64_t)idx_cur[e_cur] * p.q_block);
    rem = nsub;
  };
  // Five copies per wave request one slab (Q rows, dO rows, statistics).  Every step issues them, so that the count of
  // copies in flight is the same at every wait; once the lists are exhausted the last slab is simply requested again,
  // into a buffer nobody reads any more.
  auto issue_copy = [&](int ring, int64_t row) {
    const uint32_t dst = ring_dst + ring * kStageBytes;
    dma.copy(dst, qbase + row * kRowBytes);
    dma.copy(dst + kSlabBytes, dobase + row * kRowBytes);
    dma4(dst + 2 * kSlabBytes, stbase + row * 4, stat_off);  // every wave copies the same 256 bytes
  };
  auto advance = [&]() {
    if (!more) return;
    if (--rem == 0) next_block(); else row_next += kSlab;
  };

  // Operand registers of one slab's S and dP products: the 16 row-major fetches (Q rows, dO rows)
  struct ScoreOps {
    bf16x8 q[8], d[8];
  };
  auto fetch_score_ops = [&](const char* stage, ScoreOps& o) {
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) {
      o.q[ks] = lds_read_b128(stage, rm.rd[ks]);
      o.d[ks] = lds_read_b128(stage + kSlabBytes, rm.rd[ks]);
    }
  };
  // S and dP of one slab: 16 MFMAs, the two chains interleaved
  auto scores = [&](const ScoreOps& o, f32x16& s, f32x16& dp) {
#pragma unroll
    for (int r = 0; r < 16; ++r) { s[r] = 0.f; dp[r] = 0.f; }
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) {
      s = mfma32(o.q[ks], kreg[ks], s);
      dp = mfma32(o.d[ks], vreg[ks], dp);
    }
  };

  if (nsteps > 0) {
    e_cur = -1;
    next_block();
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      issue_copy(j, row_next);
      advance();
    }
    wait_vmem<0>();
    __syncthreads();
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) {  // loop-invariant matrix operands live in the accumulation register file
      asm volatile("" : "+a"(kreg[ks]));
      asm volatile("" : "+a"(vreg[ks]));
    }
    ScoreOps ops;
    f32x16 s_cur, dp_cur;
    fetch_score_ops(smem, ops);
    scores(ops, s_cur, dp_cur);
    fetch_score_ops(smem + kStageBytes, ops);  // a single slab: whatever the second buffer holds, never used
    // statistics of the slab whose P and dS come next: accumulator element 4g + e of half-wave h is query row 8g + 4h + e
    f32x4 l4[4], d4[4];
    auto fetch_stats = [&](const char* stage) {
      const float* st_lds = reinterpret_cast<const float*>(stage + 2 * kSlabBytes);
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        l4[g] = *reinterpret_cast<const f32x4*>(st_lds + 8 * g + 4 * h);
        d4[g] = *reinterpret_cast<const f32x4*>(st_lds + kSlab + 8 * g + 4 * h);
      }
    };
    fetch_stats(smem);
    // tile lists: predicate bits of the slab being computed, from a second walk over the same lists
    int g_cmp = -1, e_cmp = 0, cnt_cmp = 0, bits_cmp = 0;
    ConstIdx idx_cmp = nullptr;
    auto next_bits = [&]() {
      ++e_cmp;
      while (e_cmp >= cnt_cmp) {
        if (++g_cmp >= group) { bits_cmp = 0; return; }
        const int64_t lr = list_row(g_cmp);
        cnt_cmp = k_cnt[lr];
        idx_cmp = const_idx(p.k_idx + lr * row_len);
        e_cmp = 0;
      }
      bits_cmp = idx_cmp[e_cmp] & 255;
    };
    if constexpr (kTiled) {
      e_cmp = -1;
      next_bits();
    }

    // Step t (ring slot R = t % 4), entered with (S_t, dP_t) in s_cur / dp_cur and the operands of S_{t+1}, dP_{t+1} in
    // `ops`.  First half: the matrix pipe computes S_{t+1}, dP_{t+1} while the VALU turns (S_t, dP_t) into P_t, dS_t and
    // the transposed operands of slab t are fetched.  Slab t is dead after that: barrier, request slab t+4 into its
    // buffer.  Second half: dV += dO_t^T P_t, dK += Q_t^T dS_t while the operands of slab t+2 are fetched.
    auto step = [&](auto ring_c, int t) {
      const int R = ring_of(ring_c);
      const char* stage = smem + R * kStageBytes;
      bf16x8 adv[2][4], adk[2][4];
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int mb = 0; mb < 4; ++mb) {
          const int roff = 16 * j * kRowBytes;
          adv[j][mb] = cat(lds_read_tr(stage + kSlabBytes, tr.rd[mb][0] + roff), lds_read_tr(stage + kSlabBytes, tr.rd[mb][1] + roff));
          adk[j][mb] = cat(lds_read_tr(stage, tr.rd[mb][0] + roff), lds_read_tr(stage, tr.rd[mb][1] + roff));
        }
      f32x16 s_nxt, dp_nxt;
      scores(ops, s_nxt, dp_nxt);  // past the last slab: stale data, unused
      // does this wave's key block select the first / second 16 query rows of the slab?
      const bool on0 = !kTiled || ((bits_cmp >> (2 * wave)) & 1) != 0;
      const bool on1 = !kTiled || ((bits_cmp >> (2 * wave + 1)) & 1) != 0;
#pragma unroll
      for (int g = 0; g < 4; ++g)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          float pv = fast_exp2(__builtin_fmaf(s_cur[4 * g + e], c, -l4[g][e]));
          if constexpr (kTiled) pv = (g < 2 ? on0 : on1) ? pv : 0.f;  // a select: inf or NaN of a masked row is discarded
          s_cur[4 * g + e] = pv;
          dp_cur[4 * g + e] = pv * (dp_cur[4 * g + e] - d4[g][e]);
        }
      bf16x8 pk[2], dsk[2];
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        pk[j] = pack8(s_cur[8 * j + 0], s_cur[8 * j + 1], s_cur[8 * j + 2], s_cur[8 * j + 3], s_cur[8 * j + 4],
                      s_cur[8 * j + 5], s_cur[8 * j + 6], s_cur[8 * j + 7]);
        dsk[j] = pack8(dp_cur[8 * j + 0], dp_cur[8 * j + 1], dp_cur[8 * j + 2], dp_cur[8 * j + 3], dp_cur[8 * j + 4],
                       dp_cur[8 * j + 5], dp_cur[8 * j + 6], dp_cur[8 * j + 7]);
      }
#pragma unroll
      for (int j = 0; j < 2; ++j) { pin(pk[j]); pin(dsk[j]); }  // computed here, not next to their use after the barrier
      // issue order of this half, sixteen times: one matrix instruction, two of the 32 transposing fetches, five of the 80
      // vector instructions.  A wave can have 15 LDS fetches in flight at most (the counter is four bits wide), so fetches
      // are spread between the matrix instructions instead of being issued in one batch that would block the wave.
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
        __builtin_amdgcn_sched_group_barrier(0x002, kTiled ? 6 : 5, 0);
      }
      if constexpr (kTiled) next_bits();
      __builtin_amdgcn_sched_barrier(0);
      // slab t+2 must have landed (its operands are fetched below); the five copies of slab t+3 may still fly
      wait_vmem<5>();
      __syncthreads();
      const int64_t row_copy = row_next;  // slab t+4
      advance();
      fetch_score_ops(smem + ((R + 2) & 3) * kStageBytes, ops);
      fetch_stats(smem + ((R + 1) & 3) * kStageBytes);
#pragma unroll
      for (int j = 0; j < 2; ++j) {
#pragma unroll
        for (int mb = 0; mb < 4; ++mb) {
          acc_v[mb] = mfma32(adv[j][mb], pk[j], acc_v[mb]);
          acc_k[mb] = mfma32(adk[j][mb], dsk[j], acc_k[mb]);
        }
        if (j == 0) issue_copy(R, row_copy);  // behind eight queued products, not in front of them
      }
      s_cur = s_nxt;
      dp_cur = dp_nxt;
      pin(s_cur);  // the moves out of the accumulation registers happen here, under the products above
      pin(dp_cur);
#pragma unroll
      for (int i = 0; i < 8; ++i) {  // the 24 fetches: two after each of the first eight matrix instructions, then one
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 1);
        __builtin_amdgcn_sched_group_barrier(0x100, 2, 1);
        __builtin_amdgcn_sched_group_barrier(0x002, 2, 1);
      }
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 1);
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 1);
        __builtin_amdgcn_sched_group_barrier(0x002, 2, 1);
      }
      __builtin_amdgcn_sched_barrier(0);
    };
    if constexpr (kTiled) {
      for (int t = 0; t < nsteps; ++t) step(t & 3, t);  // any step count; ring slot computed at run time
    } else {
      for (int t = 0; t < nsteps; t += 4) {  // nsteps is a multiple of 4
        step(IC<0>{}, t);
        step(IC<1>{}, t + 1);
        step(IC<2>{}, t + 2);
        step(IC<3>{}, t + 3);
      }
    }
    wait_vmem<0>();  // no copy may still be writing this work-group's LDS when it ends
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

hipError_t launch_bwd_dkdv(BwdParams p, hipStream_t stream) {
  constexpr int kSmem = kRing * kStageBytes;
  p.num_items = p.B * p.Hkv * (p.Skv / 128);
  p.items_per_xcd = (p.num_items + kNumXcd - 1) / kNumXcd;
  const void* fn = p.tiled ? reinterpret_cast<const void*>(&dkdv_kernel<true>) : reinterpret_cast<const void*>(&dkdv_kernel<false>);
  hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, kSmem);
  if (e != hipSuccess) return e;
  if (p.tiled)
    hipLaunchKernelGGL(dkdv_kernel<true>, dim3(p.items_per_xcd * kNumXcd), dim3(256), kSmem, stream, p);
  else
    hipLaunchKernelGGL(dkdv_kernel<false>, dim3(p.items_per_xcd * kNumXcd), dim3(256), kSmem, stream, p);
  return hipGetLastError();
}

}  // namespace fba
