// Forward kernel: block-sparse softmax attention for gfx950, head_dim 128, bf16 in / fp32 accumulate.
//
// One work-group of 4 waves owns 128 consecutive query rows of one (batch, head); wave w owns rows [32w, 32w+32).
// The work-group walks the active-key-block list of its query block and streams every selected key block through
// LDS as 32-key slabs of K and V (a ring of four 8 KiB buffers each).
//
// Everything is kept "transposed" so that softmax statistics are per-lane scalars (lane = query row):
//   S^T[key, q]  = K[key, :] . Q[q, :]            A = K slab rows from LDS (128-bit fetches), B = Q in registers
//   P^T          = exp2(c * S^T - c * m[q])        fp32, c = log2(e) / sqrt(128); running reference m and sum l per lane
//   O^T[d, q]   += V^T[d, key] . P^T[key, q]       A = V slab through transposing LDS fetches, B = P^T packed to bf16
// The reference computes the same quantities per selected tile (flex_block_attn_h100.cu:245-290, online softmax
// :199-221, final O / l at :292); here LSE is stored as the natural-log value m/sqrt(128) + ln(l).
//
// Software pipeline.  The unit of work is a 32-key slab t.  While the VALU turns S_t into P_t, the matrix pipe computes
// S_{t+1} and adds P_{t-1} V_{t-1} into O; the three are independent, so one wave keeps both pipes busy.
// K and V slabs travel global -> LDS directly (no registers) into two rings of four 8 KiB buffers: after step t the
// buffers of K_{t+1} and V_{t-1} are dead and receive K_{t+5} and V_{t+3}, i.e. every slab is requested four steps
// before its first use.  One barrier per step orders all LDS traffic; before it each wave waits until its own copies
// of the slabs needed next have landed (all but the two youngest batches of four).
#include <type_traits>

#include "fba_common.h"
#include "fba_kernels.h"

namespace fba {

namespace {

constexpr int kSlab = 32;                      // keys per LDS slab
constexpr int kSlabBytes = kSlab * kRowBytes;  // 8 KiB
constexpr int kRing = 4;                       // slabs per ring
constexpr float kLazy = 8.f;                   // log2 headroom before the softmax reference is raised
constexpr int kFwdSlotBytes = (128 * kHeadDim + 2 * 128) * 4;  // partial result of one part of a split item

template <int N>
using IC = std::integral_constant<int, N>;

struct FwdState {
  bf16x8 qreg[8];
  f32x16 acc_o[4];
  float l_run;  // sum over the keys this half-wave has seen of bf16(P) for the lane's query row
  float m_run;
  RowMajorOffsets rm;
  TransposedOffsets tr;
  float c;
};

// S^T for 32 keys: 8 MFMAs.  k_half points at the first of the 32 key rows inside a swizzled slab.
FBA_DEVICE f32x16 qk_half(const FwdState& st, const char* k_half) {
  f32x16 s;
#pragma unroll
  for (int r = 0; r < 16; ++r) s[r] = 0.f;
#pragma unroll
  for (int ks = 0; ks < 8; ++ks) s = mfma32(lds_read_b128(k_half, st.rm.rd[ks]), st.qreg[ks], s);
  return s;
}

// O^T += V^T P^T for 32 keys: 8 MFMAs; consecutive MFMAs go to different accumulators.  `between(i)` runs behind matrix
// instruction i: the place for the global -> LDS copies a step owes, which take a wave tens of cycles each to issue.
template <typename Between>
FBA_DEVICE void pv_half(FwdState& st, const char* v_half, const bf16x8 (&pk)[2], Between between) {
#pragma unroll
  for (int j = 0; j < 2; ++j) {
#pragma unroll
    for (int mb = 0; mb < 4; ++mb) {
      const int roff = 16 * j * kRowBytes;
      const bf16x8 a = cat(lds_read_tr(v_half, st.tr.rd[mb][0] + roff), lds_read_tr(v_half, st.tr.rd[mb][1] + roff));
      st.acc_o[mb] = mfma32(a, pk[j], st.acc_o[mb]);
      between(4 * j + mb);
    }
  }
}
FBA_DEVICE void pv_half(FwdState& st, const char* v_half, const bf16x8 (&pk)[2]) {
  pv_half(st, v_half, pk, [](int) {});
}

// Raise the softmax reference if some row of the wave would otherwise see exponents above kLazy.  Until then
// P = exp2(c (S - m)) may exceed 1, which fp32 sums and bf16 P both carry.
// `active` is false for a query row whose own mask block does not select the current key block (tile lists only).
FBA_DEVICE void softmax_reference(FwdState& st, const f32x16& s, bool active) {
  float mx = s[0];
#pragma unroll
  for (int r = 1; r < 16; ++r) mx = fmaxf(mx, s[r]);
  mx = active ? mx : -INFINITY;
  // every half-wave tests the 16 keys it holds; the row maximum over both halves is formed only when the reference rises
  if (__builtin_amdgcn_ballot_w64((mx - st.m_run) * st.c > kLazy) != 0) {
    const float m_new = fmaxf(st.m_run, max_halves(mx));
    const float alpha = fast_exp2((st.m_run - m_new) * st.c);
    st.m_run = m_new;
    st.l_run *= alpha;
#pragma unroll
    for (int mb = 0; mb < 4; ++mb)
#pragma unroll
      for (int r = 0; r < 16; ++r) st.acc_o[mb][r] *= alpha;
  }
}

// P^T = exp2(c S^T - c m), packed to bf16 as the B operand of the two 16-key MFMA steps.
template <bool kTiled>
FBA_DEVICE void softmax_exp(FwdState& st, f32x16& s, bf16x8 (&pk)[2], bool active) {
  const float mc = st.m_run * st.c;
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    s[r] = fast_exp2(__builtin_fmaf(s[r], st.c, -mc));
    if constexpr (kTiled) s[r] = active ? s[r] : 0.f;
  }
#pragma unroll
  for (int j = 0; j < 2; ++j)
    pk[j] = pack8(s[8 * j + 0], s[8 * j + 1], s[8 * j + 2], s[8 * j + 3], s[8 * j + 4], s[8 * j + 5], s[8 * j + 6], s[8 * j + 7]);
  // denominator: the sum of the same bf16 P that weighs V, two values per dot-product instruction
  const bf16x2 one2 = {(__bf16)1.f, (__bf16)1.f};
#pragma unroll
  for (int j = 0; j < 2; ++j)
#pragma unroll
    for (int t = 0; t < 4; ++t)
      st.l_run = __builtin_amdgcn_fdot2_f32_bf16((bf16x2){pk[j][2 * t], pk[j][2 * t + 1]}, one2, st.l_run, false);
}

}  // namespace

// kTiled = false: q_block is a multiple of 128, the list of a work-group is the block list of its query block.
// kTiled = true: tile lists with a predicate per 16-row group (any q_block that is a multiple of 16).
// kWaves = 4: 128 query rows per work-group, two work-groups per CU.  kWaves = 12 (q_block a multiple of 384, block
// lists): 384 rows, one work-group per CU with three waves per SIMD; every K / V slab brought into LDS then feeds three
// times as many matrix instructions (the reference shares its K / V tiles between three consumer groups for the same
// reason, flex_block_attn_h100.cu:912-928).
template <bool kTiled, int kWaves>
__global__ __attribute__((amdgpu_flat_work_group_size(64 * kWaves, 64 * kWaves), amdgpu_waves_per_eu(kWaves == 12 ? 3 : 2, kWaves == 12 ? 3 : 2))) void fwd_kernel(const FwdParams p) {
  extern __shared__ __attribute__((aligned(16))) char smem[];  // K ring [4][8 KiB] | V ring [4][8 KiB]
  constexpr int TQ = 32 * kWaves;
  static_assert(!kTiled || kWaves == 4, "tile lists describe 128-row tiles");

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
  const __bf16* qp = p.q + qrow0 * kHeadDim;
  const char* kp = reinterpret_cast<const char*>(p.k + ((int64_t)(b * p.Hkv + hkv) * p.Skv) * kHeadDim);
  const char* vp = reinterpret_cast<const char*>(p.v + ((int64_t)(b * p.Hkv + hkv) * p.Skv) * kHeadDim);

  const int64_t mrow = (p.mask_bh == 1 ? 0 : (int64_t)bh) * (kTiled ? tiles_per_head : p.nQ) + (kTiled ? qt : (qt * TQ) / p.q_block);
  const int cnt = p.q_cnt[mrow];
  const ConstIdx idx = const_idx(p.q_idx + mrow * p.nK);
  auto key_block = [&](int e) -> int { return kTiled ? idx[e] >> 8 : idx[e]; };
  // predicate bit of this lane's 16-row group in a tile-list entry
  const int group_bit = 1 << (2 * wave + (l32 >> 4));
  const int nsub = p.k_block / kSlab;
  // this work-group's range of 32-key steps of the list: all of it, or part `part` of `parts` (even boundaries)
  const int steps_all = cnt * nsub;
  const int t_begin = parts == 1 ? 0 : 2 * (int)(((int64_t)(steps_all / 2) * part) / parts);
  const int t_end = parts == 1 ? steps_all : 2 * (int)(((int64_t)(steps_all / 2) * (part + 1)) / parts);
  const int nsteps = t_end - t_begin;
  const int e_begin = t_begin / nsub, sub_begin = t_begin - e_begin * nsub;

  FwdState st;
  // Q as the B operand: lane holds row l32, d = 16 ks + 8 h .. +7
#pragma unroll
  for (int ks = 0; ks < 8; ++ks) st.qreg[ks] = *reinterpret_cast<const bf16x8*>(qp + (int64_t)l32 * kHeadDim + 16 * ks + 8 * h);
  st.rm.init(lane);
  st.tr.init(lane);
  st.c = p.scale_log2e;
  st.m_run = kTiled ? -1e30f : -INFINITY;  // finite where whole slabs can be masked out, so that exp2 never sees inf - inf
  st.l_run = 0.f;
#pragma unroll
  for (int mb = 0; mb < 4; ++mb)
#pragma unroll
    for (int r = 0; r < 16; ++r) st.acc_o[mb][r] = 0.f;

  SlabDmaShared<kWaves> dma;
  dma.init(wave, lane);
  char* const k_lds = smem;
  char* const v_lds = smem + kRing * kSlabBytes;
  const uint32_t k_dst = lds_addr(k_lds);
  const uint32_t v_dst = lds_addr(v_lds);

  // Slab source offsets, in list order.  The list entry of the following key block is read one block ahead, so that
  // the scalar load is off the critical path.  V requests trail K requests by two slabs and reuse their offsets.
  const int64_t block_bytes = (int64_t)p.k_block * kRowBytes;
  int e_next = e_begin + 1, rem = nsub - sub_begin;
  int64_t src_off = nsteps > 0 ? key_block(e_begin) * block_bytes + (int64_t)sub_begin * kSlabBytes : 0;
  int blk_next = e_next < cnt ? key_block(e_next) : 0;
  auto next_off = [&]() -> int64_t {
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
  // K slabs and V slabs are brought in by different (overlapping, for 12 waves) sets of waves
  auto copy_k = [&](uint32_t dst, const char* src) { dma.copy_k(dst, src); };
  auto copy_v = [&](uint32_t dst, const char* src) { dma.copy_v(dst, src); };

  if (nsteps > 0) {
    // prologue: K_0..K_3 and V_0..V_2 requested, S_0 computed, then K_4 into the buffer of K_0
    int64_t off[5] = {0, 0, 0, 0, 0};
#pragma unroll
    for (int j = 0; j < 4; ++j)
      if (j < nsteps) {
        off[j] = next_off();
        copy_k(k_dst + j * kSlabBytes, kp + off[j]);
      }
#pragma unroll
    for (int j = 0; j < 3; ++j)
      if (j < nsteps) copy_v(v_dst + j * kSlabBytes, vp + off[j]);
    wait_vmem<0>();
    __syncthreads();
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) pin(st.qreg[ks]);
    f32x16 s_cur = qk_half(st, k_lds);
    pin(s_cur);
    __syncthreads();
    if (4 < nsteps) {
      off[4] = next_off();
      copy_k(k_dst, kp + off[4]);
    }
    int64_t hist0 = off[4], hist1 = off[3];  // offsets of the two youngest K requests

    bf16x8 p_prev[2];
    // predicate of the slab whose softmax is next (tile lists): all 16-row groups share the entry, each lane tests its bit
    int e_cmp = e_begin, rem_cmp = nsub - sub_begin;
    int bits_cmp = kTiled ? idx[e_begin] & 255 : 255;
    int bits_ahead = kTiled && e_begin + 1 < cnt ? idx[e_begin + 1] & 255 : 0;  // predicate bits of the following list entry
    // A wave whose two 16-row groups are both switched off for a slab leaves that slab's matrix work out altogether
    // (wave-uniform branches); rows switched off inside an active wave are dealt with by selects.
    const int wave_bits = 3 << (2 * wave);
    bool w_prev = false;  // did this wave form P for the previous slab?
    // The copies a step requests (K_{t+5} into the buffer of K_{t+1}, V_{t+3} into that of V_{t-1}, both free behind the
    // step's barrier) are issued by the following step, in between its first matrix instructions where the work-group
    // has block lists and four waves: a copy takes a wave tens of cycles to issue, which the matrix pipe then covers.
    // Every step requests both, so that the counter of copies in flight means the same thing at every wait; past the end
    // of the list they repeat a listed slab into a buffer that nobody reads any more.
    uint32_t owed_k_dst = 0, owed_v_dst = 0;
    const char* owed_k_src = kp;
    const char* owed_v_src = vp;
    bool owed = false;
    constexpr bool kSpread = !kTiled && kWaves == 4;

    // step t (t % 4 == R): O += P_{t-1} V_{t-1} | softmax(S_t) | S_{t+1} = K_{t+1} Q^T
    auto step = [&](auto ring_c, auto first_c, int t) {
      constexpr int R = decltype(ring_c)::value;
      constexpr bool kFirst = decltype(first_c)::value;
      const bool w_cur = !kTiled || (bits_cmp & wave_bits) != 0;
      const bool w_nxt = !kTiled || ((rem_cmp > 1 ? bits_cmp : bits_ahead) & wave_bits) != 0;
      // P_{t-1} was formed against the reference m of step t-1, so it must reach O before step t may raise m
      if constexpr (kSpread && !kFirst) {
        pv_half(st, v_lds + ((R + 3) & 3) * kSlabBytes, p_prev, [&](int i) {
          if (i == 0) dma.copy_piece(0, owed_k_dst, owed_k_src);
          if (i == 2) dma.copy_piece(1, owed_k_dst, owed_k_src);
          if (i == 4) dma.copy_piece(0, owed_v_dst, owed_v_src);
          if (i == 6) dma.copy_piece(1, owed_v_dst, owed_v_src);
        });
      } else {
        if (owed) {
          copy_k(owed_k_dst, owed_k_src);
          copy_v(owed_v_dst, owed_v_src);
        }
        if constexpr (!kFirst) {
          if (w_prev) pv_half(st, v_lds + ((R + 3) & 3) * kSlabBytes, p_prev);
        }
      }
      const bool active = !kTiled || (bits_cmp & group_bit) != 0;
      if (w_cur) softmax_reference(st, s_cur, active);
      f32x16 s_nxt;
      if (w_nxt) s_nxt = qk_half(st, k_lds + ((R + 1) & 3) * kSlabBytes);  // past the last slab: stale data, unused
      else s_nxt = s_cur;
      if (w_cur) softmax_exp<kTiled>(st, s_cur, p_prev, active);  // p_prev := P_t
      w_prev = w_cur;
      if constexpr (kTiled) {
        if (--rem_cmp == 0) {
          rem_cmp = nsub;
          ++e_cmp;
          bits_cmp = bits_ahead;
          bits_ahead = e_cmp + 1 < cnt ? idx[e_cmp + 1] & 255 : 0;
        }
      }
      // P_t is only consumed after the barrier; without the pins its arithmetic sinks there, away from the MFMAs it is
      // meant to overlap with
      pin(p_prev[0]);
      pin(p_prev[1]);
      s_cur = s_nxt;
      // K_{t+2} and V_t must have landed; the copies requested by steps t-2 and t-1 may still fly
      dma.wait_two_steps();
      __syncthreads();
      owed_v_src = vp + hist1;
      owed_v_dst = v_dst + ((R + 3) & 3) * kSlabBytes;
      hist1 = hist0;
      hist0 = next_off();
      owed_k_src = kp + hist0;
      owed_k_dst = k_dst + ((R + 1) & 3) * kSlabBytes;
      owed = true;
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
    // O += P_{n-1} V_{n-1}
    if (w_prev) pv_half(st, v_lds + ((nsteps - 1) & 3) * kSlabBytes, p_prev);
    wait_vmem<0>();  // no copy may still be writing LDS when the work-group gives it back
  }

  const float l = sum_halves(st.l_run);
  if (parts > 1) {
    // part of a split item: unnormalised O^T, the softmax reference in log2 units and the denominator go to the workspace
    float* slot = p.split.ws + ((int64_t)(item - p.split.first) * parts + part) * (kFwdSlotBytes / 4);
    float* prow = slot + (wave * 32 + l32) * kHeadDim;
#pragma unroll
    for (int mb = 0; mb < 4; ++mb)
#pragma unroll
      for (int g = 0; g < 4; ++g)
        *reinterpret_cast<f32x4*>(prow + 32 * mb + 8 * g + 4 * h) =
            (f32x4){st.acc_o[mb][4 * g + 0], st.acc_o[mb][4 * g + 1], st.acc_o[mb][4 * g + 2], st.acc_o[mb][4 * g + 3]};
    if (h == 0) {
      slot[TQ * kHeadDim + wave * 32 + l32] = st.m_run * st.c;
      slot[TQ * kHeadDim + TQ + wave * 32 + l32] = l;
    }
    return;
  }
  // epilogue: O = O^T / l, LSE = ln2 * (c m + log2 l)
  __bf16* orow = p.o + (qrow0 + l32) * kHeadDim;
  const float inv = l > 0.f ? 1.f / l : 0.f;
  if (h == 0) p.lse[qrow0 + l32] = l > 0.f ? (st.m_run * st.c + __builtin_log2f(l)) * 0.6931471805599453f : -INFINITY;
#pragma unroll
  for (int mb = 0; mb < 4; ++mb)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const bf16x4 ov = pack4(st.acc_o[mb][4 * g + 0] * inv, st.acc_o[mb][4 * g + 1] * inv, st.acc_o[mb][4 * g + 2] * inv,
                              st.acc_o[mb][4 * g + 3] * inv);
      *reinterpret_cast<bf16x4*>(orow + 32 * mb + 8 * g + 4 * h) = ov;
    }
}

// Combines the parts of the split items: O = sum_p 2^(m_p - m) O_p / sum_p 2^(m_p - m) l_p with m = max_p m_p, in part
// order.  One thread per (query row, four head-dim columns).
__global__ __attribute__((amdgpu_flat_work_group_size(256, 256))) void fwd_merge_kernel(const FwdParams p) {
  const int tid = threadIdx.x;
  const int row = blockIdx.x * 8 + (tid >> 5), c4 = (tid & 31) * 4;  // row among the 128 * (split items) rows
  const int it = row >> 7, r = row & 127;
  const int item = p.split.first + it;
  const int parts = p.split.parts;
  const float* slot0 = p.split.ws + (int64_t)it * parts * (kFwdSlotBytes / 4);
  float m = -INFINITY;
  for (int q = 0; q < parts; ++q) m = fmaxf(m, slot0[(int64_t)q * (kFwdSlotBytes / 4) + 128 * kHeadDim + r]);
  float l = 0.f;
  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  for (int q = 0; q < parts; ++q) {
    const float* slot = slot0 + (int64_t)q * (kFwdSlotBytes / 4);
    const float mq = slot[128 * kHeadDim + r];
    const float w = mq == -INFINITY ? 0.f : fast_exp2(mq - m);
    l += w * slot[128 * kHeadDim + 128 + r];
    const f32x4 o4 = *reinterpret_cast<const f32x4*>(slot + r * kHeadDim + c4);
    acc += w * o4;
  }
  const float inv = l > 0.f ? 1.f / l : 0.f;
  const int64_t orow = (int64_t)item * 128 + r;  // items are consecutive 128-row tiles of [B, Hq, Sq]
  *reinterpret_cast<bf16x4*>(p.o + orow * kHeadDim + c4) = pack4(acc[0] * inv, acc[1] * inv, acc[2] * inv, acc[3] * inv);
  if (c4 == 0) p.lse[orow] = l > 0.f ? (m + __builtin_log2f(l)) * 0.6931471805599453f : -INFINITY;
}

hipError_t launch_fwd(FwdParams p, hipStream_t stream) {
  constexpr int kSmem = 2 * kRing * kSlabBytes;
  const bool wide = !p.tiled && p.q_block % 384 == 0 && p.variant != 1;
  void (*fn)(const FwdParams) = p.tiled ? &fwd_kernel<true, 4> : wide ? &fwd_kernel<false, 12> : &fwd_kernel<false, 4>;
  const int rows = wide ? 384 : 128;
  p.num_items = p.B * p.Hq * (p.Sq / rows);
  // tail splitting for the 128-row kernels (two work-groups per compute unit)
  p.split = plan_split(p.num_items, 2, kFwdSlotBytes, wide ? nullptr : p.split.ws, p.split_ws_bytes);
  plan_xcd_mapping(p.B * p.Hq, p.split.first, p.items_per_xcd, p.split.main_wgs);
  const int split_wgs = (p.num_items - p.split.first) * p.split.parts;
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(fn), hipFuncAttributeMaxDynamicSharedMemorySize, kSmem);
  if (e != hipSuccess) return e;
  hipLaunchKernelGGL(fn, dim3(p.split.main_wgs + split_wgs), dim3(rows * 2), kSmem, stream, p);
  if (split_wgs > 0) hipLaunchKernelGGL(fwd_merge_kernel, dim3((p.num_items - p.split.first) * 16), dim3(256), 0, stream, p);
  return hipGetLastError();
}

}  // namespace fba
