// Backward, dK and dV: gfx950, head_dim 128, bf16 in / fp32 accumulate / bf16 out, no atomics.
//
// With P = exp(S/sqrt(D) - LSE), delta = rowsum(dO o O), dP = dO V^T, dS = P o (dP - delta) / sqrt(D):
//   dV = P^T dO,  dK = dS^T Q                   (reference: flex_block_attn_h100.cu:498-537)
// The reference accumulates dK and dV per CTA and adds them into fp32 buffers with reducing stores (:556, :566).  Here a
// key-major kernel owns its dK / dV rows: it walks the per-key-block lists of every query head of the GQA group and
// writes each output element once.
//
// Work-group = 128 key rows of one (batch, kv head), eight waves, two per SIMD.  Wave w works on keys 32 (w % 4) ..+31
// and on every second 32-query slab of the list (w / 4 = parity of the slab), lane = key:
//   S = Q K^T, dP = dO V^T             A = Q / dO slab rows, B = K / V rows, all from LDS (128-bit fetches)
//   P = exp2(c S - lse2[q]),  dS = P o (dP - delta[q])          (lse2, -delta per accumulator row, read from LDS; the dP
//                                                               accumulators start from -delta)
//   dV^T += dO^T P,  dK^T += Q^T dS    A = dO / Q slab through transposing LDS fetches, B = P / dS packed to bf16
// The two waves of a key group hold partial sums over their slabs; at the end they swap halves through LDS (one sends
// its dV part and finishes dK, the other the reverse).  Two waves per SIMD keep the matrix pipe busy while one of them
// waits for LDS or runs the softmax; that is why K and V stay in LDS instead of 64 registers per lane.
// LDS: ring of four (Q slab | dO slab | lse2 | -delta) buffers = two slab pairs (while one pair is being worked on, the
// other is in flight global -> LDS), then the K tile and the V tile (32 KiB each).
#include <type_traits>

#include "fba_common.h"
#include "fba_kernels.h"

namespace fba {

namespace {

constexpr int kSlab = 32;
constexpr int kSlabBytes = kSlab * kRowBytes;       // 8 KiB
constexpr int kStatBytes = 2 * kSlab * 4;           // lse2[32] | -delta[32]
constexpr int kStageBytes = 2 * kSlabBytes + kStatBytes;
constexpr int kRing = 4;
constexpr int kTileBytes = 128 * kRowBytes;         // K or V tile, 32 KiB
constexpr int kRingBase = 0;                        // the ring first: its offsets fit the 16-bit field of an LDS fetch
constexpr int kTileBase = kRing * kStageBytes;      // K tile, then V tile
constexpr int kSmemBytes = kTileBase + 2 * kTileBytes;

template <int N>
using IC = std::integral_constant<int, N>;

}  // namespace

// kTiled = false: q_block and k_block are multiples of 128; list entries are query blocks, expanded to q_block/32 slabs.
// kTiled = true: tile lists; list entries are 32-row query slabs with a predicate per (key group, 16-row half-slab).
// kHandOver: every wave also stores the bf16 dS it forms to p.ds_ws (layout: fba_common.h), so that dQ = dS K can be
// formed later without recomputing S and dP.  With tile lists the workspace is divided into (128-row query tile, 128-key
// tile) pairs and a wave that leaves a slab out stores nothing for it.
template <bool kTiled, bool kHandOver>
__global__ __attribute__((amdgpu_flat_work_group_size(512, 512), amdgpu_waves_per_eu(2, 2))) void dkdv_kernel(const BwdParams p) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  constexpr int TK = 128;
  if constexpr (kHandOver) {
    if (!workspace_holds_lists(p)) return;  // the launcher's last launch reports it
  }

  const int tid = threadIdx.x, lane = tid & 63, l32 = lane & 31, h = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int kg = wave & 3, par = wave >> 2;
  // the grid index this work-group works on: its own, or one it claims (a launch with claim counters)
  int grid_index = (int)blockIdx.x;
  if (p.queue != nullptr) {
    volatile int* claimed = reinterpret_cast<volatile int*>(smem + kSmemBytes);  // behind everything the kernel uses
    if (tid == 0) *claimed = claim_work(p.queue, xcd_id(), p.total_work);
    __syncthreads();
    grid_index = __builtin_amdgcn_readfirstlane(*claimed);
    if (grid_index < 0) return;
  }
  // whole items first (dealt to the XCDs in contiguous spans), then the parts of the split items
  int item, part = 0, parts = 1;
  if (grid_index < p.split.main_wgs) {
    item = xcd_remap(grid_index, p.items_per_xcd);
    if (item >= p.split.first) return;
  } else {
    const int s = grid_index - p.split.main_wgs;
    item = p.split.first + s / p.split.parts;
    part = s - (item - p.split.first) * p.split.parts;
    parts = p.split.parts;
  }
  const int tiles_per_head = p.Skv / TK;
  const int bhk = item / tiles_per_head;
  const int kt = item - bhk * tiles_per_head;
  const int b = bhk / p.Hkv, hkv = bhk - b * p.Hkv;
  const int group = p.Hq / p.Hkv;
  const int kblk = (kt * TK) / p.k_block;
  const int64_t krow0 = (int64_t)bhk * p.Skv + (int64_t)kt * TK;

  const int nsub = kTiled ? 1 : p.q_block / kSlab;
  const int row_len = kTiled ? p.Sq / kSlab : p.nQ;  // entries per list row
  auto list_row = [&](int g) -> int64_t {
    const int64_t bh = (int64_t)b * p.Hq + hkv * group + g;
    return (p.mask_bh == 1 ? 0 : bh) * (kTiled ? tiles_per_head : p.nK) + (kTiled ? kt : kblk);
  };
  const ConstIdx k_cnt = const_idx(p.k_cnt);
  int slabs_all = 0;
  for (int g = 0; g < group; ++g) slabs_all += k_cnt[list_row(g)];
  slabs_all *= nsub;
  // this work-group's range of listed slabs: all of them, or part `part` of `parts` (boundaries on multiples of four slabs)
  const int s_begin = parts == 1 ? 0 : 4 * (int)(((int64_t)(slabs_all / 4) * part) / parts);
  // (the last part takes what is left over: with tile lists the number of listed slabs need not be a multiple of four)
  const int nslabs = (part + 1 == parts ? slabs_all : 4 * (int)(((int64_t)(slabs_all / 4) * (part + 1)) / parts)) - s_begin;
  // (query head of the group, list entry, slab inside the query block) of slab s_begin
  int g_begin = 0, e_begin = 0, sub_begin = 0;
  if (parts > 1) {
    int s = s_begin;
    for (; g_begin < group - 1; ++g_begin) {
      const int n = k_cnt[list_row(g_begin)] * nsub;
      if (s < n) break;
      s -= n;
    }
    e_begin = s / nsub;
    sub_begin = s - e_begin * nsub;
  }

  RowMajorOffsets rm;
  rm.init(lane);
  TransposedOffsets tr;
  tr.init(lane);
  SlabDma dma;
  dma.init(kg, lane);
  const uint32_t lds0 = lds_addr(smem);
  const uint32_t ring_dst = lds0 + kRingBase;
  const int64_t rows_total = (int64_t)p.B * p.Hq * p.Sq;
  // statistics copy: lanes 0..31 fetch lse2[row0 + l], lanes 32..63 fetch -delta[row0 + l - 32]
  const uint32_t stat_off = (uint32_t)((lane >> 5) * rows_total * 4 + (lane & 31) * 4);
  const float c = p.scale_log2e;

  f32x16 acc_k[4], acc_v[4];
#pragma unroll
  for (int mb = 0; mb < 4; ++mb)
#pragma unroll
    for (int r = 0; r < 16; ++r) { acc_k[mb][r] = 0.f; acc_v[mb][r] = 0.f; }

  if (nslabs > 0) {
    // K rows by the waves of parity 0, V rows by those of parity 1: four 32-row slabs each
    {
      const char* src = reinterpret_cast<const char*>(par ? p.v : p.k) + krow0 * kRowBytes;
#pragma unroll
      for (int j = 0; j < 4; ++j) dma.copy(lds0 + kTileBase + par * kTileBytes + j * kSlabBytes, src + j * kSlabBytes);
    }
    // Cursor over (query head of the group, list entry, slab): first query row of the next slab to request.
    const char* qbase = reinterpret_cast<const char*>(p.q);
    const char* dobase = reinterpret_cast<const char*>(p.d_o);
    const char* stbase = reinterpret_cast<const char*>(p.stats);
    int g_cur = -1, e_cur = -1, cnt_cur = 0, rem = 1;
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
    auto advance = [&]() {
      if (!more) return;
      if (--rem == 0) next_block(); else row_next += kSlab;
    };
    // Five copies per wave request one slab (Q rows, dO rows, statistics), by the four waves of the slab's parity.  Every
    // step issues them, so that the count of copies in flight is the same at every wait; once the lists are exhausted
    // the last slab is simply requested again, into a buffer nobody reads any more.
    auto issue_copy = [&](int ring, int64_t row) {
      const uint32_t dst = ring_dst + ring * kStageBytes;
      dma.copy(dst, qbase + row * kRowBytes);
      dma.copy(dst + kSlabBytes, dobase + row * kRowBytes);
      dma4(dst + 2 * kSlabBytes, stbase + row * 4, stat_off);  // each of the four waves copies the same 256 bytes
    };
    auto request_pair = [&](int pair_slot) {  // slabs 2i, 2i+1 -> ring buffers 2*pair_slot, 2*pair_slot + 1
      const int64_t r0 = row_next;
      advance();
      const int64_t r1 = row_next;
      advance();
      issue_copy(2 * pair_slot + par, par ? r1 : r0);
    };
    if (parts == 1) {
      next_block();
    } else {  // start in the middle of the lists
      g_cur = g_begin;
      const int64_t lr = list_row(g_cur);
      cnt_cur = k_cnt[lr];
      idx_cur = const_idx(p.k_idx + lr * row_len);
      head_row0 = ((int64_t)b * p.Hq + hkv * group + g_cur) * p.Sq;
      e_cur = e_begin;
      row_next = head_row0 + (kTiled ? (int64_t)(idx_cur[e_cur] >> 8) * kSlab : (int64_t)idx_cur[e_cur] * p.q_block + sub_begin * kSlab);
      rem = nsub - sub_begin;
    }
    request_pair(0);
    request_pair(1);

    // tile lists: predicate bits of this wave's slab, from a second walk over the same lists (two entries per step)
    // (with the hand-over also the entry's tile-pair number and its slab inside the query tile)
    int g_cmp = -1, e_cmp = -1, cnt_cmp = 0, bits_cmp = 0, sub_cmp = 0;
    int64_t slot_cmp = 0, head_slot0 = 0;
    ConstIdx idx_cmp = nullptr, slot_idx_cmp = nullptr;
    auto enter_cmp_head = [&]() {  // list row of query head g_cmp of the group
      const int64_t lr = list_row(g_cmp);
      cnt_cmp = k_cnt[lr];
      idx_cmp = const_idx(p.k_idx + lr * row_len);
      if constexpr (kHandOver) {
        slot_idx_cmp = const_idx(p.k_slot + lr * row_len);
        const int64_t bh = (int64_t)b * p.Hq + hkv * group + g_cmp;
        head_slot0 = p.mask_bh == 1 ? bh * const_idx(p.pair_base)[tiles_per_head] : 0;
      }
    };
    auto next_bits = [&]() {
      ++e_cmp;
      while (e_cmp >= cnt_cmp) {
        if (++g_cmp >= group) { bits_cmp = 0; return; }
        enter_cmp_head();
        e_cmp = 0;
      }
      const int ent = idx_cmp[e_cmp];
      bits_cmp = ent & 255;
      if constexpr (kHandOver) {
        sub_cmp = (ent >> 8) & 3;
        slot_cmp = head_slot0 + slot_idx_cmp[e_cmp];
      }
    };
    if constexpr (kTiled) {
      if (parts > 1) {  // start in the middle of the lists, as the cursor of the copies does
        g_cmp = g_begin;
        enter_cmp_head();
        e_cmp = e_begin - 1;
      }
      next_bits();
      if (par) next_bits();
    }
    // dS hand-over: (query head of the group, list entry, slab inside the query block) of the slab this wave computes
    // next, and the pair number of entry 0 of that head's list row
    int h_g = -1, h_e = -1, h_s = 0, h_cnt = 0;
    int64_t h_slot0 = 0;
    const int64_t pair_bytes = (int64_t)p.q_block * p.k_block * 2;
    const int nsub_k = p.k_block / kSlab;
    const int t_key = 4 * ((kt * TK - kblk * p.k_block) / TK) + kg;  // this wave's 32-key slab inside the key block
    const uint32_t ho_off0 = (uint32_t)ds_unit_store_off(0, lane), ho_off1 = (uint32_t)ds_unit_store_off(1, lane);
    auto ho_next_entry = [&]() {
      ++h_e;
      while (h_e >= h_cnt) {
        if (++h_g >= group) return;
        const int64_t lr = list_row(h_g);
        h_cnt = k_cnt[lr];
        const ConstIdx pb = const_idx(p.pair_base);
        const int64_t bh = (int64_t)b * p.Hq + hkv * group + h_g;
        h_slot0 = pb[lr] + (p.mask_bh == 1 ? bh * pb[p.nK] : 0);
        h_e = 0;
      }
    };
    auto ho_advance = [&](int n) {
      h_s += n;
      if (h_s >= nsub) {  // nsub >= 4 > n
        h_s -= nsub;
        ho_next_entry();
      }
    };
    if constexpr (kHandOver && !kTiled) {
      if (parts == 1) {
        ho_next_entry();
      } else {
        h_g = g_begin;
        const int64_t lr = list_row(h_g);
        h_cnt = k_cnt[lr];
        const ConstIdx pb = const_idx(p.pair_base);
        const int64_t bh = (int64_t)b * p.Hq + hkv * group + h_g;
        h_slot0 = pb[lr] + (p.mask_bh == 1 ? bh * pb[p.nK] : 0);
        h_e = e_begin;
        h_s = sub_begin;
      }
      ho_advance(par);
    }
    wait_vmem<0>();
    __syncthreads();

    // per-lane fetch addresses with the wave's share folded in: slab addresses carry the parity's buffer, tile addresses
    // the key group's rows; what remains (pair, Q or dO, K or V, row group) is a compile-time displacement
    const LdsPtr lds = lds_ptr(smem);
    LdsPtr q_ptr[8], k_ptr[8], t_ptr[4][2];
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) {
      q_ptr[ks] = lds + rm.rd[ks] + par * kStageBytes;
      k_ptr[ks] = lds + rm.rd[ks] + kTileBase + kg * kSlabBytes;
    }
#pragma unroll
    for (int mb = 0; mb < 4; ++mb) {
      t_ptr[mb][0] = lds + tr.rd[mb][0] + par * kStageBytes;
      t_ptr[mb][1] = lds + tr.rd[mb][1] + par * kStageBytes;
    }
    const LdsPtr st_ptr = lds + par * kStageBytes + 2 * kSlabBytes + 16 * h;

    // One slab against this wave's 32 keys.  Operands are fetched right where they are used: with two waves per SIMD the
    // other wave's matrix instructions cover the wait (fetching a step ahead into a second register set measured slower).
    auto compute = [&](auto half_c) {
      constexpr int so = decltype(half_c)::value * 2 * kStageBytes;  // buffers 0, 1 or 2, 3
      f32x16 s, dp;
      // accumulator element 4g + e of half-wave h is query row 8g + 4h + e of the slab; dP starts from -delta of its row
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const f32x4 d4 = lds_read_f32x4(st_ptr + so + 4 * kSlab + 32 * g);
#pragma unroll
        for (int e = 0; e < 4; ++e) { s[4 * g + e] = 0.f; dp[4 * g + e] = d4[e]; }
      }
#pragma unroll
      for (int ks = 0; ks < 8; ++ks) {
        s = mfma32(lds_read_b128(q_ptr[ks] + so), lds_read_b128(k_ptr[ks]), s);
        dp = mfma32(lds_read_b128(q_ptr[ks] + so + kSlabBytes), lds_read_b128(k_ptr[ks] + kTileBytes), dp);
      }
      // does this wave's key block select the first / second 16 query rows of the slab?
      const bool on0 = !kTiled || ((bits_cmp >> (2 * kg)) & 1) != 0;
      const bool on1 = !kTiled || ((bits_cmp >> (2 * kg + 1)) & 1) != 0;
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const f32x4 l4 = lds_read_f32x4(st_ptr + so + 32 * g);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          float pv = fast_exp2(__builtin_fmaf(s[4 * g + e], c, -l4[e]));
          if constexpr (kTiled) pv = (g < 2 ? on0 : on1) ? pv : 0.f;  // a select: inf or NaN of a masked row is discarded
          s[4 * g + e] = pv;
          dp[4 * g + e] = pv * dp[4 * g + e];
        }
      }
      bf16x8 pk[2], dsk[2];
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        pk[j] = pack8(s[8 * j + 0], s[8 * j + 1], s[8 * j + 2], s[8 * j + 3], s[8 * j + 4], s[8 * j + 5], s[8 * j + 6], s[8 * j + 7]);
        dsk[j] = pack8(dp[8 * j + 0], dp[8 * j + 1], dp[8 * j + 2], dp[8 * j + 3], dp[8 * j + 4], dp[8 * j + 5], dp[8 * j + 6], dp[8 * j + 7]);
      }
      if constexpr (kHandOver) {
        char* unit = reinterpret_cast<char*>(p.ds_ws);
        if constexpr (kTiled)  // 16 units per tile pair, ordered (32-key slab, 32-row slab)
          unit += slot_cmp * (16 * kDsUnitBytes) + (kg * 4 + sub_cmp) * kDsUnitBytes;
        else
          unit += (h_slot0 + h_e) * pair_bytes + ((int64_t)((h_s >> 2) * nsub_k + t_key) * 4 + (h_s & 3)) * kDsUnitBytes;
        // written once, read once by another kernel much later: streaming stores, so that they do not push the Q / dO
        // slabs that other work-groups are about to fetch out of L2
        store16_stream(unit, ho_off0, dsk[0]);
        store16_stream(unit, ho_off1, dsk[1]);
      }
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int mb = 0; mb < 4; ++mb) {
          const int roff = so + 16 * j * kRowBytes;
          const bf16x8 adv = cat(lds_read_tr(t_ptr[mb][0] + kSlabBytes + roff), lds_read_tr(t_ptr[mb][1] + kSlabBytes + roff));
          acc_v[mb] = mfma32(adv, pk[j], acc_v[mb]);
          const bf16x8 adk = cat(lds_read_tr(t_ptr[mb][0] + roff), lds_read_tr(t_ptr[mb][1] + roff));
          acc_k[mb] = mfma32(adk, dsk[j], acc_k[mb]);
        }
    };

    const int npairs = (nslabs + 1) >> 1;
    auto step = [&](auto half_c, int s2) {
      // tile lists: a wave whose 32 keys are selected by neither half of the slab leaves the slab out (wave-uniform)
      const bool worked = 2 * s2 + par < nslabs && (!kTiled || ((bits_cmp >> (2 * kg)) & 3) != 0);
      if (worked) compute(half_c);
      if constexpr (kTiled) { next_bits(); next_bits(); }
      if constexpr (kHandOver && !kTiled) ho_advance(2);
      // this wave's copies of the next pair, requested one step ago, must have landed.  The two dS stores of this step, if
      // the wave made any, are younger and may still be on their way (the counter covers loads and stores alike and runs
      // down in issue order).
      if (kHandOver && worked) wait_vmem<2>(); else wait_vmem<0>();
      __syncthreads();  // everybody is done with this pair and everybody's copies of the next pair have landed
      request_pair(decltype(half_c)::value);
    };
    for (int s2 = 0; s2 < npairs; s2 += 2) {
      step(IC<0>{}, s2);
      if (s2 + 1 < npairs) step(IC<1>{}, s2 + 1);
    }
    wait_vmem<0>();
    __syncthreads();  // no copy is writing LDS any more; K, V and the ring are free

    // The two waves of a key group swap halves: parity 1 hands its dV part to parity 0 through the first 64 KiB of LDS,
    // parity 0 hands its dK part to parity 1 through the next 64 KiB (16 KiB per wave each).
    f32x4* send = reinterpret_cast<f32x4*>(smem + (par ? 0 : 65536) + kg * 16384) + lane;
    const f32x4* recv = reinterpret_cast<const f32x4*>(smem + (par ? 65536 : 0) + kg * 16384) + lane;
#pragma unroll
    for (int mb = 0; mb < 4; ++mb)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const f32x16& a = par ? acc_v[mb] : acc_k[mb];
        send[(mb * 4 + g) * 64] = (f32x4){a[4 * g + 0], a[4 * g + 1], a[4 * g + 2], a[4 * g + 3]};
      }
    __syncthreads();
#pragma unroll
    for (int mb = 0; mb < 4; ++mb)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const f32x4 r = recv[(mb * 4 + g) * 64];
        f32x16& a = par ? acc_k[mb] : acc_v[mb];
#pragma unroll
        for (int e = 0; e < 4; ++e) a[4 * g + e] += r[e];
      }
  }

  if (parts > 1) {
    // part of a split item: unscaled fp32 partial sums go to the workspace, dV tile (parity 0), then dK tile (parity 1)
    float* prow = p.split.ws + ((int64_t)(item - p.split.first) * parts + part) * (2 * TK * kHeadDim) + par * (TK * kHeadDim) +
                  (kg * 32 + l32) * kHeadDim;
#pragma unroll
    for (int mb = 0; mb < 4; ++mb)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const f32x16& a = par ? acc_k[mb] : acc_v[mb];
        *reinterpret_cast<f32x4*>(prow + 32 * mb + 8 * g + 4 * h) = (f32x4){a[4 * g + 0], a[4 * g + 1], a[4 * g + 2], a[4 * g + 3]};
      }
    return;
  }
  // parity 0 writes dV, parity 1 writes dK (both zero when no query block selects this key tile)
  __bf16* orow = (par ? p.dk : p.dv) + (krow0 + kg * 32 + l32) * kHeadDim;
  const float oscale = par ? p.scale : 1.f;
#pragma unroll
  for (int mb = 0; mb < 4; ++mb)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const f32x16& a = par ? acc_k[mb] : acc_v[mb];
      *reinterpret_cast<bf16x4*>(orow + 32 * mb + 8 * g + 4 * h) =
          pack4(a[4 * g + 0] * oscale, a[4 * g + 1] * oscale, a[4 * g + 2] * oscale, a[4 * g + 3] * oscale);
    }
}

hipError_t launch_bwd_dkdv(BwdParams p, hipStream_t stream) {
  p.num_items = p.B * p.Hkv * (p.Skv / 128);
  // tail splitting (one work-group per compute unit); a part stores two 128 x 128 fp32 tiles
  void* const caller_ws = p.split.ws;  // whether or not anything is split
  p.split = plan_split(p.num_items, 1, 2 * 128 * kHeadDim * 4, p.split.ws, p.split_ws_bytes);
  plan_xcd_mapping(p.B * p.Hkv, p.split.first, p.items_per_xcd, p.split.main_wgs);
  const int split_items = p.num_items - p.split.first;
  const bool hand_over = p.ds_ws != nullptr;
  void (*fn)(const BwdParams) = p.tiled ? (hand_over ? &dkdv_kernel<true, true> : &dkdv_kernel<true, false>)
                                        : (hand_over ? &dkdv_kernel<false, true> : &dkdv_kernel<false, false>);
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(fn), hipFuncAttributeMaxDynamicSharedMemorySize, kSmemBytes + 16);
  if (e != hipSuccess) return e;
  // large launches let the work-groups claim their grid indices, with some work-groups more than indices (claim_work)
  p.total_work = p.split.main_wgs + split_items * p.split.parts;
  int grid = p.total_work;
  p.queue = nullptr;
  if (claims_wanted(p.items_per_xcd, p.total_work, 1))
    p.queue = work_queue_in(caller_ws, p.split_ws_bytes, (int64_t)split_items * p.split.parts * 2 * 128 * kHeadDim * 4);
  if (p.queue != nullptr) {
    if ((e = launch_queue_reset(p.queue, stream)) != hipSuccess) return e;
    grid += surplus_work_groups(p.total_work);
  }
  hipLaunchKernelGGL(fn, dim3(grid), dim3(512), kSmemBytes + 16, stream, p);
  if (split_items > 0) {
    const int64_t row0 = (int64_t)p.split.first * 128;
    e = launch_partial_sum(p.split.ws, p.split.parts, 2 * 128 * kHeadDim, p.dv, row0, split_items, 1.f, stream);
    if (e != hipSuccess) return e;
    e = launch_partial_sum(p.split.ws + 128 * kHeadDim, p.split.parts, 2 * 128 * kHeadDim, p.dk, row0, split_items, p.scale, stream);
    if (e != hipSuccess) return e;
  }
  if (hand_over) {
    return launch_poison_unless_fit(p, p.dk, p.dv, (int64_t)p.B * p.Hkv * p.Skv * kHeadDim, stream);
  }
  return hipGetLastError();
}

}  // namespace fba
