// Backward, dK and dV, 64 keys per wave: gfx950, head_dim 128, bf16 in / fp32 accumulate / bf16 out, no atomics.
//
// Same mathematics, lists, hand-over layout and tail splitting as dkdv_kernel (fba_bwd_dkdv.hip); what differs is the shape
// of a wave's work.  Work-group = 128 key rows, four waves, one per SIMD.  Wave w works on keys 64 (w % 2) .. +63 (two
// 32-key groups) and on every second 32-query slab of the list (w / 2 = parity of the slab).  Every Q / dO operand fetched
// from LDS, row-major or transposed, then feeds two matrix instructions, one per key group, and the K rows of the wave
// stay in registers for the whole list: 40 KiB of LDS reads per 64 matrix instructions instead of 96 KiB.  The price is
// one wave per SIMD: dK and dV accumulators alone are 256 registers per lane (kept in accumulation registers), and
// nothing but the wave's own instruction order overlaps softmax arithmetic with matrix work.
// LDS: ring of six (Q slab | dO slab | lse2 | -delta) buffers, three per slab parity, then the V tile (32 KiB).
#include <type_traits>

#include "fba_common.h"
#include "fba_kernels.h"

namespace fba {

namespace {

constexpr int kSlab = 32;
constexpr int kSlabBytes = kSlab * kRowBytes;       // 8 KiB
constexpr int kStatBytes = 2 * kSlab * 4;           // lse2[32] | -delta[32]
constexpr int kStageBytes = 2 * kSlabBytes + kStatBytes;
constexpr int kRing = 6;                            // three buffers per slab parity
constexpr int kTileBytes = 128 * kRowBytes;         // K or V tile, 32 KiB
constexpr int kRingBase = 0;                        // the ring first: its offsets fit the 16-bit field of an LDS fetch
constexpr int kTileBase = kRing * kStageBytes;      // V tile
constexpr int kSmemBytes = kTileBase + kTileBytes;   // ring + V tile (130 KiB); the final exchange re-uses the first 128 KiB

template <int N>
using IC = std::integral_constant<int, N>;

// acc += a b with the accumulator held in accumulation registers.  dK and dV of 64 keys are 256 registers per lane, all
// the accumulation registers a wave has; S and dP, which the softmax arithmetic reads, must therefore live in ordinary
// registers, and the compiler does not mix the two forms of the instruction on its own.  Written as inline asm, so the
// compiler does not know that it is a matrix instruction and inserts none of the wait states one needs; that is safe
// here because (a) its A and B operands come from LDS fetches and from conversion instructions, never straight from
// another matrix instruction, (b) two of these on one accumulator are always at least eight matrix instructions apart,
// and (c) the accumulators are read only after drain_matrix_pipe() below.
FBA_DEVICE void mfma32_acc(f32x16& acc, bf16x8 a, bf16x8 b) {
  asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b));
}
// More idle cycles than any matrix instruction needs to retire its result.
FBA_DEVICE void drain_matrix_pipe() { asm volatile("s_nop 15\n\ts_nop 15\n\ts_nop 15\n\ts_nop 15" ::: "memory"); }

}  // namespace

// Block lists only (q_block and k_block multiples of 128; list entries are query blocks, expanded to q_block/32 slabs).
// kHandOver: every wave also stores the bf16 dS it forms to p.ds_ws (layout: fba_common.h), so that dQ = dS K can be
// formed later without recomputing S and dP.
template <bool kHandOver>
__global__ __attribute__((amdgpu_flat_work_group_size(256, 256), amdgpu_waves_per_eu(1, 1))) void dkdv64_kernel(const BwdParams p) {
  constexpr bool kTiled = false;
  extern __shared__ __attribute__((aligned(16))) char smem[];
  constexpr int TK = 128;
  const int tid = threadIdx.x, lane = tid & 63, l32 = lane & 31, h = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int kg = wave & 1, par = wave >> 1;  // 64-key group, slab parity
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
  if constexpr (kHandOver) {
    // lists that number more pairs than the workspace holds: no slab is touched, nothing is stored into the workspace
    // (the launcher's last launch then reports it)
    if (!workspace_holds_lists(p)) slabs_all = 0;
  }
  // this work-group's range of listed slabs: all of them, or part `part` of `parts` (boundaries on multiples of four slabs;
  // block lists only)
  const int s_begin = parts == 1 ? 0 : 4 * (int)(((int64_t)(slabs_all / 4) * part) / parts);
  const int nslabs = (parts == 1 ? slabs_all : 4 * (int)(((int64_t)(slabs_all / 4) * (part + 1)) / parts)) - s_begin;
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
  // the two waves of a parity bring in a slab together, 16 rows (four wave-level copies) each
  uint32_t dma_off[4];
#pragma unroll
  for (int g = 0; g < 4; ++g) {
    const int row = 16 * kg + 4 * g + (lane >> 4);
    dma_off[g] = (uint32_t)(row * kRowBytes + (((lane & 15) ^ swz(row)) << 4));
  }
  const uint32_t dma_dst = (uint32_t)(16 * kg * kRowBytes);
  auto copy_slab = [&](uint32_t slab_lds, const char* src) {
#pragma unroll
    for (int g = 0; g < 4; ++g) dma16(slab_lds + dma_dst + g * 4 * kRowBytes, src, dma_off[g]);
  };
  const uint32_t lds0 = lds_addr(smem);
  const uint32_t ring_dst = lds0 + kRingBase;
  const int64_t rows_total = (int64_t)p.B * p.Hq * p.Sq;
  // statistics copy: lanes 0..31 fetch lse2[row0 + l], lanes 32..63 fetch -delta[row0 + l - 32]
  const uint32_t stat_off = (uint32_t)((lane >> 5) * rows_total * 4 + (lane & 31) * 4);
  const float c = p.scale_log2e;

  f32x16 acc_k[2][4], acc_v[2][4];  // [32-key group][32 head-dim columns]
#pragma unroll
  for (int grp = 0; grp < 2; ++grp)
#pragma unroll
    for (int mb = 0; mb < 4; ++mb)
#pragma unroll
      for (int r = 0; r < 16; ++r) { acc_k[grp][mb][r] = 0.f; acc_v[grp][mb][r] = 0.f; }

  if (nslabs > 0) {
    // V tile into LDS: wave w brings in rows 32 w .. 32 w + 31 (two slabs' worth of copies)
    {
      const char* src = reinterpret_cast<const char*>(p.v) + (krow0 + 32 * wave) * kRowBytes;
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const uint32_t dst = lds0 + kTileBase + wave * kSlabBytes + j * 16 * kRowBytes;
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const int row = 4 * g + (lane >> 4);  // row inside the 16-row half; swz depends on row % 16 only
          dma16(dst + g * 4 * kRowBytes, src + j * 16 * kRowBytes, (uint32_t)(row * kRowBytes + (((lane & 15) ^ swz(row)) << 4)));
        }
      }
    }
    // K rows of the wave's two key groups as B operands, in registers for the whole list: lane holds key l32 of the group,
    // d = 16 ks + 8 h .. +7
    bf16x8 kreg[2][8];
    {
      const __bf16* kp = p.k + (krow0 + 64 * kg + l32) * kHeadDim + 8 * h;
#pragma unroll
      for (int grp = 0; grp < 2; ++grp)
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) kreg[grp][ks] = *reinterpret_cast<const bf16x8*>(kp + grp * 32 * kHeadDim + 16 * ks);
    }
    // Cursor over (query head of the group, list entry, pair of slabs).  Slabs are numbered in list order; slabs 2i and 2i+1
    // form pair i, the first for the waves of parity 0, the second for those of parity 1.  A pair never straddles two query
    // blocks (q_block is a multiple of 128 and ranges start on multiples of four slabs), so the cursor moves a pair at a
    // time: first query row of the next pair, and (hand-over) the byte offset of the dS unit that the pair's first slab and
    // this wave's first key group own in the workspace.  Requests run two pairs ahead of the arithmetic; the unit offsets
    // wait in two variables until their slab's dS is stored, so the lists are walked once only.
    const char* qbase = reinterpret_cast<const char*>(p.q);
    const char* dobase = reinterpret_cast<const char*>(p.d_o);
    const char* stbase = reinterpret_cast<const char*>(p.stats);
    const int64_t pair_bytes = (int64_t)p.q_block * p.k_block * 2;
    const int nsub_k = p.k_block / kSlab;
    const int t_key = 4 * ((kt * TK - kblk * p.k_block) / TK) + 2 * kg;  // this wave's first 32-key slab inside the key block
    const uint32_t ho_off0 = (uint32_t)ds_unit_store_off(0, lane);  // the second chunk's offset is formed from it at the store
    // The common step (the next pair lies in the same query block) is a handful of scalar additions; what the step adds is
    // kept in variables that turn to zero once every listed pair has been requested, so that the cursor then stays on the
    // last pair without a test of its own.
    int g_cur = -1, e_cur = -1, cnt_cur = 0, rem = 1, sub = 0;
    int row_step = 2 * kSlab;
    int64_t unit_step = 2 * kDsUnitBytes;                   // to the next pair inside a 128-row tile
    int64_t tile_step = (int64_t)(nsub_k * 4 - 4) * kDsUnitBytes;  // on top of it, from a tile's last pair to the next tile's first
    ConstIdx idx_cur = nullptr;
    int64_t row_next = 0, head_row0 = 0, unit_next = 0, slot0_cur = 0;
    auto enter_head = [&](int g) {  // list row, first query row and first pair number of query head g of the group
      const int64_t lr = list_row(g);
      cnt_cur = k_cnt[lr];
      idx_cur = const_idx(p.k_idx + lr * row_len);
      const int64_t bh = (int64_t)b * p.Hq + hkv * group + g;
      head_row0 = bh * p.Sq;
      if constexpr (kHandOver) {
        const ConstIdx pb = const_idx(p.pair_base);
        slot0_cur = pb[lr] + (p.mask_bh == 1 ? bh * pb[p.nK] : 0);
      }
    };
    auto enter_block = [&](int first_sub) {  // entry e_cur of the current head, starting at slab first_sub (a multiple of 4)
      row_next = head_row0 + (int64_t)idx_cur[e_cur] * p.q_block + first_sub * kSlab;
      if constexpr (kHandOver)
        unit_next = (slot0_cur + e_cur) * pair_bytes + ((int64_t)((first_sub >> 2) * nsub_k + t_key) * 4) * kDsUnitBytes;
      sub = first_sub;
      rem = (nsub - first_sub) >> 1;
    };
    auto next_block = [&]() {  // first pair of the next listed query block, if any
      ++e_cur;
      while (e_cur >= cnt_cur && g_cur + 1 < group) {
        enter_head(++g_cur);
        e_cur = 0;
      }
      if (e_cur < cnt_cur) {
        enter_block(0);
      } else {  // nothing left: every further step repeats the last pair
        row_step = 0;
        unit_step = 0;
        tile_step = 0;
        rem = 1 << 30;
      }
    };
    auto advance = [&]() {  // to the next pair
      if (rem == 1) {
        next_block();
      } else {
        --rem;
        row_next += row_step;
        sub += 2;
        // units of a pair are ordered (128-row tile of the block, 32-key slab, slab inside the tile)
        if constexpr (kHandOver) unit_next += unit_step + ((sub & 3) ? 0 : tile_step);
      }
    };
    // Nine copies per wave request one slab (Q rows, dO rows, statistics), by the two waves of the slab's parity.  Every
    // step issues them, so that the count of copies in flight is the same at every wait; once the lists are exhausted
    // the last slab is simply requested again, into a buffer nobody reads any more.
    auto issue_copy = [&](int ring, int64_t row) {
      const uint32_t dst = ring_dst + ring * kStageBytes;
      copy_slab(dst, qbase + row * kRowBytes);
      copy_slab(dst + kSlabBytes, dobase + row * kRowBytes);
      dma4(dst + 2 * kSlabBytes, stbase + row * 4, stat_off);  // both waves copy the same 256 bytes
    };
    // the same request one copy at a time (i = 0..8), for spreading over a phase of matrix instructions
    uint32_t stat_off_loop = stat_off;
    auto issue_copy_part = [&](int i, uint32_t dst, int64_t row) {
      if (i < 4) dma16(dst + dma_dst + i * 4 * kRowBytes, qbase + row * kRowBytes, dma_off[i]);
      else if (i < 8) dma16(dst + kSlabBytes + dma_dst + (i - 4) * 4 * kRowBytes, dobase + row * kRowBytes, dma_off[i - 4]);
      else dma4(dst + 2 * kSlabBytes, stbase + row * 4, stat_off_loop);
    };
    // A parity keeps three buffers: ring buffer 3 * par + (i % 3) holds its slab of pair i.
    if (parts == 1) {
      next_block();
    } else {  // start in the middle of the lists
      g_cur = g_begin;
      enter_head(g_cur);
      e_cur = e_begin;
      enter_block(sub_begin);
    }
    // pairs 0 and 1 are requested here; their dS units wait in unit_cur (the slab whose softmax is next) and unit_nxt
    int64_t unit_cur = unit_next + par * kDsUnitBytes;
    issue_copy(3 * par + 0, row_next + par * kSlab);
    advance();
    int64_t unit_nxt = unit_next + par * kDsUnitBytes;
    issue_copy(3 * par + 1, row_next + par * kSlab);
    advance();
    wait_vmem<0>();
    __syncthreads();
    // a value of its own from here on: held in one register through the loop instead of being fetched back from the
    // spill area wherever the compiler had cut the kernel-long live range
    asm volatile("" : "+v"(stat_off_loop));

    // Per-lane fetch addresses with the wave's share folded in: slab addresses carry the parity's three buffers, V
    // addresses the wave's 64 keys.  One register each: the operand step (row-major fetches) and the column block and row
    // half (transposed fetches) only move the 16-byte chunk inside a 256-byte row, chunk c of row r living in slot
    // c ^ swz(r), so they are exclusive-ors with constants below 256; everything added here is a multiple of 256.
    static_assert(kStageBytes % 256 == 0 && kTileBase % 256 == 0 && kSlabBytes % 256 == 0, "the exclusive-ors below touch bits 5..7");
    const LdsPtr lds = lds_ptr(smem);
    const LdsPtr q_base = lds + rm.rd[0] + par * 3 * kStageBytes;
    const LdsPtr v_base = lds + rm.rd[0] + kTileBase + kg * 2 * kSlabBytes;
    const LdsPtr t_base = lds + tr.rd[0][0] + par * 3 * kStageBytes;
    auto flip = [](LdsPtr ptr, uint32_t bits) { return (LdsPtr)(uintptr_t)((uint32_t)(uintptr_t)ptr ^ bits); };
    auto row_major = [&](LdsPtr base, int ks) { return flip(base, 32u * ks); };  // operand step ks of a slab (base: step 0)
    auto transposed = [&](LdsPtr base, int mb, int half) {                        // column block mb, rows +8 * half
      return flip(base, (uint32_t)(mb << 6 | half << 5)) + half * 8 * kRowBytes;
    };
    const LdsPtr st_ptr = lds + par * 3 * kStageBytes + 2 * kSlabBytes + 16 * h;
#pragma unroll
    for (int grp = 0; grp < 2; ++grp)
#pragma unroll
      for (int ks = 0; ks < 8; ++ks) pin(kreg[grp][ks]);

    // Software pipeline over the wave's slabs t = 0, 1, ...: while the vector unit turns S_t, dP_t into P_t, dS_t, the matrix
    // pipe adds slab t-1 into dV and dK; then it forms S_{t+1}, dP_{t+1}.  One wave per SIMD has nobody else to hide behind,
    // so the interleaving is written out: one accumulating matrix instruction, then the arithmetic of one accumulator
    // element of both products, each anchored in place.
    f32x16 s[2], dp[2];
    // P and dS of a slab, packed as B operands.  Two sets: the slab that is accumulated reads one while the arithmetic of
    // the next slab fills the other, so that no value has to be moved when a slab is done (the loop below is unrolled by two).
    bf16x8 pk[2][2][2], dsk[2][2][2];  // [set][key group][16-query step]

    // S, dP of the slab in the buffer at byte offset `so` against this wave's 64 keys: every Q / dO operand feeds both key
    // groups.  S comes first, so that while the matrix pipe works on dP the vector unit can already turn S of the first key
    // group into P = exp2(S c - lse) (in place): a wave alone on its SIMD pays for every instruction it issues, and the
    // other phase, softmax_and_accumulate(), has more arithmetic than its matrix instructions cover, this one less.
    // Matrix instructions go in fours, two operand steps each; the operands of the next four are requested before a four
    // is issued, and the scheduling fences keep the compiler from moving the requests back next to their use, where the
    // wave would wait for every fetch.
    auto scores = [&](auto extras_c, auto set_c, int so, uint32_t req_dst, int64_t req_row, char* ds_unit) {
      constexpr bool kExtras = decltype(extras_c)::value;
      constexpr int kSet = decltype(set_c)::value;  // the set that holds dS of the slab to store  // false for the wave's first slab: nothing to copy or store yet
      // accumulator element 4g + e of half-wave h is query row 8g + 4h + e of the slab; dP starts from -delta of its row
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const f32x4 d4 = lds_read_f32x4(st_ptr + so + 4 * kSlab + 32 * g);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          s[0][4 * g + e] = 0.f; s[1][4 * g + e] = 0.f;
          dp[0][4 * g + e] = d4[e]; dp[1][4 * g + e] = d4[e];
        }
      }
      LdsPtr qs = q_base + so, vs = v_base;
      asm volatile("" : "+v"(qs), "+v"(vs));  // one register each; the eight addresses are formed where they are used
      bf16x8 qa = lds_read_b128(row_major(qs, 0)), qb = lds_read_b128(row_major(qs, 1));
      bf16x8 da, db, va0, va1, vb0, vb1;
      f32x4 l4;  // lse * log2(e) of the rows whose P comes next
#pragma unroll
      for (int j = 0; j < 4; ++j) {  // S: operand steps 2j, 2j+1
        bf16x8 qa_n = qa, qb_n = qb;
        if (j < 3) {
          qa_n = lds_read_b128(row_major(qs, 2 * j + 2));
          qb_n = lds_read_b128(row_major(qs, 2 * j + 3));
        } else {  // the first operands of dP
          da = lds_read_b128(row_major(qs, 0) + kSlabBytes);
          va0 = lds_read_b128(row_major(vs, 0));
          va1 = lds_read_b128(row_major(vs, 0) + kSlabBytes);
          db = lds_read_b128(row_major(qs, 1) + kSlabBytes);
          vb0 = lds_read_b128(row_major(vs, 1));
          vb1 = lds_read_b128(row_major(vs, 1) + kSlabBytes);
          l4 = lds_read_f32x4(st_ptr + so);
        }
        __builtin_amdgcn_sched_barrier(0);
        // the copies of the slab after next are issued one at a time behind every second matrix instruction (vector-memory
        // instructions that follow each other closely cost the wave more), the last one in the dP part ahead of the first
        // dS store: copies first, stores last, so that the wait before the next barrier lets the four youngest
        // operations, the stores, stay in flight
        s[0] = mfma32(qa, kreg[0][2 * j], s[0]);
        s[1] = mfma32(qa, kreg[1][2 * j], s[1]);
        if constexpr (kExtras) issue_copy_part(2 * j, req_dst, req_row);
        s[0] = mfma32(qb, kreg[0][2 * j + 1], s[0]);
        s[1] = mfma32(qb, kreg[1][2 * j + 1], s[1]);
        if constexpr (kExtras) issue_copy_part(2 * j + 1, req_dst, req_row);
        __builtin_amdgcn_sched_barrier(0);
        qa = qa_n; qb = qb_n;
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) {  // dP: operand steps 2j, 2j+1; P of the first key group, rows 8j + 4h + 0..3
        bf16x8 da_n = da, db_n = db, va0_n = va0, va1_n = va1, vb0_n = vb0, vb1_n = vb1;
        f32x4 l4_n = l4;
        if (j < 3) {
          da_n = lds_read_b128(row_major(qs, 2 * j + 2) + kSlabBytes);
          va0_n = lds_read_b128(row_major(vs, 2 * j + 2));
          va1_n = lds_read_b128(row_major(vs, 2 * j + 2) + kSlabBytes);
          db_n = lds_read_b128(row_major(qs, 2 * j + 3) + kSlabBytes);
          vb0_n = lds_read_b128(row_major(vs, 2 * j + 3));
          vb1_n = lds_read_b128(row_major(vs, 2 * j + 3) + kSlabBytes);
          l4_n = lds_read_f32x4(st_ptr + so + 32 * (j + 1));
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          if (e == 0) dp[0] = mfma32(da, va0, dp[0]);
          if constexpr (kExtras) {
            if (e == 1 && j == 0) issue_copy_part(8, req_dst, req_row);
          }
          if (e == 1) dp[1] = mfma32(da, va1, dp[1]);
          if (e == 2) dp[0] = mfma32(db, vb0, dp[0]);
          if (e == 3) dp[1] = mfma32(db, vb1, dp[1]);
          float pv = fast_exp2(__builtin_fmaf(s[0][4 * j + e], c, -l4[e]));
          asm volatile("" : "+v"(pv));  // keeps this element's arithmetic behind its matrix instruction
          s[0][4 * j + e] = pv;
        }
        if constexpr (kHandOver && kExtras) {  // scores() runs only while the wave has a further slab, so ds_unit is set
          if (j & 1) store16_stream_second(ds_unit + (j >> 1) * 4 * kDsUnitBytes, ho_off0, dsk[kSet][j >> 1][1]);
          else store16_stream(ds_unit + (j >> 1) * 4 * kDsUnitBytes, ho_off0, dsk[kSet][j >> 1][0]);
        }
        __builtin_amdgcn_sched_barrier(0);
        da = da_n; db = db_n; va0 = va0_n; va1 = va1_n; vb0 = vb0_n; vb1 = vb1_n; l4 = l4_n;
      }
    };

    // P_t, dS_t from s, dp (statistics in the buffer at `so`), interleaved with dV += dO^T P, dK += Q^T dS of the previous
    // slab (buffer at `po`, operands pk / dsk).  Eight groups of four
    // matrix instructions (one transposed dO operand and one transposed Q operand, each against both key groups) and four
    // accumulator elements of arithmetic; the operands and statistics of group n+1 are requested before group n starts.
    auto softmax_and_accumulate = [&](auto in_c, int so, int po) {
      constexpr int kIn = decltype(in_c)::value;  // set of the slab that is accumulated; the new P, dS go to the other
      bf16x2 pw[2][8], dw[2][8];  // new P and dS, packed: [key group][register pair]
      LdsPtr ts = t_base + po;
      asm volatile("" : "+v"(ts));
      auto fetch_dv = [&](int n) {
        const int roff = 16 * (n >> 2) * kRowBytes, mb = n & 3;
        return cat(lds_read_tr(transposed(ts, mb, 0) + kSlabBytes + roff), lds_read_tr(transposed(ts, mb, 1) + kSlabBytes + roff));
      };
      auto fetch_dk = [&](int n) {
        const int roff = 16 * (n >> 2) * kRowBytes, mb = n & 3;
        return cat(lds_read_tr(transposed(ts, mb, 0) + roff), lds_read_tr(transposed(ts, mb, 1) + roff));
      };
      bf16x8 adv = fetch_dv(0), adk = fetch_dk(0);
      f32x4 l4 = {0.f, 0.f, 0.f, 0.f};  // statistics of the second key group's rows only: scores() left P of the first group
#pragma unroll
      for (int n = 0; n < 8; ++n) {  // n = 4 j + mb for the matrix work, 4 grp + g for the arithmetic
        bf16x8 adv_n = adv, adk_n = adk;
        f32x4 l4_n = l4;
        if (n < 7) {
          adv_n = fetch_dv(n + 1);
          adk_n = fetch_dk(n + 1);
          if (n >= 3) l4_n = lds_read_f32x4(st_ptr + so + 32 * ((n + 1) & 3));
        }
        __builtin_amdgcn_sched_barrier(0);
        const int j = n >> 2, mb = n & 3, grp = n >> 2, g = n & 3;
        float pv[4], dsv[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          if (e == 0) mfma32_acc(acc_v[0][mb], adv, pk[kIn][0][j]);
          if (e == 1) mfma32_acc(acc_v[1][mb], adv, pk[kIn][1][j]);
          if (e == 2) mfma32_acc(acc_k[0][mb], adk, dsk[kIn][0][j]);
          if (e == 3) mfma32_acc(acc_k[1][mb], adk, dsk[kIn][1][j]);
          pv[e] = grp == 0 ? s[0][4 * g + e] : fast_exp2(__builtin_fmaf(s[1][4 * g + e], c, -l4[e]));
          dsv[e] = pv[e] * dp[grp][4 * g + e];
          if (e & 1) {
            bf16x2 p2 = __builtin_convertvector((f32x2){pv[e - 1], pv[e]}, bf16x2);
            bf16x2 d2 = __builtin_convertvector((f32x2){dsv[e - 1], dsv[e]}, bf16x2);
            asm volatile("" : "+v"(p2), "+v"(d2));
            pw[grp][2 * g + (e >> 1)] = p2;
            dw[grp][2 * g + (e >> 1)] = d2;
          } else {
            asm volatile("" : "+v"(pv[e]), "+v"(dsv[e]));  // keeps this element's arithmetic behind its matrix instruction
          }
        }
        __builtin_amdgcn_sched_barrier(0);
        adv = adv_n; adk = adk_n; l4 = l4_n;
      }
#pragma unroll
      for (int grp = 0; grp < 2; ++grp)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          pk[1 - kIn][grp][j] = cat(__builtin_shufflevector(pw[grp][4 * j + 0], pw[grp][4 * j + 1], 0, 1, 2, 3),
                           __builtin_shufflevector(pw[grp][4 * j + 2], pw[grp][4 * j + 3], 0, 1, 2, 3));
          dsk[1 - kIn][grp][j] = cat(__builtin_shufflevector(dw[grp][4 * j + 0], dw[grp][4 * j + 1], 0, 1, 2, 3),
                            __builtin_shufflevector(dw[grp][4 * j + 2], dw[grp][4 * j + 3], 0, 1, 2, 3));
        }
    };

    const int nlocal = nslabs >> 1;  // slabs of this wave's parity (nslabs is a multiple of four)
#pragma unroll
    for (int grp = 0; grp < 2; ++grp)
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int e = 0; e < 8; ++e) { pk[0][grp][j][e] = (__bf16)0.f; dsk[0][grp][j][e] = (__bf16)0.f; }
    // The zeros are written here and now (an opaque pin: the compiler cannot put them off or form them again later).
    // Left to itself it writes them right in front of the first accumulating matrix instruction, which, being inline asm,
    // gets none of the wait states the compiler gives a matrix instruction that reads a register the vector unit has
    // just written, and then multiplies by whatever the registers held before.
#pragma unroll
    for (int grp = 0; grp < 2; ++grp)
#pragma unroll
      for (int j = 0; j < 2; ++j) asm volatile("" : "+v"(pk[0][grp][j]), "+v"(dsk[0][grp][j]));
    scores(std::false_type{}, IC<0>{}, 0, 0, 0, nullptr);
    // Iteration t: slab t lives in buffer t % 3, slab t-1 in (t+2) % 3, slab t+1 in (t+1) % 3; P, dS of slab t-1 in set
    // t % 2.  The first iteration adds nothing (P = dS = 0 against the finite rows of slab 0).  An iteration has no branch
    // but the cursor's change of block; the wave's last slab is handled behind the loop.
    int cur = 0, prev = 0, nxt = kStageBytes;
    auto iteration = [&](auto in_c) {
      constexpr int kIn = decltype(in_c)::value;
      softmax_and_accumulate(in_c, cur, prev);
      char* ds_unit = nullptr;  // where dS_t goes
      if constexpr (kHandOver) ds_unit = reinterpret_cast<char*>(p.ds_ws) + unit_cur;
      // slab t+2 will replace slab t-1 (past the end of the lists: a repeat of the last slab that nobody reads); its copies
      // are issued in between the matrix instructions of scores().  The cursor moves on here, while the last matrix
      // instructions of this slab still run.
      const int64_t req_row = row_next + par * kSlab;
      unit_cur = unit_nxt;
      unit_nxt = unit_next + par * kDsUnitBytes;
      advance();
      // this wave's copies of slab t+1, requested during the previous iteration, must have landed; the four dS stores issued
      // after them may still be on their way (the counter covers loads and stores alike, in issue order; before the first
      // iteration nothing is in flight)
      if constexpr (kHandOver) wait_vmem<4>(); else wait_vmem<0>();
      __syncthreads();  // everybody is done with slab t-1 and everybody's copies of slab t+1 have landed
      const int freed = nxt + kStageBytes == 3 * kStageBytes ? 0 : nxt + kStageBytes;  // buffer of slab t-1 = buffer of slab t+2
      const uint32_t req_dst = ring_dst + 3 * par * kStageBytes + freed;
      scores(std::true_type{}, IC<1 - kIn>{}, nxt, req_dst, req_row, ds_unit);
      prev = cur;
      cur = nxt;
      nxt = freed;
    };
    // The compiler zeroes the accumulation registers where it likes, possibly right in front of the first matrix
    // instruction that adds to them, and does not know that those instructions (inline asm) read them: every accumulator
    // is pinned here, written, and a few wait states separate the writes from the first read.
#pragma unroll
    for (int grp = 0; grp < 2; ++grp)
#pragma unroll
      for (int mb = 0; mb < 4; ++mb) {
        asm volatile("" : "+a"(acc_v[grp][mb]));
        asm volatile("" : "+a"(acc_k[grp][mb]));
      }
    asm volatile("s_nop 7");
    iteration(IC<0>{});  // nlocal is even and at least 2: iterations 0 .. nlocal-2, an odd number of them
    for (int t = 1; t + 1 < nlocal; t += 2) {
      iteration(IC<1>{});
      iteration(IC<0>{});
    }
    // the wave's last slab (an odd one): no scores() follows that could carry its dS stores
    softmax_and_accumulate(IC<1>{}, cur, prev);
    if constexpr (kHandOver) {
      char* ds_unit = reinterpret_cast<char*>(p.ds_ws) + unit_cur;
#pragma unroll
      for (int grp = 0; grp < 2; ++grp) {
        store16_stream(ds_unit + grp * 4 * kDsUnitBytes, ho_off0, dsk[0][grp][0]);
        store16_stream_second(ds_unit + grp * 4 * kDsUnitBytes, ho_off0, dsk[0][grp][1]);
      }
    }
    // ... and its share of dV, dK (the arithmetic of this call runs on stale registers and is dropped)
    softmax_and_accumulate(IC<0>{}, nxt, cur);
    wait_vmem<0>();
    __syncthreads();  // no copy is writing LDS any more; V and the ring are free

    drain_matrix_pipe();
    // The two waves of a key group swap halves: parity 1 hands its dV part to parity 0 through the first 64 KiB of LDS,
    // parity 0 hands its dK part to parity 1 through the next 64 KiB (32 KiB per wave each).
    f32x4* send = reinterpret_cast<f32x4*>(smem + (par ? 0 : 65536) + kg * 32768) + lane;
    const f32x4* recv = reinterpret_cast<const f32x4*>(smem + (par ? 65536 : 0) + kg * 32768) + lane;
#pragma unroll
    for (int grp = 0; grp < 2; ++grp)
#pragma unroll
      for (int mb = 0; mb < 4; ++mb)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const f32x16& a = par ? acc_v[grp][mb] : acc_k[grp][mb];
          send[((grp * 4 + mb) * 4 + g) * 64] = (f32x4){a[4 * g + 0], a[4 * g + 1], a[4 * g + 2], a[4 * g + 3]};
        }
    __syncthreads();
#pragma unroll
    for (int grp = 0; grp < 2; ++grp)
#pragma unroll
      for (int mb = 0; mb < 4; ++mb)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const f32x4 r = recv[((grp * 4 + mb) * 4 + g) * 64];
          f32x16& a = par ? acc_k[grp][mb] : acc_v[grp][mb];
#pragma unroll
          for (int e = 0; e < 4; ++e) a[4 * g + e] += r[e];
        }
  }

  if (parts > 1) {
    // part of a split item: unscaled fp32 partial sums go to the workspace, dV tile (parity 0), then dK tile (parity 1)
    float* prow = p.split.ws + ((int64_t)(item - p.split.first) * parts + part) * (2 * TK * kHeadDim) + par * (TK * kHeadDim) +
                  (kg * 64 + l32) * kHeadDim;
#pragma unroll
    for (int grp = 0; grp < 2; ++grp)
#pragma unroll
      for (int mb = 0; mb < 4; ++mb)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const f32x16& a = par ? acc_k[grp][mb] : acc_v[grp][mb];
          *reinterpret_cast<f32x4*>(prow + grp * 32 * kHeadDim + 32 * mb + 8 * g + 4 * h) = (f32x4){a[4 * g + 0], a[4 * g + 1], a[4 * g + 2], a[4 * g + 3]};
        }
    return;
  }
  // parity 0 writes dV, parity 1 writes dK (both zero when no query block selects this key tile)
  __bf16* orow = (par ? p.dk : p.dv) + (krow0 + kg * 64 + l32) * kHeadDim;
  const float oscale = par ? p.scale : 1.f;
#pragma unroll
  for (int grp = 0; grp < 2; ++grp)
#pragma unroll
    for (int mb = 0; mb < 4; ++mb)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const f32x16& a = par ? acc_k[grp][mb] : acc_v[grp][mb];
        *reinterpret_cast<bf16x4*>(orow + grp * 32 * kHeadDim + 32 * mb + 8 * g + 4 * h) =
            pack4(a[4 * g + 0] * oscale, a[4 * g + 1] * oscale, a[4 * g + 2] * oscale, a[4 * g + 3] * oscale);
      }
}

hipError_t launch_bwd_dkdv64(BwdParams p, hipStream_t stream) {
  p.num_items = p.B * p.Hkv * (p.Skv / 128);
  // tail splitting (one work-group per compute unit); a part stores two 128 x 128 fp32 tiles
  void* const caller_ws = p.split.ws;  // whether or not anything is split
  p.split = plan_split(p.num_items, 1, 2 * 128 * kHeadDim * 4, p.split.ws, p.split_ws_bytes);
  plan_xcd_mapping(p.B * p.Hkv, p.split.first, p.items_per_xcd, p.split.main_wgs);
  const int split_items = p.num_items - p.split.first;
  void (*fn)(const BwdParams) = p.ds_ws != nullptr ? &dkdv64_kernel<true> : &dkdv64_kernel<false>;
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(fn), hipFuncAttributeMaxDynamicSharedMemorySize, kSmemBytes + 16);
  if (e != hipSuccess) return e;
  // Launches of several rounds with contiguous spans per XCD let the work-groups claim their grid indices, with some more
  // work-groups than indices, so that an XCD that is through early takes over from the others (claim_work).
  p.total_work = p.split.main_wgs + split_items * p.split.parts;
  int grid = p.total_work;
  p.queue = nullptr;
  if (claims_wanted(p.items_per_xcd, p.total_work, 1))
    p.queue = work_queue_in(caller_ws, p.split_ws_bytes, (int64_t)split_items * p.split.parts * 2 * 128 * kHeadDim * 4);
  if (p.queue != nullptr) {
    if ((e = launch_queue_reset(p.queue, stream)) != hipSuccess) return e;
    grid += surplus_work_groups(p.total_work);
  }
  hipLaunchKernelGGL(fn, dim3(grid), dim3(256), kSmemBytes + 16, stream, p);
  if (split_items > 0) {
    const int64_t row0 = (int64_t)p.split.first * 128;
    e = launch_partial_sum(p.split.ws, p.split.parts, 2 * 128 * kHeadDim, p.dv, row0, split_items, 1.f, stream);
    if (e != hipSuccess) return e;
    e = launch_partial_sum(p.split.ws + 128 * kHeadDim, p.split.parts, 2 * 128 * kHeadDim, p.dk, row0, split_items, p.scale, stream);
    if (e != hipSuccess) return e;
  }
  if (p.ds_ws != nullptr) {
    return launch_poison_unless_fit(p, p.dk, p.dv, (int64_t)p.B * p.Hkv * p.Skv * kHeadDim, stream);
  }
  return hipGetLastError();
}

}  // namespace fba
