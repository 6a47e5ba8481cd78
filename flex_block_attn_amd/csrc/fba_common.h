// Device-side building blocks shared by the gfx950 attention kernels: vector types, MFMA wrappers, the
// swizzled LDS tile layout and the operand fetches that go with it.
//
// LDS tile layout.  A tile is ROWS x 128 bf16, row-major, 256 bytes per row = 16 chunks of 16 bytes.  Chunk c of
// row r lives at chunk slot c ^ swz(r), swz(r) = ((r & 3) << 2) | ((r >> 2) & 3).  With 64 four-byte banks:
//   * a 128-bit row-major operand fetch (16 lanes = 16 consecutive rows, one chunk column) touches 16 distinct
//     slots, i.e. every bank once;
//   * a transposing 64-bit fetch (half a wave = 4 consecutive rows x 64 contiguous bytes) lands in 4 distinct
//     64-byte bank groups, again every bank once;
//   * the global->LDS copy (16 lanes = one row, 16 chunks) is conflict-free by construction.
//
// MFMA 32x32x16 bf16 register layouts (lane = 32*h + i):
//   A (32 x 16): row i,  k = 8h .. 8h+7          B (16 x 32): col i, k = 8h .. 8h+7
//   C (32 x 32): col i,  acc[4g + e] is row 8g + 4h + e
// The A and B layouts are the same function of (lane, k), so an accumulator whose summed index sits in the
// registers can be re-used, after bf16 packing, as either operand of the next product.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace fba {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

#define FBA_LDS __attribute__((address_space(3)))
#define FBA_CONST __attribute__((address_space(4)))
#define FBA_DEVICE __device__ __forceinline__

constexpr int kHeadDim = 128;
constexpr int kRowBytes = kHeadDim * 2;  // one bf16 row of a tile
constexpr int kWave = 64;
constexpr int kNumXcd = 8;

FBA_DEVICE int swz(int row) { return ((row & 3) << 2) | ((row >> 2) & 3); }

// byte offset of (row, chunk) inside a swizzled tile
FBA_DEVICE int tile_off(int row, int chunk) { return row * kRowBytes + ((chunk ^ swz(row)) << 4); }

FBA_DEVICE f32x16 mfma32(bf16x8 a, bf16x8 b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0); }

FBA_DEVICE bf16x8 lds_read_b128(const char* base, int off) {
  return *reinterpret_cast<const bf16x8*>(base + off);
}

// Transposing 64-bit LDS fetch.  Within each group of 16 lanes, destination lane i receives, as element j,
// element (i % 4) of the 8 bytes addressed by source lane 4*j + i/4.
FBA_DEVICE bf16x4 lds_read_tr(const char* base, int off) {
  return __builtin_amdgcn_ds_read_tr16_b64_v4bf16((FBA_LDS bf16x4*)(base + off));
}

// The same fetches through pointers into LDS.  A per-lane address that is kept as such a pointer, with the base of the
// work-group's LDS already folded in, goes into the fetch instruction as it is and constant displacements into its offset
// field; an integer offset added to `smem` at every use costs a vector add per fetch instead.
typedef const FBA_LDS char* LdsPtr;
FBA_DEVICE LdsPtr lds_ptr(const void* p) { return (LdsPtr)p; }
FBA_DEVICE bf16x8 lds_read_b128(LdsPtr p) { return *reinterpret_cast<const FBA_LDS bf16x8*>(p); }
FBA_DEVICE f32x4 lds_read_f32x4(LdsPtr p) { return *reinterpret_cast<const FBA_LDS f32x4*>(p); }
FBA_DEVICE bf16x4 lds_read_tr(LdsPtr p) { return __builtin_amdgcn_ds_read_tr16_b64_v4bf16((FBA_LDS bf16x4*)p); }

FBA_DEVICE bf16x8 cat(bf16x4 lo, bf16x4 hi) { return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7); }

// eight fp32 accumulators -> eight bf16 (round to nearest even)
FBA_DEVICE bf16x8 pack8(float a0, float a1, float a2, float a3, float a4, float a5, float a6, float a7) {
  bf16x2 p0 = __builtin_convertvector((f32x2){a0, a1}, bf16x2);
  bf16x2 p1 = __builtin_convertvector((f32x2){a2, a3}, bf16x2);
  bf16x2 p2 = __builtin_convertvector((f32x2){a4, a5}, bf16x2);
  bf16x2 p3 = __builtin_convertvector((f32x2){a6, a7}, bf16x2);
  bf16x4 lo = __builtin_shufflevector(p0, p1, 0, 1, 2, 3);
  bf16x4 hi = __builtin_shufflevector(p2, p3, 0, 1, 2, 3);
  return cat(lo, hi);
}

FBA_DEVICE bf16x4 pack4(float a0, float a1, float a2, float a3) {
  bf16x2 p0 = __builtin_convertvector((f32x2){a0, a1}, bf16x2);
  bf16x2 p1 = __builtin_convertvector((f32x2){a2, a3}, bf16x2);
  return __builtin_shufflevector(p0, p1, 0, 1, 2, 3);
}

// Exchange between the two half-waves.  v_permlane32_swap a, b exchanges the upper half of a with the lower half of b,
// so for a = b = x it leaves a = {x.lo, x.lo} and b = {x.hi, x.hi}.  Issued as inline asm: through the compiler builtin
// with two copies of one value, the two results come back as the same register.  The s_nop covers the wait states the
// instruction needs after a VALU write of its operands.
struct HalfPair {
  float lo, hi;  // value of this lane's row in the lower / upper half-wave
};
FBA_DEVICE HalfPair both_halves(float x) {
  float a = x, b = x;
  asm("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(a), "+v"(b));
  return {a, b};
}
FBA_DEVICE float max_halves(float x) {
  const HalfPair p = both_halves(x);
  return fmaxf(p.lo, p.hi);
}
FBA_DEVICE float sum_halves(float x) {
  const HalfPair p = both_halves(x);
  return p.lo + p.hi;
}

// Wait until no vector-memory load is outstanding (vmcnt = 0; expcnt and lgkmcnt fields left at their maxima).
FBA_DEVICE void wait_vmem_all() { __builtin_amdgcn_s_waitcnt(0x0F70); }

// Keep a loaded value where it is: the compiler may not sink its load below this point.
template <typename T>
FBA_DEVICE void pin(T& v) { asm volatile("" : "+v"(v)); }

FBA_DEVICE float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// Work-group id -> logical work item.  per_xcd > 0: each XCD (work-groups are dealt to the 8 XCDs round-robin) owns one
// contiguous span of per_xcd logical items, so that the items that share K/V (same batch and head) meet in one L2.
// per_xcd == 0: items in work-group order, i.e. consecutive tiles of a head dealt round-robin to the XCDs (launches with
// fewer heads than XCDs, where contiguous spans would have several XCDs stream different parts of one head at once:
// measured 13-17 % slower).
FBA_DEVICE int xcd_remap(int bid, int per_xcd) { return per_xcd > 0 ? (bid % kNumXcd) * per_xcd + bid / kNumXcd : bid; }

// Work claimed instead of given.  The hardware deals work-groups to the eight XCDs round-robin, as many to a fast XCD as to
// a slow one, and an XCD that is through with its share idles until the kernel ends.  A launch with a claim counter per XCD
// (zeroed beforehand) has some work-groups more than grid indices to do; every work-group claims an index of its own XCD
// (index = 8 k + XCD for the k-th claim there, so neighbours in the index space still meet in one L2) and, once those are
// used up, of the XCD that has most left (all shares being equal, the one that has claimed least); a work-group that finds
// nothing left exits.  Returns -1 then.  One lane calls this.
FBA_DEVICE int claim_work(int* counters, int xcd, int total) {
  int k = atomicAdd(&counters[xcd], 1);
  if (kNumXcd * k + xcd < total) return kNumXcd * k + xcd;
  // own share used up: take from the XCD that has claimed least so far, i.e. has most left
  for (int tries = 0; tries < kNumXcd; ++tries) {
    int best = -1, least = 0x7fffffff;
    for (int y = 0; y < kNumXcd; ++y) {
      const int c = __atomic_load_n(&counters[y], __ATOMIC_RELAXED);
      if (kNumXcd * c + y < total && c < least) {
        least = c;
        best = y;
      }
    }
    if (best < 0) return -1;
    k = atomicAdd(&counters[best], 1);
    if (kNumXcd * k + best < total) return kNumXcd * k + best;
  }
  return -1;
}
// XCD the wave runs on (0..7): XCC_ID field of the hardware register of that name.
FBA_DEVICE int xcd_id() { return __builtin_amdgcn_s_getreg(20 | (3 << 11)) & (kNumXcd - 1); }

// Cooperative copy of ROWS x 128 bf16 from global (row stride 256 B) into registers, then into a swizzled tile.
// 256 threads; thread t owns chunk t % 16 of rows t / 16 + 16 i.
template <int ROWS>
struct TileCopy {
  static constexpr int kIters = ROWS / 16;
  u32x4 reg[kIters];
  FBA_DEVICE void load(const __bf16* __restrict__ g, int tid) {
    const char* p = reinterpret_cast<const char*>(g) + (tid >> 4) * kRowBytes + (tid & 15) * 16;
#pragma unroll
    for (int i = 0; i < kIters; ++i) reg[i] = *reinterpret_cast<const u32x4*>(p + i * 16 * kRowBytes);
  }
  // same, from a wave-uniform byte base plus the per-thread offset (tid >> 4) * 256 + (tid & 15) * 16
  FBA_DEVICE void load(const char* __restrict__ base, uint32_t thread_off) {
#pragma unroll
    for (int i = 0; i < kIters; ++i) reg[i] = *reinterpret_cast<const u32x4*>(base + thread_off + i * 16 * kRowBytes);
  }
  // wr_off = tile_off(tid >> 4, tid & 15), precomputed by the caller
  FBA_DEVICE void store(char* tile, int wr_off) const {
#pragma unroll
    for (int i = 0; i < kIters; ++i) *reinterpret_cast<u32x4*>(tile + wr_off + i * 16 * kRowBytes) = reg[i];
  }
};

// Read-only view of a block-index list in global memory.  Loads through the constant address space stay scalar loads
// (s_load_dword) wherever they sit, also behind inline asm and barriers.
typedef const FBA_CONST int32_t* ConstIdx;
FBA_DEVICE ConstIdx const_idx(const int32_t* p) { return (ConstIdx)(uintptr_t)p; }

// Address of a __shared__ object inside the work-group's LDS allocation.
FBA_DEVICE uint32_t lds_addr(const void* p) { return (uint32_t)(uintptr_t)(FBA_LDS const char*)p; }

// Direct global -> LDS copy, 16 bytes per lane: lane l's bytes land at lds_base + 16 l; it fetches them from
// gbase + lane_off.  lds_base and gbase must be wave-uniform.  Completion is tracked by the vector-memory counter only;
// the compiler is not told that LDS changes (no memory clobber either: that would turn the scalar loads of the block
// lists into vector loads), so the caller orders the copy against LDS reads with wait_vmem<N>() and a barrier.  (M0 carries the LDS address; one wait state separates its write from the load.)
FBA_DEVICE void dma16(uint32_t lds_base, const char* gbase, uint32_t lane_off) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
               :
               : "s"(lds_base), "v"(lane_off), "s"(gbase)
               : "m0");
}

// Same copy with the streaming hint: for data that is read exactly once, so that it does not displace what other
// work-groups are about to re-read from L2.
FBA_DEVICE void dma16_stream(uint32_t lds_base, const char* gbase, uint32_t lane_off) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 nt"
               :
               : "s"(lds_base), "v"(lane_off), "s"(gbase)
               : "m0");
}

// Streaming 16-byte store per lane to gbase + lane_off with the base in scalar registers: the compiler forms 64-bit
// addresses per lane for such a store (a vector add and twice the address traffic per store), which a wave alone on its
// SIMD pays for.  gbase must be wave-uniform.  Like the copies above the store is tracked by the vector-memory counter
// only; the compiler does not know of it, so the caller orders it against whatever reads the data (nothing inside the
// kernels that use it).
FBA_DEVICE void store16_stream(char* gbase, uint32_t lane_off, bf16x8 value) {
  asm volatile("global_store_dwordx4 %0, %1, %2 nt" : : "v"(lane_off), "v"(value), "s"(gbase));
}

// The same store to gbase + (lane_off ^ 128) + 1024: where a lane's second offset differs from its first in bit 7 and by
// 1024 (ds_unit_store_off(1, lane) against ds_unit_store_off(0, lane)), it is formed here from the first instead of being
// held in a register of its own for the whole kernel.
FBA_DEVICE void store16_stream_second(char* gbase, uint32_t lane_off, bf16x8 value) {
  uint32_t second;
  asm volatile("v_xor_b32 %0, 128, %1\n\tglobal_store_dwordx4 %0, %2, %3 offset:1024 nt"
               : "=&v"(second)
               : "v"(lane_off), "v"(value), "s"(gbase));
}

// Same for 4 bytes per lane (lane l's dword lands at lds_base + 4 l).
FBA_DEVICE void dma4(uint32_t lds_base, const char* gbase, uint32_t lane_off) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2"
               :
               : "s"(lds_base), "v"(lane_off), "s"(gbase)
               : "m0");
}

// Wait until at most N vector-memory loads are outstanding (N < 64; the counter's two high bits sit in bits 15:14).
template <int N>
FBA_DEVICE void wait_vmem() { __builtin_amdgcn_s_waitcnt(0x0F70 | (N & 15) | ((N >> 4) << 14)); }

// Direct copy of a 32-row slab (32 x 128 bf16, 8 KiB) from global memory into a swizzled LDS tile by the 4 waves of a
// work-group.  A wave-level copy fills 1 KiB = 4 rows; wave w owns rows 8w .. 8w+7 (two copies).  Lane l lands in row
// 8w + 4g + l/16, chunk slot l%16, so it fetches chunk (l%16) ^ swz(row) of that row.
struct SlabDma {
  uint32_t off[2];
  uint32_t wave_dst;  // byte offset of the wave's rows inside a slab
  FBA_DEVICE void init(int wave, int lane) {
#pragma unroll
    for (int g = 0; g < 2; ++g) {
      const int row = 8 * wave + 4 * g + (lane >> 4);
      off[g] = (uint32_t)(row * kRowBytes + (((lane & 15) ^ swz(row)) << 4));
    }
    wave_dst = (uint32_t)(wave * 8 * kRowBytes);
  }
  // slab_lds: LDS address of the slab buffer; src: global address of the slab's first row (both wave-uniform)
  FBA_DEVICE void copy(uint32_t slab_lds, const char* src) const {
    dma16(slab_lds + wave_dst, src, off[0]);
    dma16(slab_lds + wave_dst + 4 * kRowBytes, src, off[1]);
  }
  // the two halves of copy(), for callers that spread them out
  FBA_DEVICE void copy_piece(int i, uint32_t slab_lds, const char* src) const {
    dma16(slab_lds + wave_dst + i * 4 * kRowBytes, src, off[i]);
  }
};

// The same copy for the two slabs (K, V) a step of a query-major kernel brings in, by the kWaves waves of its work-group.
// A wave-level copy fills 4 rows; a slab is eight of them.  kWaves = 4: wave w copies rows 8w .. 8w+7 of both slabs.
// kWaves = 12: rows 4w .. 4w+3 of the K slab by waves 0..7, rows 4(w-4) .. of the V slab by waves 4..11, so waves 4..7
// issue two copies per step and the others one.
template <int kWaves>
struct SlabDmaShared {
  static_assert(kWaves == 4 || kWaves == 12, "4 or 12 waves");
  uint32_t off[2];  // kWaves = 4: the wave's two row groups; kWaves = 12: its row group in the K slab, in the V slab
  uint32_t dst[2];
  bool has_k, has_v;
  FBA_DEVICE static uint32_t lane_off(int row_group, int lane) {
    const int row = 4 * row_group + (lane >> 4);
    return (uint32_t)(row * kRowBytes + (((lane & 15) ^ swz(row)) << 4));
  }
  FBA_DEVICE void init(int wave, int lane) {
    if constexpr (kWaves == 4) {
      has_k = has_v = true;
      off[0] = lane_off(2 * wave, lane);
      off[1] = lane_off(2 * wave + 1, lane);
      dst[0] = (uint32_t)(2 * wave * 4 * kRowBytes);
      dst[1] = dst[0] + 4 * kRowBytes;
    } else {
      has_k = wave < 8;
      has_v = wave >= 4;
      const int gk = wave & 7, gv = (wave - 4) & 7;
      off[0] = lane_off(gk, lane);
      off[1] = lane_off(gv, lane);
      dst[0] = (uint32_t)(gk * 4 * kRowBytes);
      dst[1] = (uint32_t)(gv * 4 * kRowBytes);
    }
  }
  FBA_DEVICE void copy_k(uint32_t slab_lds, const char* src) const {
    if constexpr (kWaves == 4) {
      dma16(slab_lds + dst[0], src, off[0]);
      dma16(slab_lds + dst[1], src, off[1]);
    } else {
      if (has_k) dma16(slab_lds + dst[0], src, off[0]);
    }
  }
  FBA_DEVICE void copy_v(uint32_t slab_lds, const char* src) const {
    if constexpr (kWaves == 4) {
      copy_k(slab_lds, src);
    } else {
      if (has_v) dma16(slab_lds + dst[1], src, off[1]);
    }
  }
  // Piece i (0 or 1) of the wave's share of a slab copy with four waves, for callers that spread the pieces out.
  FBA_DEVICE void copy_piece(int i, uint32_t slab_lds, const char* src) const {
    static_assert(kWaves == 4, "pieces exist with four waves only");
    dma16(slab_lds + dst[i], src, off[i]);
  }
  // Wait until only the copies this wave issued during the last two steps (one K and one V request each) may be in flight.
  FBA_DEVICE void wait_two_steps() const {
    if constexpr (kWaves == 4) {
      wait_vmem<8>();
    } else {
      if (has_k && has_v) wait_vmem<4>(); else wait_vmem<2>();
    }
  }
};

// Per-lane LDS offsets for row-major A/B operand fetches of a 32-row slab: rd[ks] addresses row (lane % 32),
// chunk 2*ks + lane/32.  Add 32*kRowBytes per further slab (rows stay congruent mod 16, so swz is unchanged).
struct RowMajorOffsets {
  int rd[8];
  FBA_DEVICE void init(int lane) {
    const int r = lane & 31, h = lane >> 5;
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) rd[ks] = tile_off(r, 2 * ks + h);
  }
};

// Per-lane LDS offsets for transposed operand fetches.  A fetch covers 4 rows (the summed index) x 64 columns...
// For a 16-wide slice of the summed index starting at row R (R % 16 == 0) and column block cb (32 columns), the lane
// issues two fetches: rows R + 4h + (lane/4)%4 and the same + 8; columns 32*cb + 16*((lane/16)%2) + 4*(lane%4).
// The two fetches give k = 8h+0..3 and 8h+4..7 of an operand whose row/col index is 32*cb + lane%32, provided the other
// operand enumerates the summed index as  R + 8*(t/4) + 4h + t%4  for t = 0..7 (which is exactly the order the 32x32
// accumulator layout hands its rows out in).
struct TransposedOffsets {
  int rd[4][2];  // [column block][+8 rows]
  FBA_DEVICE void init(int lane) {
    const int h = lane >> 5;
    const int rl = 4 * h + ((lane >> 2) & 3);
    const int cl = 2 * ((lane >> 4) & 1) + ((lane & 3) >> 1);
    const int inner = (lane & 1) * 8;
#pragma unroll
    for (int cb = 0; cb < 4; ++cb) {
      rd[cb][0] = tile_off(rl, 4 * cb + cl) + inner;
      rd[cb][1] = tile_off(rl + 8, 4 * cb + cl) + inner;
    }
  }
};

// dS hand-over between the key-major and the query-major backward kernel.  A "unit" is dS of one 32-query slab
// against 32 keys, 2 KiB of bf16, cut into 256 slots of 8 bytes: slot (key, u) holds dS[4u .. 4u+3][key].  In the
// key-major kernel lane (key = lane % 32, h = lane / 32) holds, as packed register chunk j, the slots u = 4j + h and
// u = 4j + 2 + h of its key, 16 bytes.  It stores chunk j at byte offset ds_unit_store_off(j, lane): every 16 lanes
// fill one contiguous 256 bytes (whole cache lines per pass of the store), and the rotation by 4 h + 8 j inside those
// 256 bytes spreads the slots that one transposing 64-bit LDS fetch of the query-major kernel touches (4 keys x both h
// x both halves, for two values of j per half-wave) over all 64 banks.
FBA_DEVICE int ds_unit_store_off(int j, int lane) {
  const int key = lane & 31, h = lane >> 5;
  return j * 1024 + (lane >> 4) * 256 + ((((key & 15) + 4 * h + 8 * j) & 15) << 4);
}
// Byte offset of slot (key, u) inside a unit.
FBA_DEVICE int ds_unit_slot_off(int key, int u) {
  const int j = u >> 2, half = (u >> 1) & 1, h = u & 1;
  return j * 1024 + (2 * h + (key >> 4)) * 256 + ((((key & 15) + 4 * h + 8 * j) & 15) << 4) + half * 8;
}
// Units of one block pair (q_block x k_block) are ordered for the reader: unit ((tq * (k_block / 32) + t) * 4 + w) is
// 32-query slab 4 tq + w of the query block against 32-key slab t of the key block, so a 128-row query tile tq reads its
// whole share of the pair as one ascending stream, 8 KiB (four units, one per wave) per 32-key step.
constexpr int kDsUnitBytes = 2048;

// Do the pairs that the lists of a hand-over call number fit the workspace?  P is BwdParams: pair_base holds the exclusive
// prefix sums of the rows this call covers (rows + 1 entries); the workspace pointer is where pair 0 would live, the call
// touches the pairs from pair_base[0] up to pair_base[rows], once per (batch, head) when all share one mask.
template <typename P>
FBA_DEVICE bool workspace_holds_lists(const P& p) {
  const ConstIdx pb = const_idx(p.pair_base);
  const int64_t rows = p.mask_bh * (p.tiled ? p.Skv / 128 : p.nK);
  const int64_t listed = (int64_t)(pb[rows] - pb[0]) * (p.mask_bh == 1 ? (int64_t)p.B * p.Hq : 1);
  return listed <= p.ws_pairs;
}

}  // namespace fba
