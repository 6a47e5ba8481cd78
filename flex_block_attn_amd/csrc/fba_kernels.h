// Host-visible parameter blocks and launchers of the gfx950 kernels.  Internal to the shared library; the public
// surface is the C ABI in include/fba.h.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace fba {

// Active-block lists, as produced by the compaction kernel.
//   q_cnt [mask_bh, nQ], q_idx [mask_bh, nQ, nK]: for every query block the ascending selected key blocks.
//   k_cnt [mask_bh, nK], k_idx [mask_bh, nK, nQ]: for every key block the ascending query blocks that select it.
// mask_bh is B*Hq, or 1 when one 2-D mask is shared by every (batch, head).

// Tail splitting.  Work-groups are handed to free slots in index order, so the last (items % slots) items of a launch
// would run as a partial round with most compute units idle.  With a workspace, those items are cut into `parts` ranges of
// their lists, each run by its own work-group at the end of the grid; the work-groups store fp32 partial results into the
// workspace and a small merge kernel combines them in a fixed order.  Items [0, first) run whole.
struct SplitPlan {
  float* ws;      // null: nothing is split
  int first;      // first item that is split
  int parts;      // work-groups per split item (>= 2 when ws is set)
  int main_wgs;   // work-groups in front of the split ones (a multiple of the XCD count)
};

// Items and work-group slots of a launch -> plan (first = num_items, parts = 1 when nothing is split).  `slot_bytes` is
// what one part stores; the workspace must hold (num_items - first) * parts of them.  main_wgs is left to the launcher.
SplitPlan plan_split(int num_items, int wgs_per_cu, int64_t slot_bytes, void* ws, int64_t ws_bytes);

// How the whole items of a launch are dealt to the XCDs (see xcd_remap): contiguous spans when the launch has at least
// one (batch, head) per XCD, work-group order otherwise.  Sets items_per_xcd and the number of work-groups that come
// before the split ones.
inline void plan_xcd_mapping(int heads, int whole_items, int& items_per_xcd, int& main_wgs) {
  constexpr int kXcds = 8;
  if (heads >= kXcds) {
    items_per_xcd = (whole_items + kXcds - 1) / kXcds;
    main_wgs = items_per_xcd * kXcds;
  } else {
    items_per_xcd = 0;
    main_wgs = whole_items;
  }
}

constexpr int kSplitMaxSlots = 512;                           // two work-groups on each of 256 compute units
constexpr int64_t kSplitSlotBytes = 128 * 128 * 4 * 2;        // dK and dV partials of a key tile; forward: O^T + (m, l)
constexpr int64_t kSplitWsBytes = (kSplitMaxSlots / 2) * kSplitSlotBytes + (1 << 20);

struct FwdParams {
  const __bf16* q;
  const __bf16* k;
  const __bf16* v;
  __bf16* o;
  float* lse;  // [B, Hq, Sq], natural log
  const int32_t* q_cnt;
  const int32_t* q_idx;
  int64_t mask_bh;
  int B, Hq, Hkv, Sq, Skv, nQ, nK, q_block, k_block;
  float scale_log2e;  // log2(e) / sqrt(head_dim)
  int num_items, items_per_xcd;
  // tiled = 1: q_cnt / q_idx are tile lists (qt_cnt [mask_bh, Sq/128], qt_ent [mask_bh, Sq/128, nK], see
  // tile_lists_kernel) instead of block lists
  int tiled;
  int64_t split_ws_bytes;  // size of split.ws as handed in by the caller
  int variant;  // 0: 384-row work-groups where q_block allows (measurement of that variant); 1: 128-row work-groups
  SplitPlan split;
};

struct BwdParams {
  const __bf16* q;
  const __bf16* k;
  const __bf16* v;
  const __bf16* d_o;
  const float* stats;  // [2, B, Hq, Sq]: lse * log2(e), then -delta = -rowsum(dO o O)
  __bf16* dq;
  __bf16* dk;
  __bf16* dv;
  const int32_t* q_cnt;
  const int32_t* q_idx;
  const int32_t* k_cnt;
  const int32_t* k_idx;
  int64_t mask_bh;
  int B, Hq, Hkv, Sq, Skv, nQ, nK, q_block, k_block;
  float scale;        // 1 / sqrt(head_dim)
  float scale_log2e;  // log2(e) / sqrt(head_dim)
  int num_items, items_per_xcd;
  // tiled = 1: q_cnt / q_idx are qt_cnt / qt_ent and k_cnt / k_idx are kt_cnt [mask_bh, Skv/128] /
  // kt_ent [mask_bh, Skv/128, Sq/32] (see tile_lists_kernel)
  int tiled;
  // dS hand-over (null when unused).  The key-major kernel stores dS of every selected block pair into ds_ws and the
  // query-major kernel reads it back instead of recomputing S and dP.  Block lists:
  //   pair_base [mask_bh * nK + 1]: exclusive prefix sum of k_cnt; the last entry is the number of pairs in the lists
  //   q_slot    [mask_bh, nQ, nK]:  pair number of entry e of query block I, i.e. pair_base[m, J] + position of I in
  //                                 k_idx[m, J, :] for J = q_idx[m, I, e]; -1 beyond q_cnt
  // Pair n of head bh lives at ds_ws + (n + (mask_bh == 1 ? bh * pairs : 0)) * q_block * k_block * 2 bytes.
  // Tile lists (see tile_slots_kernel): the pairs are (128-row query tile, 128-key tile) pairs of 32 KiB,
  //   pair_base [mask_bh * Skv/128 + 1]:        exclusive prefix sum of the listed tile pairs per key tile
  //   k_slot    [mask_bh, Skv/128, Sq/32]:      pair number of every kt_ent entry
  //   q_slot    [mask_bh, Sq/128, Skv/128]:     pair number of (query tile, key tile), -1 where nothing is listed
  //   zero_unit: 2 KiB of zeros in device memory, read in place of a dS unit that no wave stored
  __bf16* ds_ws;
  int64_t ws_pairs;  // pairs ds_ws has room for
  const int32_t* pair_base;
  const int32_t* q_slot;
  const int32_t* k_slot;
  const char* zero_unit;
  SplitPlan split;
  // dkdv64_kernel: claim counters, one per XCD, in the caller's tail-splitting workspace (null: work-group i does grid
  // index i), and the number of grid indices there are to claim (see claim_work)
  int* queue;
  int total_work;
  int64_t split_ws_bytes;  // size of split.ws as handed in by the caller
};

hipError_t launch_mask_compact(const uint8_t* mask, int64_t mask_bh, int nQ, int nK, int32_t* q_cnt, int32_t* q_idx,
                               int32_t* k_cnt, int32_t* k_idx, hipStream_t stream);
hipError_t launch_tile_lists(const uint8_t* mask, int64_t mask_bh, int nQ, int nK, int q_block, int k_block, int n_qt,
                             int n_kt, int n_qs, int32_t* qt_cnt, int32_t* qt_ent, int32_t* kt_cnt, int32_t* kt_ent,
                             hipStream_t stream);
hipError_t launch_block_mean(const __bf16* x, float* out, int64_t n_blocks, int block, hipStream_t stream);
hipError_t launch_ssta_mask(const float* q_mean, const float* k_mean, const uint8_t* base, uint8_t* mask, int64_t BH, int Hq, int Hkv, int nQ,
                            int nK, int q_block, int k_block, int topk, int band, int sink, hipStream_t stream);
hipError_t launch_tile_permute(const void* x, void* out, int64_t n_seq, int T, int H, int W, int tT, int tH, int tW,
                               int to_tiles, hipStream_t stream);
hipError_t launch_fwd(FwdParams p, hipStream_t stream);
hipError_t launch_bwd_stats(const __bf16* o, const __bf16* d_o, const float* lse, float* stats, int64_t rows, hipStream_t stream);
hipError_t launch_bwd_dq(BwdParams p, hipStream_t stream);
hipError_t launch_bwd_dkdv(BwdParams p, hipStream_t stream);
hipError_t launch_bwd_dkdv64(BwdParams p, hipStream_t stream);  // block lists only: 64 keys per wave, one wave per SIMD
hipError_t launch_bwd_dq_from_ds(BwdParams p, hipStream_t stream);
// The lists of a hand-over call live in device memory, so only kernels can tell whether the pairs they number fit the
// workspace.  Every kernel that stores or fetches dS tests it first (workspace_holds_lists, fba_common.h) and returns at
// once when they do not; this launch then fills `n` bf16 values at `out_a` (and at `out_b` unless null) with NaN, so that
// the call fails loudly instead of writing out of bounds.
hipError_t launch_poison_unless_fit(const BwdParams& p, __bf16* out_a, __bf16* out_b, int64_t n, hipStream_t stream);
// Room for the claim counters behind `partial_bytes` of partial results in a tail-splitting workspace (null if there is
// none), and the launch that zeroes them.
int* work_queue_in(void* ws, int64_t ws_bytes, int64_t partial_bytes);
// Is a launch of `total_work` grid indices at `wgs_per_cu` work-groups per compute unit worth claiming?  (At least four
// rounds; FBA_CLAIM_WORK=0 in the environment switches claiming off, for measurements.)
bool claims_wanted(int items_per_xcd, int total_work, int wgs_per_cu);
// Work-groups launched on top of the grid indices of a claiming launch: an eighth more, a whole number per XCD.
inline int surplus_work_groups(int total_work) { return (total_work / 8 + 7) / 8 * 8; }
hipError_t launch_queue_reset(int* queue, hipStream_t stream);
int device_compute_units();
hipError_t launch_partial_sum(const float* ws, int parts, int64_t slot_floats, __bf16* out, int64_t out_row0, int n_items, float scale,
                              hipStream_t stream);
hipError_t launch_probe_mfma(const float* src, float* sink, int work_groups, int iters, hipStream_t stream);
hipError_t launch_probe_read(const void* src, int64_t bytes, uint32_t* sink, int work_groups, hipStream_t stream);
hipError_t launch_pair_slots(const int32_t* q_cnt, const int32_t* q_idx, const int32_t* k_cnt, const int32_t* k_idx, int64_t mask_bh,
                             int nQ, int nK, int32_t* pair_base, int32_t* q_slot, hipStream_t stream);
hipError_t launch_tile_slots(const int32_t* kt_cnt, const int32_t* kt_ent, int64_t mask_bh, int n_qt, int n_kt, int n_qs,
                             int32_t* pair_base, int32_t* kt_slot, int32_t* slot_table, hipStream_t stream);

}  // namespace fba
