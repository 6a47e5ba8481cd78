/*
 * C ABI of the gfx950 block-sparse attention library (libfba_gfx950.so).
 *
 * The library replaces the compiled half of the reference operator: the pybind11 module `flex_block_attn_cuda`
 * (attn.cpp:25-31) with its two entry points attn_forward / attn_backward, whose host launchers live at
 * flex_block_attn/flex_block_attn_h100.cu:810-1007 and :1009-1267.  Differences in contract:
 *   - plain pointers and sizes, no torch types; the caller owns every buffer (the reference allocates its outputs
 *     with torch::empty / torch::zeros, flex_block_attn_h100.cu:865-874, :1077-1093);
 *   - everything is enqueued on the HIP stream passed in and nothing synchronises the device (the reference brackets
 *     every launch with cudaDeviceSynchronize, :882, :1004-1005, :1113, :1212-1213);
 *   - the block mask is consumed as compacted index lists produced by fba_mask_compact rather than rescanned by
 *     every work-group (:134-135, :247-248, :672, :738); the transposed lists replace the transposed mask copies of
 *     flex_block_attn/flex_block_attn_interface.py:85-86;
 *   - gradients are written as bf16 directly (the reference returns fp32 buffers filled by reducing stores).
 *
 * Tensor layout, as in the reference (flex_block_attn_h100.cu:820-858): q [B, Hq, Sq, 128], k and v
 * [B, Hkv, Skv, 128], o like q; bf16, contiguous, 16-byte aligned.  lse and delta are fp32 [B, Hq, Sq].
 * Hq must be a multiple of Hkv (:843-844); kv head = q head / (Hq / Hkv).
 *
 * Every function returns FBA_OK or an error code; fba_last_error() gives the message of the calling thread's last
 * failure.  No function throws or aborts.
 */
#ifndef FBA_H_
#define FBA_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FBA_OK 0
#define FBA_ERR_INVALID 1     /* an argument violates the contract (shape, alignment, null pointer) */
#define FBA_ERR_UNSUPPORTED 2 /* valid for the operator, but no kernel variant covers it yet */
#define FBA_ERR_HIP 3         /* a HIP runtime call failed */

/* Library version: major * 1000 + minor; the minor number goes up whenever an argument list in this header changes, so a
 * binding can refuse a library built from another header (flex_block_attn_amd/_lib.py does). */
#define FBA_VERSION 2003
int32_t fba_version(void);

/* Message for the last non-OK return on the calling thread ("" if none). The pointer stays valid until the next
 * failing call on the same thread. */
const char* fba_last_error(void);

/*
 * Mask compaction.  Replaces the per-CTA mask scans of flex_block_attn_h100.cu:110, :134, :171, :247 (forward) and
 * :645, :672, :703, :738, :780 (backward, on the transposed mask).
 *   mask     [mask_bh, nQ, nK] bytes, non-zero = selected; mask_bh = B*Hq, or 1 for one mask shared by all (b, h)
 *   q_cnt    [mask_bh, nQ]        number of selected key blocks of each query block
 *   q_idx    [mask_bh, nQ, nK]    their indices, ascending, padded with -1
 *   k_cnt    [mask_bh, nK]        number of query blocks selecting each key block
 *   k_idx    [mask_bh, nK, nQ]    their indices, ascending, padded with -1
 */
int32_t fba_mask_compact(const uint8_t* mask, int64_t mask_bh, int32_t nQ, int32_t nK, int32_t* q_cnt, int32_t* q_idx,
                         int32_t* k_cnt, int32_t* k_idx, void* hip_stream);

/*
 * Tail splitting (no counterpart in the reference).  Work-groups are handed to free compute-unit slots in index order,
 * so the last (items % slots) 128-row tiles of a launch would run as a partial round with most of the GPU idle; the same
 * holds for a whole launch with fewer tiles than slots.  Entry points that take `split_ws` cut the lists of those tiles
 * into up to eight ranges, run each range in a work-group of its own at the end of the grid, store fp32 partial results
 * into split_ws and combine them in a small second launch, in a fixed order (results stay bit-reproducible).
 *   split_ws        null (nothing is split), or 16-byte aligned device memory owned by the caller for the duration of
 *                   the call's work on the stream; its contents before and after are meaningless
 *   split_ws_bytes  its size; fba_split_workspace_bytes() is what the planner can use at most (a smaller buffer limits
 *                   the number of ranges, never correctness)
 * On tile lists forward and the dK/dV kernel split; the dQ kernels do not.
 * The same workspace lends its last 256 bytes (when they lie behind the partial results) to the dK/dV kernels of launches of
 * four rounds and more: eight counters, zeroed by a one-wave launch in front, from which the work-groups claim the tile they
 * work on, with an eighth more work-groups launched than there are tiles.  The hardware deals work-groups to the eight
 * XCDs in equal numbers; with claims an XCD that is through with its share takes over tiles of the others instead of
 * idling.  Which work-group computes a tile does not enter the result.
 */
int64_t fba_split_workspace_bytes(void);

/*
 * Forward.  Replaces attn_forward (attn.cpp:29, flex_block_attn_h100.cu:810-1007; kernel :52-318).
 * Writes o (bf16) and lse (fp32, natural log of the row's softmax denominator including the 1/sqrt(128) scale;
 * -inf and o = 0 for a query block with an empty list).  nQ = Sq / q_block, nK = Skv / k_block.
 * Needs q_block and k_block to be multiples of 128 (otherwise FBA_ERR_UNSUPPORTED: use fba_tile_lists + fba_fwd_tiled).
 */
int32_t fba_fwd(const void* q, const void* k, const void* v, void* o, float* lse, const int32_t* q_cnt,
                const int32_t* q_idx, int64_t mask_bh, int32_t B, int32_t Hq, int32_t Hkv, int32_t Sq, int32_t Skv,
                int32_t head_dim, int32_t q_block, int32_t k_block,
                void* split_ws, int64_t split_ws_bytes, void* hip_stream);

/*
 * Backward, three stream-ordered launches.  Replaces attn_backward (attn.cpp:30,
 * flex_block_attn_h100.cu:1009-1267): bwd_attend_prep_ker (:324-389) and bwd_attend_ker (:572-802).
 *   stats    [2, B, Hq, Sq] fp32 workspace written by the call: lse * log2(e), then -delta = -rowsum(dO o O)
 *   dq       [B, Hq, Sq, 128] bf16;  dk, dv [B, Hkv, Skv, 128] bf16 (summed over the query heads of a GQA group)
 * Every output element is written exactly once; no buffer needs clearing beforehand.
 */
int32_t fba_bwd(const void* q, const void* k, const void* v, const void* o, const void* d_o, const float* lse,
                float* stats, void* dq, void* dk, void* dv, const int32_t* q_cnt, const int32_t* q_idx,
                const int32_t* k_cnt, const int32_t* k_idx, int64_t mask_bh, int32_t B, int32_t Hq, int32_t Hkv,
                int32_t Sq, int32_t Skv, int32_t head_dim, int32_t q_block, int32_t k_block,
                void* split_ws, int64_t split_ws_bytes, void* hip_stream);

/* The three stages of fba_bwd, separately (for profiling one kernel at a time); rows = B * Hq * Sq. */
int32_t fba_bwd_stats(const void* o, const void* d_o, const float* lse, float* stats, int64_t rows, int32_t head_dim,
                      void* hip_stream);
int32_t fba_bwd_dq(const void* q, const void* k, const void* v, const void* d_o, const float* stats, void* dq,
                   const int32_t* q_cnt, const int32_t* q_idx, int64_t mask_bh, int32_t B, int32_t Hq, int32_t Hkv,
                   int32_t Sq, int32_t Skv, int32_t head_dim, int32_t q_block, int32_t k_block,
                   void* split_ws, int64_t split_ws_bytes, void* hip_stream);
int32_t fba_bwd_dkdv(const void* q, const void* k, const void* v, const void* d_o, const float* stats, void* dk, void* dv,
                     const int32_t* k_cnt, const int32_t* k_idx, int64_t mask_bh, int32_t B, int32_t Hq, int32_t Hkv,
                     int32_t Sq, int32_t Skv, int32_t head_dim, int32_t q_block, int32_t k_block,
                     void* split_ws, int64_t split_ws_bytes, void* hip_stream);

/*
 * Backward with dS handed over in memory.  fba_bwd computes S and dP twice, once in the key-major kernel (dK, dV) and
 * once in the query-major kernel (dQ), because no kernel may add into rows it does not own.  The reference avoids the
 * second computation with reducing stores into fp32 dQ (flex_block_attn_h100.cu:707-708); fp32 atomic adds run at
 * about 1.4 TB/s on this GPU, far too slow for that.  Here the key-major kernel instead stores the bf16 dS of every
 * selected block pair once into `ds_ws` and a light query-major kernel forms dQ = dS K from it: ten products per pair
 * instead of fourteen, still no atomics, bit-reproducible, at the price of the workspace.  Block lists only
 * (q_block and k_block multiples of 128).
 *   fba_pair_slots   numbers the pairs: pair_base [mask_bh * nK + 1] = exclusive prefix sum of k_cnt (last entry =
 *                    number of pairs in the lists), q_slot [mask_bh, nQ, nK] = the pair number of every q_idx entry
 *                    (-1 beyond q_cnt).
 *   ds_ws            n_pairs * q_block * k_block bf16, 16-byte aligned; n_pairs = selected pairs over all (batch,
 *                    head): the sum of k_cnt, times B * Hq when mask_bh == 1.  ds_ws_bytes is its size.  The lists live
 *                    in device memory and are not read back, so the host cannot tell whether they belong to this
 *                    n_pairs; the kernels can: the call touches the pairs from pair_base[0] up to the last entry of
 *                    pair_base (times B * Hq when mask_bh == 1), and if ds_ws_bytes does not hold that many, no kernel
 *                    stores or fetches any dS and dq, dk, dv come back filled with NaN (the return code stays FBA_OK).
 *                    q_slot must come from the same fba_pair_slots call as pair_base.
 * Every head's dS is independent: a caller short of memory may run these entry points once per group of kv heads through
 * one smaller workspace, with all pointers moved to the group's first head (B = 1) and ds_ws moved back by the pairs in
 * front of the group when the mask is per head (the pair numbers in the lists are absolute).
 * Other arguments as fba_bwd; dq, dk, dv agree with fba_bwd's to within bf16 rounding of dS (dk, dv bit for bit).
 */
int32_t fba_pair_slots(const int32_t* q_cnt, const int32_t* q_idx, const int32_t* k_cnt, const int32_t* k_idx, int64_t mask_bh,
                       int32_t nQ, int32_t nK, int32_t* pair_base, int32_t* q_slot, void* hip_stream);
int32_t fba_bwd_handover(const void* q, const void* k, const void* v, const void* o, const void* d_o, const float* lse, float* stats,
                         void* ds_ws, int64_t ds_ws_bytes, void* dq, void* dk, void* dv, const int32_t* q_cnt, const int32_t* q_idx,
                         const int32_t* k_cnt, const int32_t* k_idx, const int32_t* pair_base, const int32_t* q_slot, int64_t n_pairs,
                         int64_t mask_bh, int32_t B, int32_t Hq, int32_t Hkv, int32_t Sq, int32_t Skv, int32_t head_dim,
                         int32_t q_block, int32_t k_block,
                         void* split_ws, int64_t split_ws_bytes, void* hip_stream);
/* Its two attention stages separately (after fba_bwd_stats), for profiling one kernel at a time. */
int32_t fba_bwd_dkdv_handover(const void* q, const void* k, const void* v, const void* d_o, const float* stats, void* dk, void* dv,
                              void* ds_ws, int64_t ds_ws_bytes, const int32_t* k_cnt, const int32_t* k_idx, const int32_t* pair_base,
                              int64_t n_pairs, int64_t mask_bh, int32_t B, int32_t Hq, int32_t Hkv, int32_t Sq, int32_t Skv,
                              int32_t head_dim, int32_t q_block, int32_t k_block,
                              void* split_ws, int64_t split_ws_bytes, void* hip_stream);
int32_t fba_bwd_dq_from_ds(const void* k, const void* ds_ws, int64_t ds_ws_bytes, void* dq, const int32_t* q_cnt, const int32_t* q_idx,
                           const int32_t* q_slot, const int32_t* pair_base, int64_t n_pairs, int64_t mask_bh, int32_t B, int32_t Hq,
                           int32_t Hkv, int32_t Sq, int32_t Skv, int32_t head_dim, int32_t q_block, int32_t k_block,
                           void* split_ws, int64_t split_ws_bytes, void* hip_stream);

/*
 * fba_bwd without the `stats` argument, for callers that cannot allocate device memory (tight serving loops, harnesses
 * that forbid hipMalloc).  It has no counterpart in the reference, whose host launcher
 * allocates with torch (flex_block_attn_h100.cu:1077-1093).  The statistics live in a 32 MiB array that is part of the
 * library's device image, so the call allocates and frees nothing; it serves up to 4 194 304 query rows
 * (B * Hq * Sq <= 2^22) and returns FBA_ERR_UNSUPPORTED beyond that.  Every call on a GPU uses that GPU's one array:
 * calls that overlap on one GPU (two streams, two threads) race on it; calls ordered on one stream do not.  Results
 * are bit-identical to fba_bwd's.
 */
int32_t fba_bwd_noalloc(const void* q, const void* k, const void* v, const void* o, const void* d_o, const float* lse,
                        void* dq, void* dk, void* dv, const int32_t* q_cnt, const int32_t* q_idx, const int32_t* k_cnt,
                        const int32_t* k_idx, int64_t mask_bh, int32_t B, int32_t Hq, int32_t Hkv, int32_t Sq, int32_t Skv,
                        int32_t head_dim, int32_t q_block, int32_t k_block, void* hip_stream);

/*
 * Block sizes that are not multiples of 128 (the reference allows any q_block % 16 == 0 and kv_block % 64 == 0,
 * flex_block_attn_interface.py:18-20; its kernels handle them with a second, finer mask and -inf fills,
 * flex_block_attn_h100.cu:166-243, :512-522).  Here the kernels keep their 128-row tiles and consume tile lists whose
 * entries carry predicates; Sq and Skv must be multiples of 128.
 *   qt_cnt   [mask_bh, Sq/128]         entries per 128-row query tile
 *   qt_ent   [mask_bh, Sq/128, nK]     (J << 8) | bits, ascending J; bit g: 16-row group g of the tile selects key block J
 *   kt_cnt   [mask_bh, Skv/128]        entries per 128-row key tile
 *   kt_ent   [mask_bh, Skv/128, Sq/32] (s << 8) | bits, ascending s; bit 2w+f: keys 32w..32w+31 of the tile are selected by
 *                                      rows 16f..16f+15 of the 32-row query slab s
 * Unused entries are -1.  fba_fwd_tiled / fba_bwd_tiled take these lists and are otherwise fba_fwd / fba_bwd.
 */
int32_t fba_tile_lists(const uint8_t* mask, int64_t mask_bh, int32_t nQ, int32_t nK, int32_t q_block, int32_t k_block,
                       int32_t* qt_cnt, int32_t* qt_ent, int32_t* kt_cnt, int32_t* kt_ent, void* hip_stream);
int32_t fba_fwd_tiled(const void* q, const void* k, const void* v, void* o, float* lse, const int32_t* qt_cnt,
                      const int32_t* qt_ent, int64_t mask_bh, int32_t B, int32_t Hq, int32_t Hkv, int32_t Sq, int32_t Skv,
                      int32_t head_dim, int32_t q_block, int32_t k_block,
                      void* split_ws, int64_t split_ws_bytes, void* hip_stream);
int32_t fba_bwd_tiled(const void* q, const void* k, const void* v, const void* o, const void* d_o, const float* lse,
                      float* stats, void* dq, void* dk, void* dv, const int32_t* qt_cnt, const int32_t* qt_ent,
                      const int32_t* kt_cnt, const int32_t* kt_ent, int64_t mask_bh, int32_t B, int32_t Hq, int32_t Hkv,
                      int32_t Sq, int32_t Skv, int32_t head_dim, int32_t q_block, int32_t k_block,
                      void* split_ws, int64_t split_ws_bytes, void* hip_stream);

/*
 * fba_bwd_tiled with dS handed over in memory, as fba_bwd_handover does for block lists (the reference's counterpart
 * are the reducing stores into fp32 dQ, flex_block_attn_h100.cu:707-708).  The workspace is divided into pairs of a
 * 128-row query tile and a 128-key tile (32 KiB of bf16 dS each); only the 2 KiB units whose rows select their keys are
 * written and read.
 *   fba_tile_slots  numbers the listed tile pairs: pair_base [mask_bh * Skv/128 + 1] = exclusive prefix sum of the
 *                   distinct query tiles in every kt_ent row (last entry = number of pairs in the lists), kt_slot
 *                   [mask_bh, Skv/128, Sq/32] = pair number of every kt_ent entry (-1 beyond kt_cnt), slot_table
 *                   [mask_bh, Sq/128, Skv/128] = pair number of (query tile, key tile), -1 where nothing is listed.
 *                   n_qt = Sq/128, n_kt = Skv/128.
 *   ds_ws           n_pairs * 32 KiB, 16-byte aligned; n_pairs = listed tile pairs over all (batch, head): the last
 *                   entry of pair_base, times B * Hq when mask_bh == 1.  As for fba_bwd_handover, lists that number more
 *                   pairs than ds_ws_bytes holds leave the workspace untouched and dq, dk, dv filled with NaN.
 * Other arguments as fba_bwd_tiled; dk, dv agree with fba_bwd_tiled's bit for bit, dq to within bf16 rounding of dS.
 */
int32_t fba_tile_slots(const int32_t* kt_cnt, const int32_t* kt_ent, int64_t mask_bh, int32_t n_qt, int32_t n_kt, int32_t* pair_base,
                       int32_t* kt_slot, int32_t* slot_table, void* hip_stream);
int32_t fba_bwd_tiled_handover(const void* q, const void* k, const void* v, const void* o, const void* d_o, const float* lse, float* stats,
                               void* ds_ws, int64_t ds_ws_bytes, void* dq, void* dk, void* dv, const int32_t* qt_cnt,
                               const int32_t* qt_ent, const int32_t* kt_cnt, const int32_t* kt_ent, const int32_t* pair_base,
                               const int32_t* kt_slot, const int32_t* slot_table, int64_t n_pairs, int64_t mask_bh, int32_t B,
                               int32_t Hq, int32_t Hkv, int32_t Sq, int32_t Skv, int32_t head_dim, int32_t q_block, int32_t k_block,
                               void* split_ws, int64_t split_ws_bytes, void* hip_stream);

/*
 * Callers' side of the operator for video models.  The reference names these steps but never released them
 * (create_sta_3d_mask, create_ssta_3d_mask, create_moba_3d_mask, ssta_3d_attention: flex_block_attn/__init__.py:7-12,
 * README.md:54-55); they are specified here and checked against their own CPU restatement.
 *
 * fba_block_mean: out[s, g, :] = mean of rows g*block .. (g+1)*block-1 of x[s], x [n_seq, S, 128] bf16, out
 *   [n_seq, S/block, 128] fp32.
 * fba_ssta_mask: mask[b, h, i, j] (bool bytes, [B, Hq, nQ, nK]) = j is one of the `topk` key blocks with the largest
 *   <q_mean[b,h,i], k_mean[b, h / (Hq/Hkv), j]> (equal scores: lower j first), or |j - (i*q_block)/k_block| <= band, or
 *   j < sink, or base[i, j] (base: bool bytes [nQ, nK] shared by every (b, h), e.g. a sliding-tile mask; may be null).
 *   band = -1 switches the band off.  nK <= 4096 (FBA_ERR_UNSUPPORTED beyond).
 * fba_tile_permute: moves 256-byte token rows of x [n_seq, T*H*W, 128] bf16 between raster order of the (T, H, W) grid
 *   and tile order (tiles of tile_t x tile_h x tile_w tokens, tiles in raster order of the tile grid, tokens in raster
 *   order inside a tile), so that one tile is one contiguous block of the attention; to_tiles = 0 is the inverse.
 */
int32_t fba_block_mean(const void* x, float* out, int64_t n_seq, int32_t S, int32_t block, int32_t head_dim, void* hip_stream);
int32_t fba_ssta_mask(const float* q_mean, const float* k_mean, const uint8_t* base, uint8_t* mask, int32_t B, int32_t Hq, int32_t Hkv, int32_t nQ,
                      int32_t nK, int32_t q_block, int32_t k_block, int32_t topk, int32_t band, int32_t sink,
                      void* hip_stream);
int32_t fba_tile_permute(const void* x, void* out, int64_t n_seq, int32_t T, int32_t H, int32_t W, int32_t tile_t,
                         int32_t tile_h, int32_t tile_w, int32_t head_dim, int32_t to_tiles, void* hip_stream);

/*
 * Diagnostic, no counterpart in the reference: `work_groups` x 4 waves each issue `iters` x 4 independent
 * v_mfma_f32_32x32x16_bf16 on register operands taken from src (1024 floats in device memory; null: all-zero operands)
 * and write a checksum per thread to sink (work_groups * 256 floats).  The launch executes
 * work_groups * 4 * iters * 4 * 32768 FLOP; timed by the caller it gives the rate the matrix pipe sustains on such data,
 * which on this GPU depends on the data (the clock follows the switching activity).
 */
int32_t fba_probe_mfma(const float* src, float* sink, int32_t work_groups, int32_t iters, void* hip_stream);

/*
 * Diagnostic, no counterpart in the reference: `work_groups` x 256 lanes read the `bytes` at src (device memory, a
 * multiple of 32 KiB) once, eight 16-byte streaming loads per lane in flight, and write nothing (sink: 4 bytes of device
 * memory that stay as they are unless the data folds to one particular word).  Timed by the caller over a buffer much
 * larger than the caches it gives the rate at which a read-only kernel pulls from device memory on this GPU, the
 * yardstick for the kernel that reads the dS workspace back.
 */
int32_t fba_probe_read(const void* src, int64_t bytes, uint32_t* sink, int32_t work_groups, void* hip_stream);

#ifdef __cplusplus
}
#endif

#endif /* FBA_H_ */
