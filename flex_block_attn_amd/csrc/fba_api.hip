// C ABI entry points: argument validation, variant selection, launches.  See include/fba.h for the contract.
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>

#include "../../include/fba.h"
#include "fba_kernels.h"

namespace {

thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

struct Shape {
  int64_t mask_bh;
  int B, Hq, Hkv, Sq, Skv, D, q_block, k_block;
};

// Shape rules of the operator (flex_block_attn_interface.py:18-32, flex_block_attn_h100.cu:833-850).
int check_shape(const Shape& s) {
  if (s.D != 128) return fail(FBA_ERR_INVALID, "head_dim must be 128, got %d", s.D);
  if (s.B <= 0 || s.Hq <= 0 || s.Hkv <= 0 || s.Sq <= 0 || s.Skv <= 0)
    return fail(FBA_ERR_INVALID, "B, Hq, Hkv, Sq, Skv must be positive (got %d %d %d %d %d)", s.B, s.Hq, s.Hkv, s.Sq, s.Skv);
  if (s.Hq % s.Hkv != 0) return fail(FBA_ERR_INVALID, "Hq (%d) must be a multiple of Hkv (%d)", s.Hq, s.Hkv);
  if (s.q_block <= 0 || s.q_block % 16 != 0) return fail(FBA_ERR_INVALID, "q_block (%d) must be a positive multiple of 16", s.q_block);
  if (s.k_block <= 0 || s.k_block % 64 != 0) return fail(FBA_ERR_INVALID, "k_block (%d) must be a positive multiple of 64", s.k_block);
  if (s.k_block % s.q_block != 0 && s.q_block % s.k_block != 0)
    return fail(FBA_ERR_INVALID, "one of q_block (%d), k_block (%d) must divide the other", s.q_block, s.k_block);
  if (s.Sq % s.q_block != 0) return fail(FBA_ERR_INVALID, "Sq (%d) must be a multiple of q_block (%d)", s.Sq, s.q_block);
  if (s.Skv % s.k_block != 0) return fail(FBA_ERR_INVALID, "Skv (%d) must be a multiple of k_block (%d)", s.Skv, s.k_block);
  if (s.mask_bh != 1 && s.mask_bh != (int64_t)s.B * s.Hq)
    return fail(FBA_ERR_INVALID, "mask_bh (%lld) must be 1 or B*Hq (%lld)", (long long)s.mask_bh, (long long)s.B * s.Hq);
  if ((int64_t)s.B * s.Hq * (int64_t)(s.Sq / 128 + 1) > 0x7fffffffLL || (int64_t)s.B * s.Hkv * (int64_t)(s.Skv / 128 + 1) > 0x7fffffffLL)
    return fail(FBA_ERR_INVALID, "problem too large for a 32-bit work-item index");
  return FBA_OK;
}

int check_ptrs(std::initializer_list<std::pair<const char*, const void*>> ps) {
  for (auto& kv : ps) {
    if (kv.second == nullptr) return fail(FBA_ERR_INVALID, "%s is null", kv.first);
    if (!aligned16(kv.second)) return fail(FBA_ERR_INVALID, "%s is not 16-byte aligned", kv.first);
  }
  return FBA_OK;
}

// Which dK/dV kernel runs on block lists: the one with 64 keys per wave (one wave per SIMD) by default.  It is about 9 %
// faster than the one with 32 keys per wave (two waves per SIMD) without the dS hand-over and about 7 % faster with it
// (a wave alone on its SIMD pays for every cycle its dS stores take to issue).  Both do the same arithmetic in the same
// order.  FBA_DKDV_KEYS_PER_WAVE = 32 or 64 overrides the choice (measurement of the two).
hipError_t launch_dkdv_variant(fba::BwdParams& p, hipStream_t stream) {
  const char* env = getenv("FBA_DKDV_KEYS_PER_WAVE");
  const int keys = env ? atoi(env) : 64;
  if (!p.tiled && keys == 64) return fba::launch_bwd_dkdv64(p, stream);
  return fba::launch_bwd_dkdv(p, stream);
}

int hip_fail(hipError_t e, const char* what) { return fail(FBA_ERR_HIP, "%s: %s", what, hipGetErrorString(e)); }

// Optional workspace for tail splitting: null (nothing is split), or 16-byte aligned with a non-negative size.
int check_split_ws(const void* ws, int64_t bytes) {
  if (ws == nullptr) return FBA_OK;
  if (!aligned16(ws)) return fail(FBA_ERR_INVALID, "split_ws is not 16-byte aligned");
  if (bytes < 0) return fail(FBA_ERR_INVALID, "split_ws_bytes must not be negative");
  return FBA_OK;
}

}  // namespace

extern "C" {

int32_t fba_version(void) { return FBA_VERSION; }

const char* fba_last_error(void) { return g_err; }

int64_t fba_split_workspace_bytes(void) { return fba::kSplitWsBytes; }

int32_t fba_mask_compact(const uint8_t* mask, int64_t mask_bh, int32_t nQ, int32_t nK, int32_t* q_cnt, int32_t* q_idx,
                         int32_t* k_cnt, int32_t* k_idx, void* hip_stream) {
  if (mask_bh <= 0 || nQ <= 0 || nK <= 0)
    return fail(FBA_ERR_INVALID, "mask_bh, nQ, nK must be positive (got %lld %d %d)", (long long)mask_bh, nQ, nK);
  if (!mask || !q_cnt || !q_idx || !k_cnt || !k_idx) return fail(FBA_ERR_INVALID, "null pointer argument");
  hipError_t e = fba::launch_mask_compact(mask, mask_bh, nQ, nK, q_cnt, q_idx, k_cnt, k_idx, (hipStream_t)hip_stream);
  return e == hipSuccess ? FBA_OK : hip_fail(e, "mask_compact launch");
}

}  // extern "C"

namespace {

// Which list flavour a shape needs: block lists when both block sizes are multiples of the 128-row kernel tiles, tile
// lists otherwise.  Tile lists need Sq and Skv to be multiples of 128.
int check_lists(const Shape& s, bool tiled, const char* what) {
  const bool aligned = s.q_block % 128 == 0 && s.k_block % 128 == 0;
  if (!tiled && !aligned)
    return fail(FBA_ERR_UNSUPPORTED, "%s: q_block (%d) and k_block (%d) are not both multiples of 128; build tile lists "
                "with fba_tile_lists and call the _tiled entry point", what, s.q_block, s.k_block);
  if (tiled && (s.Sq % 128 != 0 || s.Skv % 128 != 0))
    return fail(FBA_ERR_UNSUPPORTED, "%s: tile lists need Sq (%d) and Skv (%d) to be multiples of 128", what, s.Sq, s.Skv);
  return FBA_OK;
}

int fwd_impl(const void* q, const void* k, const void* v, void* o, float* lse, const int32_t* q_cnt, const int32_t* q_idx,
             int64_t mask_bh, int32_t B, int32_t Hq, int32_t Hkv, int32_t Sq, int32_t Skv, int32_t head_dim, int32_t q_block,
             int32_t k_block, void* split_ws, int64_t split_ws_bytes, void* hip_stream, bool tiled) {
  const Shape s{mask_bh, B, Hq, Hkv, Sq, Skv, head_dim, q_block, k_block};
  if (int rc = check_shape(s)) return rc;
  if (int rc = check_ptrs({{"q", q}, {"k", k}, {"v", v}, {"o", o}})) return rc;
  if (!lse || !q_cnt || !q_idx) return fail(FBA_ERR_INVALID, "null pointer argument");
  if (int rc = check_lists(s, tiled, "forward")) return rc;
  if (int rc = check_split_ws(split_ws, split_ws_bytes)) return rc;
  fba::FwdParams p{};
  p.q = (const __bf16*)q; p.k = (const __bf16*)k; p.v = (const __bf16*)v; p.o = (__bf16*)o; p.lse = lse;
  p.q_cnt = q_cnt; p.q_idx = q_idx; p.mask_bh = mask_bh;
  p.B = B; p.Hq = Hq; p.Hkv = Hkv; p.Sq = Sq; p.Skv = Skv; p.nQ = Sq / q_block; p.nK = Skv / k_block;
  p.q_block = q_block; p.k_block = k_block;
  p.scale_log2e = 1.4426950408889634f / 11.313708498984761f;
  p.tiled = tiled ? 1 : 0;
  p.split.ws = (float*)split_ws; p.split_ws_bytes = split_ws_bytes;
  {
    const char* rows = getenv("FBA_FWD_TILE_ROWS");
    p.variant = rows && atoi(rows) == 384 ? 0 : 1;  // 128-row work-groups unless asked otherwise
  }
  hipError_t e = fba::launch_fwd(p, (hipStream_t)hip_stream);
  return e == hipSuccess ? FBA_OK : hip_fail(e, "forward launch");
}

}  // namespace

extern "C" {

int32_t fba_fwd(const void* q, const void* k, const void* v, void* o, float* lse, const int32_t* q_cnt,
                const int32_t* q_idx, int64_t mask_bh, int32_t B, int32_t Hq, int32_t Hkv, int32_t Sq, int32_t Skv,
                int32_t head_dim, int32_t q_block, int32_t k_block, void* split_ws, int64_t split_ws_bytes, void* hip_stream) {
  return fwd_impl(q, k, v, o, lse, q_cnt, q_idx, mask_bh, B, Hq, Hkv, Sq, Skv, head_dim, q_block, k_block, split_ws, split_ws_bytes,
                  hip_stream, false);
}

int32_t fba_fwd_tiled(const void* q, const void* k, const void* v, void* o, float* lse, const int32_t* qt_cnt,
                      const int32_t* qt_ent, int64_t mask_bh, int32_t B, int32_t Hq, int32_t Hkv, int32_t Sq, int32_t Skv,
                      int32_t head_dim, int32_t q_block, int32_t k_block, void* split_ws, int64_t split_ws_bytes,
                      void* hip_stream) {
  return fwd_impl(q, k, v, o, lse, qt_cnt, qt_ent, mask_bh, B, Hq, Hkv, Sq, Skv, head_dim, q_block, k_block, split_ws, split_ws_bytes, hip_stream, true);
}

int32_t fba_block_mean(const void* x, float* out, int64_t n_seq, int32_t S, int32_t block, int32_t head_dim, void* hip_stream) {
  if (head_dim != 128) return fail(FBA_ERR_INVALID, "head_dim must be 128, got %d", head_dim);
  if (n_seq <= 0 || S <= 0) return fail(FBA_ERR_INVALID, "n_seq and S must be positive (got %lld %d)", (long long)n_seq, S);
  if (block <= 0 || block % 16 != 0 || S % block != 0)
    return fail(FBA_ERR_INVALID, "block (%d) must be a positive multiple of 16 that divides S (%d)", block, S);
  if (!out) return fail(FBA_ERR_INVALID, "out is null");
  if (int rc = check_ptrs({{"x", x}})) return rc;
  hipError_t e = fba::launch_block_mean((const __bf16*)x, out, n_seq * (S / block), block, (hipStream_t)hip_stream);
  return e == hipSuccess ? FBA_OK : hip_fail(e, "block_mean launch");
}

int32_t fba_ssta_mask(const float* q_mean, const float* k_mean, const uint8_t* base, uint8_t* mask, int32_t B, int32_t Hq, int32_t Hkv, int32_t nQ,
                      int32_t nK, int32_t q_block, int32_t k_block, int32_t topk, int32_t band, int32_t sink,
                      void* hip_stream) {
  if (B <= 0 || Hq <= 0 || Hkv <= 0 || nQ <= 0 || nK <= 0)
    return fail(FBA_ERR_INVALID, "B, Hq, Hkv, nQ, nK must be positive (got %d %d %d %d %d)", B, Hq, Hkv, nQ, nK);
  if (Hq % Hkv != 0) return fail(FBA_ERR_INVALID, "Hq (%d) must be a multiple of Hkv (%d)", Hq, Hkv);
  if (q_block <= 0 || k_block <= 0) return fail(FBA_ERR_INVALID, "q_block and k_block must be positive");
  if (topk < 0 || band < -1 || sink < 0) return fail(FBA_ERR_INVALID, "topk, sink must be >= 0 and band >= -1 (got %d %d %d)", topk, sink, band);
  if (!q_mean || !k_mean || !mask) return fail(FBA_ERR_INVALID, "null pointer argument");
  if (nK > 4096) return fail(FBA_ERR_UNSUPPORTED, "at most 4096 key blocks are ranked per query block (got %d)", nK);
  if ((int64_t)B * Hq > 65535) return fail(FBA_ERR_UNSUPPORTED, "B*Hq (%lld) must be at most 65535", (long long)B * Hq);
  hipError_t e = fba::launch_ssta_mask(q_mean, k_mean, base, mask, (int64_t)B * Hq, Hq, Hkv, nQ, nK, q_block, k_block, topk, band,
                                       sink, (hipStream_t)hip_stream);
  return e == hipSuccess ? FBA_OK : hip_fail(e, "ssta_mask launch");
}

int32_t fba_tile_permute(const void* x, void* out, int64_t n_seq, int32_t T, int32_t H, int32_t W, int32_t tile_t,
                         int32_t tile_h, int32_t tile_w, int32_t head_dim, int32_t to_tiles, void* hip_stream) {
  if (head_dim != 128) return fail(FBA_ERR_INVALID, "head_dim must be 128, got %d", head_dim);
  if (n_seq <= 0 || T <= 0 || H <= 0 || W <= 0 || tile_t <= 0 || tile_h <= 0 || tile_w <= 0)
    return fail(FBA_ERR_INVALID, "n_seq, grid and tile extents must be positive");
  if (T % tile_t != 0 || H % tile_h != 0 || W % tile_w != 0)
    return fail(FBA_ERR_INVALID, "tile (%d, %d, %d) must divide the grid (%d, %d, %d)", tile_t, tile_h, tile_w, T, H, W);
  if ((int64_t)T * H * W > 0x7fffffffLL) return fail(FBA_ERR_INVALID, "grid too large");
  if (x == out) return fail(FBA_ERR_INVALID, "x and out must not alias");
  if (int rc = check_ptrs({{"x", x}, {"out", out}})) return rc;
  hipError_t e = fba::launch_tile_permute(x, out, n_seq, T, H, W, tile_t, tile_h, tile_w, to_tiles ? 1 : 0, (hipStream_t)hip_stream);
  return e == hipSuccess ? FBA_OK : hip_fail(e, "tile_permute launch");
}

int32_t fba_tile_lists(const uint8_t* mask, int64_t mask_bh, int32_t nQ, int32_t nK, int32_t q_block, int32_t k_block,
                       int32_t* qt_cnt, int32_t* qt_ent, int32_t* kt_cnt, int32_t* kt_ent, void* hip_stream) {
  if (mask_bh <= 0 || nQ <= 0 || nK <= 0)
    return fail(FBA_ERR_INVALID, "mask_bh, nQ, nK must be positive (got %lld %d %d)", (long long)mask_bh, nQ, nK);
  if (q_block <= 0 || q_block % 16 != 0) return fail(FBA_ERR_INVALID, "q_block (%d) must be a positive multiple of 16", q_block);
  if (k_block <= 0 || k_block % 64 != 0) return fail(FBA_ERR_INVALID, "k_block (%d) must be a positive multiple of 64", k_block);
  const int64_t Sq = (int64_t)nQ * q_block, Skv = (int64_t)nK * k_block;
  if (Sq % 128 != 0 || Skv % 128 != 0)
    return fail(FBA_ERR_UNSUPPORTED, "tile lists need Sq (%lld) and Skv (%lld) to be multiples of 128", (long long)Sq, (long long)Skv);
  if (Sq / 32 >= (1 << 23) || nK >= (1 << 23)) return fail(FBA_ERR_INVALID, "sequence too long for 24-bit list entries");
  if (!mask || !qt_cnt || !qt_ent || !kt_cnt || !kt_ent) return fail(FBA_ERR_INVALID, "null pointer argument");
  hipError_t e = fba::launch_tile_lists(mask, mask_bh, nQ, nK, q_block, k_block, (int)(Sq / 128), (int)(Skv / 128), (int)(Sq / 32),
                                        qt_cnt, qt_ent, kt_cnt, kt_ent, (hipStream_t)hip_stream);
  return e == hipSuccess ? FBA_OK : hip_fail(e, "tile_lists launch");
}

static int fill_bwd(fba::BwdParams& p, const Shape& s) {
  p.mask_bh = s.mask_bh;
  p.B = s.B; p.Hq = s.Hq; p.Hkv = s.Hkv; p.Sq = s.Sq; p.Skv = s.Skv; p.nQ = s.Sq / s.q_block; p.nK = s.Skv / s.k_block;
  p.q_block = s.q_block; p.k_block = s.k_block;
  p.scale = 1.f / 11.313708498984761f;
  p.scale_log2e = 1.4426950408889634f / 11.313708498984761f;
  return FBA_OK;
}

int32_t fba_bwd_stats(const void* o, const void* d_o, const float* lse, float* stats, int64_t rows, int32_t head_dim,
                      void* hip_stream) {
  if (head_dim != 128) return fail(FBA_ERR_INVALID, "head_dim must be 128, got %d", head_dim);
  if (rows < 0 || rows >= (1LL << 30)) return fail(FBA_ERR_INVALID, "rows must be in [0, 2^30)");
  if (int rc = check_ptrs({{"o", o}, {"d_o", d_o}})) return rc;
  if (!lse || !stats) return fail(FBA_ERR_INVALID, "null pointer argument");
  hipError_t e = fba::launch_bwd_stats((const __bf16*)o, (const __bf16*)d_o, lse, stats, rows, (hipStream_t)hip_stream);
  return e == hipSuccess ? FBA_OK : hip_fail(e, "stats launch");
}

static int dq_impl(const void* q, const void* k, const void* v, const void* d_o, const float* stats, void* dq,
                   const int32_t* q_cnt, const int32_t* q_idx, int64_t mask_bh, int32_t B, int32_t Hq, int32_t Hkv,
                   int32_t Sq, int32_t Skv, int32_t head_dim, int32_t q_block, int32_t k_block, void* split_ws, int64_t split_ws_bytes,
                   void* hip_stream, bool tiled) {
  const Shape s{mask_bh, B, Hq, Hkv, Sq, Skv, head_dim, q_block, k_block};
  if (int rc = check_shape(s)) return rc;
  if (int rc = check_ptrs({{"q", q}, {"k", k}, {"v", v}, {"d_o", d_o}, {"dq", dq}})) return rc;
  if (!stats || !q_cnt || !q_idx) return fail(FBA_ERR_INVALID, "null pointer argument");
  if (int rc = check_lists(s, tiled, "dq")) return rc;
  if (int rc = check_split_ws(split_ws, split_ws_bytes)) return rc;
  fba::BwdParams p{};
  fill_bwd(p, s);
  p.tiled = tiled ? 1 : 0;
  p.q = (const __bf16*)q; p.k = (const __bf16*)k; p.v = (const __bf16*)v; p.d_o = (const __bf16*)d_o;
  p.stats = stats; p.dq = (__bf16*)dq; p.q_cnt = q_cnt; p.q_idx = q_idx;
  p.split.ws = (float*)split_ws; p.split_ws_bytes = split_ws_bytes;
  hipError_t e = fba::launch_bwd_dq(p, (hipStream_t)hip_stream);
  return e == hipSuccess ? FBA_OK : hip_fail(e, "dq launch");
}

static int dkdv_impl(const void* q, const void* k, const void* v, const void* d_o, const float* stats, void* dk, void* dv,
                     const int32_t* k_cnt, const int32_t* k_idx, int64_t mask_bh, int32_t B, int32_t Hq, int32_t Hkv,
                     int32_t Sq, int32_t Skv, int32_t head_dim, int32_t q_block, int32_t k_block, void* split_ws, int64_t split_ws_bytes,
                     void* hip_stream, bool tiled) {
  const Shape s{mask_bh, B, Hq, Hkv, Sq, Skv, head_dim, q_block, k_block};
  if (int rc = check_shape(s)) return rc;
  if (int rc = check_ptrs({{"q", q}, {"k", k}, {"v", v}, {"d_o", d_o}, {"dk", dk}, {"dv", dv}})) return rc;
  if (!stats || !k_cnt || !k_idx) return fail(FBA_ERR_INVALID, "null pointer argument");
  if (int rc = check_lists(s, tiled, "dkdv")) return rc;
  if (int rc = check_split_ws(split_ws, split_ws_bytes)) return rc;
  if ((int64_t)B * Hq * Sq >= (1LL << 30)) return fail(FBA_ERR_INVALID, "B*Hq*Sq must be below 2^30");
  fba::BwdParams p{};
  fill_bwd(p, s);
  p.tiled = tiled ? 1 : 0;
  p.q = (const __bf16*)q; p.k = (const __bf16*)k; p.v = (const __bf16*)v; p.d_o = (const __bf16*)d_o;
  p.stats = stats; p.dk = (__bf16*)dk; p.dv = (__bf16*)dv; p.k_cnt = k_cnt; p.k_idx = k_idx;
  p.split.ws = (float*)split_ws; p.split_ws_bytes = split_ws_bytes;
  hipError_t e = launch_dkdv_variant(p, (hipStream_t)hip_stream);
  return e == hipSuccess ? FBA_OK : hip_fail(e, "dkdv launch");
}

static int bwd_impl(const void* q, const void* k, const void* v, const void* o, const void* d_o, const float* lse,
                    float* stats, void* dq, void* dk, void* dv, const int32_t* q_cnt, const int32_t* q_idx,
                    const int32_t* k_cnt, const int32_t* k_idx, int64_t mask_bh, int32_t B, int32_t Hq, int32_t Hkv,
                    int32_t Sq, int32_t Skv, int32_t head_dim, int32_t q_block, int32_t k_block, void* split_ws, int64_t split_ws_bytes,
                    void* hip_stream, bool tiled) {
  const Shape s{mask_bh, B, Hq, Hkv, Sq, Skv, head_dim, q_block, k_block};
  if (int rc = check_shape(s)) return rc;
  if (int rc = check_lists(s, tiled, "backward")) return rc;
  if (int rc = check_split_ws(split_ws, split_ws_bytes)) return rc;
  // everything is validated before the first launch, so that a rejected call leaves nothing on the stream
  if (int rc = check_ptrs({{"q", q}, {"k", k}, {"v", v}, {"o", o}, {"d_o", d_o}, {"dq", dq}, {"dk", dk}, {"dv", dv}})) return rc;
  if (!lse || !stats || !q_cnt || !q_idx || !k_cnt || !k_idx) return fail(FBA_ERR_INVALID, "null pointer argument");
  if ((int64_t)B * Hq * Sq >= (1LL << 30)) return fail(FBA_ERR_INVALID, "B*Hq*Sq must be below 2^30");
  if (int rc = fba_bwd_stats(o, d_o, lse, stats, (int64_t)B * Hq * Sq, head_dim, hip_stream)) return rc;
  if (int rc = dkdv_impl(q, k, v, d_o, stats, dk, dv, k_cnt, k_idx, mask_bh, B, Hq, Hkv, Sq, Skv, head_dim, q_block, k_block,
                         split_ws, split_ws_bytes, hip_stream, tiled))
    return rc;
  return dq_impl(q, k, v, d_o, stats, dq, q_cnt, q_idx, mask_bh, B, Hq, Hkv, Sq, Skv, head_dim, q_block, k_block, split_ws, split_ws_bytes,
                 hip_stream, tiled);
}

int32_t fba_bwd_dq(const void* q, const void* k, const void* v, const void* d_o, const float* stats, void* dq,
                   const int32_t* q_cnt, const int32_t* q_idx, int64_t mask_bh, int32_t B, int32_t Hq, int32_t Hkv,
                   int32_t Sq, int32_t Skv, int32_t head_dim, int32_t q_block, int32_t k_block, void* split_ws, int64_t split_ws_bytes,
                   void* hip_stream) {
  return dq_impl(q, k, v, d_o, stats, dq, q_cnt, q_idx, mask_bh, B, Hq, Hkv, Sq, Skv, head_dim, q_block, k_block, split_ws, split_ws_bytes,
                 hip_stream, false);
}

int32_t fba_bwd_dkdv(const void* q, const void* k, const void* v, const void* d_o, const float* stats, void* dk, void* dv,
                     const int32_t* k_cnt, const int32_t* k_idx, int64_t mask_bh, int32_t B, int32_t Hq, int32_t Hkv,
                     int32_t Sq, int32_t Skv, int32_t head_dim, int32_t q_block, int32_t k_block, void* split_ws, int64_t split_ws_bytes,
                     void* hip_stream) {
  return dkdv_impl(q, k, v, d_o, stats, dk, dv, k_cnt, k_idx, mask_bh, B, Hq, Hkv, Sq, Skv, head_dim, q_block, k_block, split_ws,
                   split_ws_bytes, hip_stream, false);
}

int32_t fba_bwd(const void* q, const void* k, const void* v, const void* o, const void* d_o, const float* lse,
                float* stats, void* dq, void* dk, void* dv, const int32_t* q_cnt, const int32_t* q_idx,
                const int32_t* k_cnt, const int32_t* k_idx, int64_t mask_bh, int32_t B, int32_t Hq, int32_t Hkv,
                int32_t Sq, int32_t Skv, int32_t head_dim, int32_t q_block, int32_t k_block, void* split_ws, int64_t split_ws_bytes,
                void* hip_stream) {
  return bwd_impl(q, k, v, o, d_o, lse, stats, dq, dk, dv, q_cnt, q_idx, k_cnt, k_idx, mask_bh, B, Hq, Hkv, Sq, Skv, head_dim,
                  q_block, k_block, split_ws, split_ws_bytes, hip_stream, false);
}

int32_t fba_probe_mfma(const float* src, float* sink, int32_t work_groups, int32_t iters, void* hip_stream) {
  if (work_groups <= 0 || iters <= 0) return fail(FBA_ERR_INVALID, "work_groups and iters must be positive (got %d %d)", work_groups, iters);
  if (!sink) return fail(FBA_ERR_INVALID, "sink is null");
  hipError_t e = fba::launch_probe_mfma(src, sink, work_groups, iters, (hipStream_t)hip_stream);
  return e == hipSuccess ? FBA_OK : hip_fail(e, "probe launch");
}

int32_t fba_probe_read(const void* src, int64_t bytes, uint32_t* sink, int32_t work_groups, void* hip_stream) {
  if (work_groups <= 0 || bytes <= 0 || bytes % 32768 != 0)
    return fail(FBA_ERR_INVALID, "work_groups must be positive and bytes a positive multiple of 32768 (got %d %lld)", work_groups, (long long)bytes);
  if (!src || !sink) return fail(FBA_ERR_INVALID, "src or sink is null");
  hipError_t e = fba::launch_probe_read(src, bytes, sink, work_groups, (hipStream_t)hip_stream);
  return e == hipSuccess ? FBA_OK : hip_fail(e, "probe launch");
}

int32_t fba_pair_slots(const int32_t* q_cnt, const int32_t* q_idx, const int32_t* k_cnt, const int32_t* k_idx, int64_t mask_bh,
                       int32_t nQ, int32_t nK, int32_t* pair_base, int32_t* q_slot, void* hip_stream) {
  if (mask_bh <= 0 || nQ <= 0 || nK <= 0)
    return fail(FBA_ERR_INVALID, "mask_bh, nQ, nK must be positive (got %lld %d %d)", (long long)mask_bh, nQ, nK);
  if (mask_bh * (int64_t)nQ * nK > 0x7fffffffLL) return fail(FBA_ERR_INVALID, "more than 2^31 mask entries");
  if (!q_cnt || !q_idx || !k_cnt || !k_idx || !pair_base || !q_slot) return fail(FBA_ERR_INVALID, "null pointer argument");
  hipError_t e = fba::launch_pair_slots(q_cnt, q_idx, k_cnt, k_idx, mask_bh, nQ, nK, pair_base, q_slot, (hipStream_t)hip_stream);
  return e == hipSuccess ? FBA_OK : hip_fail(e, "pair_slots launch");
}

// Arguments of the dS hand-over, checked once for all three entry points that take them.
static int check_handover(const Shape& s, const void* ds_ws, int64_t ds_ws_bytes, const int32_t* pair_base, int64_t n_pairs, const char* what) {
  if (s.q_block % 128 != 0 || s.k_block % 128 != 0)
    return fail(FBA_ERR_UNSUPPORTED, "%s: the dS hand-over needs q_block (%d) and k_block (%d) to be multiples of 128", what, s.q_block, s.k_block);
  if (!pair_base) return fail(FBA_ERR_INVALID, "pair_base is null");
  if (int rc = check_ptrs({{"ds_ws", ds_ws}})) return rc;
  if (n_pairs < 0) return fail(FBA_ERR_INVALID, "n_pairs must not be negative");
  const int64_t need = n_pairs * (int64_t)s.q_block * s.k_block * 2;
  if (ds_ws_bytes < need)
    return fail(FBA_ERR_INVALID, "%s: ds_ws holds %lld bytes, %lld pairs of %d x %d need %lld", what, (long long)ds_ws_bytes,
                (long long)n_pairs, s.q_block, s.k_block, (long long)need);
  return FBA_OK;
}

int32_t fba_bwd_dkdv_handover(const void* q, const void* k, const void* v, const void* d_o, const float* stats, void* dk, void* dv,
                              void* ds_ws, int64_t ds_ws_bytes, const int32_t* k_cnt, const int32_t* k_idx, const int32_t* pair_base,
                              int64_t n_pairs, int64_t mask_bh, int32_t B, int32_t Hq, int32_t Hkv, int32_t Sq, int32_t Skv,
                              int32_t head_dim, int32_t q_block, int32_t k_block, void* split_ws, int64_t split_ws_bytes,
                              void* hip_stream) {
  const Shape s{mask_bh, B, Hq, Hkv, Sq, Skv, head_dim, q_block, k_block};
  if (int rc = check_shape(s)) return rc;
  if (int rc = check_handover(s, ds_ws, ds_ws_bytes, pair_base, n_pairs, "dkdv")) return rc;
  if (int rc = check_split_ws(split_ws, split_ws_bytes)) return rc;
  if (int rc = check_ptrs({{"q", q}, {"k", k}, {"v", v}, {"d_o", d_o}, {"dk", dk}, {"dv", dv}})) return rc;
  if (!stats || !k_cnt || !k_idx) return fail(FBA_ERR_INVALID, "null pointer argument");
  if ((int64_t)B * Hq * Sq >= (1LL << 30)) return fail(FBA_ERR_INVALID, "B*Hq*Sq must be below 2^30");
  fba::BwdParams p{};
  fill_bwd(p, s);
  p.q = (const __bf16*)q; p.k = (const __bf16*)k; p.v = (const __bf16*)v; p.d_o = (const __bf16*)d_o;
  p.stats = stats; p.dk = (__bf16*)dk; p.dv = (__bf16*)dv; p.k_cnt = k_cnt; p.k_idx = k_idx;
  p.ds_ws = (__bf16*)ds_ws; p.pair_base = pair_base;
  p.ws_pairs = ds_ws_bytes / ((int64_t)q_block * k_block * 2);
  p.split.ws = (float*)split_ws; p.split_ws_bytes = split_ws_bytes;
  hipError_t e = launch_dkdv_variant(p, (hipStream_t)hip_stream);
  return e == hipSuccess ? FBA_OK : hip_fail(e, "dkdv (hand-over) launch");
}

int32_t fba_bwd_dq_from_ds(const void* k, const void* ds_ws, int64_t ds_ws_bytes, void* dq, const int32_t* q_cnt, const int32_t* q_idx,
                           const int32_t* q_slot, const int32_t* pair_base, int64_t n_pairs, int64_t mask_bh, int32_t B, int32_t Hq,
                           int32_t Hkv, int32_t Sq, int32_t Skv, int32_t head_dim, int32_t q_block, int32_t k_block, void* split_ws,
                           int64_t split_ws_bytes, void* hip_stream) {
  const Shape s{mask_bh, B, Hq, Hkv, Sq, Skv, head_dim, q_block, k_block};
  if (int rc = check_shape(s)) return rc;
  if (int rc = check_handover(s, ds_ws, ds_ws_bytes, pair_base, n_pairs, "dq")) return rc;
  if (int rc = check_split_ws(split_ws, split_ws_bytes)) return rc;
  if (int rc = check_ptrs({{"k", k}, {"dq", dq}})) return rc;
  if (!q_cnt || !q_idx || !q_slot) return fail(FBA_ERR_INVALID, "null pointer argument");
  fba::BwdParams p{};
  fill_bwd(p, s);
  p.k = (const __bf16*)k; p.dq = (__bf16*)dq; p.q_cnt = q_cnt; p.q_idx = q_idx;
  p.ds_ws = (__bf16*)const_cast<void*>(ds_ws); p.pair_base = pair_base; p.q_slot = q_slot;
  p.ws_pairs = ds_ws_bytes / ((int64_t)q_block * k_block * 2);
  p.split.ws = (float*)split_ws; p.split_ws_bytes = split_ws_bytes;
  hipError_t e = fba::launch_bwd_dq_from_ds(p, (hipStream_t)hip_stream);
  return e == hipSuccess ? FBA_OK : hip_fail(e, "dq (from dS) launch");
}

int32_t fba_bwd_handover(const void* q, const void* k, const void* v, const void* o, const void* d_o, const float* lse, float* stats,
                         void* ds_ws, int64_t ds_ws_bytes, void* dq, void* dk, void* dv, const int32_t* q_cnt, const int32_t* q_idx,
                         const int32_t* k_cnt, const int32_t* k_idx, const int32_t* pair_base, const int32_t* q_slot, int64_t n_pairs,
                         int64_t mask_bh, int32_t B, int32_t Hq, int32_t Hkv, int32_t Sq, int32_t Skv, int32_t head_dim,
                         int32_t q_block, int32_t k_block, void* split_ws, int64_t split_ws_bytes, void* hip_stream) {
  const Shape s{mask_bh, B, Hq, Hkv, Sq, Skv, head_dim, q_block, k_block};
  if (int rc = check_shape(s)) return rc;
  // everything is validated before the first launch, so that a rejected call leaves nothing on the stream
  if (int rc = check_handover(s, ds_ws, ds_ws_bytes, pair_base, n_pairs, "backward")) return rc;
  if (int rc = check_split_ws(split_ws, split_ws_bytes)) return rc;
  if (int rc = check_ptrs({{"q", q}, {"k", k}, {"v", v}, {"o", o}, {"d_o", d_o}, {"dq", dq}, {"dk", dk}, {"dv", dv}})) return rc;
  if (!lse || !stats || !q_cnt || !q_idx || !k_cnt || !k_idx || !q_slot) return fail(FBA_ERR_INVALID, "null pointer argument");
  if ((int64_t)B * Hq * Sq >= (1LL << 30)) return fail(FBA_ERR_INVALID, "B*Hq*Sq must be below 2^30");
  if (int rc = fba_bwd_stats(o, d_o, lse, stats, (int64_t)B * Hq * Sq, head_dim, hip_stream)) return rc;
  if (int rc = fba_bwd_dkdv_handover(q, k, v, d_o, stats, dk, dv, ds_ws, ds_ws_bytes, k_cnt, k_idx, pair_base, n_pairs, mask_bh, B, Hq,
                                     Hkv, Sq, Skv, head_dim, q_block, k_block, split_ws, split_ws_bytes, hip_stream))
    return rc;
  return fba_bwd_dq_from_ds(k, ds_ws, ds_ws_bytes, dq, q_cnt, q_idx, q_slot, pair_base, n_pairs, mask_bh, B, Hq, Hkv, Sq, Skv, head_dim,
                            q_block, k_block, split_ws, split_ws_bytes, hip_stream);
}

int32_t fba_tile_slots(const int32_t* kt_cnt, const int32_t* kt_ent, int64_t mask_bh, int32_t n_qt, int32_t n_kt, int32_t* pair_base,
                       int32_t* kt_slot, int32_t* slot_table, void* hip_stream) {
  if (mask_bh <= 0 || n_qt <= 0 || n_kt <= 0)
    return fail(FBA_ERR_INVALID, "mask_bh, n_qt, n_kt must be positive (got %lld %d %d)", (long long)mask_bh, n_qt, n_kt);
  if (mask_bh * (int64_t)n_kt * n_qt * 4 > 0x7fffffffLL) return fail(FBA_ERR_INVALID, "more than 2^31 tile-list entries");
  if (!kt_cnt || !kt_ent || !pair_base || !kt_slot || !slot_table) return fail(FBA_ERR_INVALID, "null pointer argument");
  hipError_t e = fba::launch_tile_slots(kt_cnt, kt_ent, mask_bh, n_qt, n_kt, 4 * n_qt, pair_base, kt_slot, slot_table, (hipStream_t)hip_stream);
  return e == hipSuccess ? FBA_OK : hip_fail(e, "tile_slots launch");
}

int32_t fba_bwd_tiled_handover(const void* q, const void* k, const void* v, const void* o, const void* d_o, const float* lse, float* stats,
                               void* ds_ws, int64_t ds_ws_bytes, void* dq, void* dk, void* dv, const int32_t* qt_cnt,
                               const int32_t* qt_ent, const int32_t* kt_cnt, const int32_t* kt_ent, const int32_t* pair_base,
                               const int32_t* kt_slot, const int32_t* slot_table, int64_t n_pairs, int64_t mask_bh, int32_t B,
                               int32_t Hq, int32_t Hkv, int32_t Sq, int32_t Skv, int32_t head_dim, int32_t q_block, int32_t k_block,
                               void* split_ws, int64_t split_ws_bytes, void* hip_stream) {
  const Shape s{mask_bh, B, Hq, Hkv, Sq, Skv, head_dim, q_block, k_block};
  if (int rc = check_shape(s)) return rc;
  if (int rc = check_lists(s, true, "backward")) return rc;
  if (int rc = check_split_ws(split_ws, split_ws_bytes)) return rc;
  // everything is validated before the first launch, so that a rejected call leaves nothing on the stream
  if (int rc = check_ptrs({{"q", q}, {"k", k}, {"v", v}, {"o", o}, {"d_o", d_o}, {"dq", dq}, {"dk", dk}, {"dv", dv}, {"ds_ws", ds_ws}})) return rc;
  if (!lse || !stats || !qt_cnt || !qt_ent || !kt_cnt || !kt_ent || !pair_base || !kt_slot || !slot_table)
    return fail(FBA_ERR_INVALID, "null pointer argument");
  if ((int64_t)B * Hq * Sq >= (1LL << 30)) return fail(FBA_ERR_INVALID, "B*Hq*Sq must be below 2^30");
  if (n_pairs < 0) return fail(FBA_ERR_INVALID, "n_pairs must not be negative");
  const int64_t need = n_pairs * 128 * 128 * 2;
  if (ds_ws_bytes < need)
    return fail(FBA_ERR_INVALID, "backward: ds_ws holds %lld bytes, %lld tile pairs of 128 x 128 need %lld", (long long)ds_ws_bytes,
                (long long)n_pairs, (long long)need);
  if (int rc = fba_bwd_stats(o, d_o, lse, stats, (int64_t)B * Hq * Sq, head_dim, hip_stream)) return rc;
  fba::BwdParams p{};
  fill_bwd(p, s);
  p.tiled = 1;
  p.q = (const __bf16*)q; p.k = (const __bf16*)k; p.v = (const __bf16*)v; p.d_o = (const __bf16*)d_o;
  p.stats = stats; p.dq = (__bf16*)dq; p.dk = (__bf16*)dk; p.dv = (__bf16*)dv;
  p.q_cnt = qt_cnt; p.q_idx = qt_ent; p.k_cnt = kt_cnt; p.k_idx = kt_ent;
  p.ds_ws = (__bf16*)ds_ws; p.pair_base = pair_base; p.k_slot = kt_slot; p.q_slot = slot_table;
  p.ws_pairs = ds_ws_bytes / (128 * 128 * 2);
  p.split.ws = (float*)split_ws; p.split_ws_bytes = split_ws_bytes;
  hipError_t e = fba::launch_bwd_dkdv(p, (hipStream_t)hip_stream);
  if (e != hipSuccess) return hip_fail(e, "dkdv (tile lists, hand-over) launch");
  e = fba::launch_bwd_dq_from_ds(p, (hipStream_t)hip_stream);
  return e == hipSuccess ? FBA_OK : hip_fail(e, "dq (from dS, tile lists) launch");
}

}  // extern "C"

namespace {

// Workspace of fba_bwd_noalloc: the two statistics planes of backward (lse * log2(e), -delta) for up to kScratchRows
// query rows, 32 MiB, held by every GPU the library is loaded on until the process ends.  In host code the array's name
// is only a handle for hipGetSymbolAddress; kernels get the device address looked up below.
constexpr int64_t kScratchRows = 1LL << 22;
constexpr int kMaxDevices = 64;
static __device__ __align__(256) float scratch[2 * kScratchRows];
float* g_scratch_addr[kMaxDevices] = {};
std::mutex g_scratch_mutex;

// Device address of `scratch` on the current device (each GPU has its own copy at its own address); looked up on the
// first call on that device.
int scratch_address(float** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return hip_fail(e, "hipGetDevice");
  if (dev < 0 || dev >= kMaxDevices) return fail(FBA_ERR_UNSUPPORTED, "device ordinal %d is beyond the %d devices supported", dev, kMaxDevices);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_addr[dev] == nullptr) {
    void* ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return hip_fail(e, "hipGetSymbolAddress(scratch)");
    if (ptr == nullptr) return fail(FBA_ERR_HIP, "hipGetSymbolAddress(scratch) returned a null address");
    g_scratch_addr[dev] = static_cast<float*>(ptr);
  }
  *out = g_scratch_addr[dev];
  return FBA_OK;
}

}  // namespace

extern "C" {

int32_t fba_bwd_noalloc(const void* q, const void* k, const void* v, const void* o, const void* d_o, const float* lse,
                        void* dq, void* dk, void* dv, const int32_t* q_cnt, const int32_t* q_idx, const int32_t* k_cnt,
                        const int32_t* k_idx, int64_t mask_bh, int32_t B, int32_t Hq, int32_t Hkv, int32_t Sq, int32_t Skv,
                        int32_t head_dim, int32_t q_block, int32_t k_block, void* hip_stream) {
  const int64_t rows = (int64_t)B * Hq * Sq;
  if (B > 0 && Hq > 0 && Sq > 0 && rows > kScratchRows)
    return fail(FBA_ERR_UNSUPPORTED, "fba_bwd_noalloc: B*Hq*Sq = %lld query rows exceed the built-in workspace of %lld rows; "
                "call fba_bwd with a caller-owned stats buffer", (long long)rows, (long long)kScratchRows);
  float* stats = nullptr;
  if (int rc = scratch_address(&stats)) return rc;
  return bwd_impl(q, k, v, o, d_o, lse, stats, dq, dk, dv, q_cnt, q_idx, k_cnt, k_idx, mask_bh, B, Hq, Hkv, Sq, Skv, head_dim,
                  q_block, k_block, nullptr, 0, hip_stream, false);
}

int32_t fba_bwd_tiled(const void* q, const void* k, const void* v, const void* o, const void* d_o, const float* lse,
                      float* stats, void* dq, void* dk, void* dv, const int32_t* qt_cnt, const int32_t* qt_ent,
                      const int32_t* kt_cnt, const int32_t* kt_ent, int64_t mask_bh, int32_t B, int32_t Hq, int32_t Hkv,
                      int32_t Sq, int32_t Skv, int32_t head_dim, int32_t q_block, int32_t k_block,
                      void* split_ws, int64_t split_ws_bytes, void* hip_stream) {
  return bwd_impl(q, k, v, o, d_o, lse, stats, dq, dk, dv, qt_cnt, qt_ent, kt_cnt, kt_ent, mask_bh, B, Hq, Hkv, Sq, Skv, head_dim,
                  q_block, k_block, split_ws, split_ws_bytes, hip_stream, true);
}

}  // extern "C"
