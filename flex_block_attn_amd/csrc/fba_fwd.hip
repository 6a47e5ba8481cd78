// Forward kernel: block-sparse softmax attention for gfx950, head_dim 128, bf16 in / fp32 accumulate.
//
// One work-group of 4 waves owns 128*QB consecutive query rows of one (batch, head); wave w owns rows
// [32*QB*w, 32*QB*(w+1)).  The work-group walks the active-key-block list of its query block and streams every
// selected key block through LDS as 64-key slabs of K and V (two stages, one barrier per slab).
//
// Per slab and wave, in "transposed" form so that softmax statistics are per-lane scalars:
//   S^T[key, q]  = K[key, :] . Q[q, :]            A = K slab rows from LDS (128-bit fetches), B = Q in registers
//   P^T          = exp2(c * S^T - c * m[q])        fp32, c = log2(e) / sqrt(128); running max m and sum l per lane
//   O^T[d, q]   += V^T[d, key] . P^T[key, q]       A = V slab through transposing LDS fetches, B = P^T packed to bf16
// The reference computes the same quantities per selected tile (flex_block_attn_h100.cu:245-290, online softmax
// :199-221, final O / l at :292); here LSE is stored as the natural-log value m/sqrt(128) + ln(l).
#include "fba_common.h"
#include "fba_kernels.h"

namespace fba {

template <int QB>
__global__ __attribute__((amdgpu_flat_work_group_size(256, 256))) void fwd_kernel(const FwdParams p) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  constexpr int TQ = 128 * QB;
  constexpr int kSlab = 64;
  constexpr int kTileBytes = kSlab * kRowBytes;  // 16 KiB
  // smem: [stage][K | V]

  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, l32 = lane & 31, h = lane >> 5;
  const int item = xcd_remap(blockIdx.x, p.items_per_xcd);
  if (item >= p.num_items) return;
  const int tiles_per_head = p.Sq / TQ;
  const int bh = item / tiles_per_head;
  const int qt = item - bh * tiles_per_head;
  const int b = bh / p.Hq, hq = bh - b * p.Hq;
  const int hkv = hq / (p.Hq / p.Hkv);

  const __bf16* qp = p.q + ((int64_t)bh * p.Sq + (int64_t)qt * TQ + wave * 32 * QB) * kHeadDim;
  const __bf16* kp = p.k + ((int64_t)(b * p.Hkv + hkv) * p.Skv) * kHeadDim;
  const __bf16* vp = p.v + ((int64_t)(b * p.Hkv + hkv) * p.Skv) * kHeadDim;

  const int qblk = (qt * TQ) / p.q_block;
  const int64_t mrow = (p.mask_bh == 1 ? 0 : (int64_t)bh) * p.nQ + qblk;
  const int cnt = p.q_cnt[mrow];
  const int32_t* __restrict__ idx = p.q_idx + mrow * p.nK;
  const int nsub = p.k_block / kSlab;
  const int nsteps = cnt * nsub;

  // Q as the B operand: lane holds row (32 n + l32), d = 16 ks + 8 h .. +7
  bf16x8 qreg[QB][8];
#pragma unroll
  for (int n = 0; n < QB; ++n)
#pragma unroll
    for (int ks = 0; ks < 8; ++ks)
      qreg[n][ks] = *reinterpret_cast<const bf16x8*>(qp + (int64_t)(32 * n + l32) * kHeadDim + 16 * ks + 8 * h);

  RowMajorOffsets rm;
  rm.init(lane);
  TransposedOffsets tr;
  tr.init(lane);
  const int wr_off = tile_off(tid >> 4, tid & 15);

  f32x16 acc_o[QB][4];
  float m_run[QB], l_run[QB];
#pragma unroll
  for (int n = 0; n < QB; ++n) {
    m_run[n] = -INFINITY;
    l_run[n] = 0.f;
#pragma unroll
    for (int mb = 0; mb < 4; ++mb)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc_o[n][mb][r] = 0.f;
  }
  const float c = p.scale_log2e;

  TileCopy<kSlab> kc, vc;
  int e_next = 0, s_next = 0;  // list entry / slab of the next tile to fetch
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

  for (int step = 0; step < nsteps; ++step) {
    const char* ks_lds = smem + (step & 1) * 2 * kTileBytes;
    const char* vs_lds = ks_lds + kTileBytes;
    char* nxt = smem + ((step + 1) & 1) * 2 * kTileBytes;
    const bool more = step + 1 < nsteps;
    if (more) fetch();

    // S^T = K Q^T
    f32x16 s[QB][2];
#pragma unroll
    for (int n = 0; n < QB; ++n)
#pragma unroll
      for (int m2 = 0; m2 < 2; ++m2)
#pragma unroll
        for (int r = 0; r < 16; ++r) s[n][m2][r] = 0.f;
#pragma unroll
    for (int m2 = 0; m2 < 2; ++m2)
#pragma unroll
      for (int ks = 0; ks < 8; ++ks) {
        const bf16x8 a = lds_read_b128(ks_lds, rm.rd[ks] + m2 * 32 * kRowBytes);
#pragma unroll
        for (int n = 0; n < QB; ++n) s[n][m2] = mfma32(a, qreg[n][ks], s[n][m2]);
      }

    // online softmax, per lane (= per query row; the two half-waves hold disjoint keys of the same row)
    bf16x8 pk[QB][2][2];
#pragma unroll
    for (int n = 0; n < QB; ++n) {
      float mx = m_run[n];
#pragma unroll
      for (int m2 = 0; m2 < 2; ++m2)
#pragma unroll
        for (int r = 0; r < 16; ++r) mx = fmaxf(mx, s[n][m2][r]);
      mx = max_halves(mx);
      const float alpha = fast_exp2((m_run[n] - mx) * c);
      m_run[n] = mx;
      const float mc = mx * c;
      float rs = 0.f;
#pragma unroll
      for (int m2 = 0; m2 < 2; ++m2)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const float pv = fast_exp2(__builtin_fmaf(s[n][m2][r], c, -mc));
          s[n][m2][r] = pv;
          rs += pv;
        }
      l_run[n] = l_run[n] * alpha + rs;
#pragma unroll
      for (int mb = 0; mb < 4; ++mb)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc_o[n][mb][r] *= alpha;
#pragma unroll
      for (int m2 = 0; m2 < 2; ++m2)
#pragma unroll
        for (int j = 0; j < 2; ++j)
          pk[n][m2][j] = pack8(s[n][m2][8 * j + 0], s[n][m2][8 * j + 1], s[n][m2][8 * j + 2], s[n][m2][8 * j + 3],
                               s[n][m2][8 * j + 4], s[n][m2][8 * j + 5], s[n][m2][8 * j + 6], s[n][m2][8 * j + 7]);
    }

    // O^T += V^T P^T
#pragma unroll
    for (int mb = 0; mb < 4; ++mb)
#pragma unroll
      for (int m2 = 0; m2 < 2; ++m2)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          const int roff = (32 * m2 + 16 * j) * kRowBytes;
          const bf16x8 a = cat(lds_read_tr(vs_lds, tr.rd[mb][0] + roff), lds_read_tr(vs_lds, tr.rd[mb][1] + roff));
#pragma unroll
          for (int n = 0; n < QB; ++n) acc_o[n][mb] = mfma32(a, pk[n][m2][j], acc_o[n][mb]);
        }

    if (more) {
      kc.store(nxt, wr_off);
      vc.store(nxt + kTileBytes, wr_off);
    }
    __syncthreads();
  }

  // epilogue: O = O^T / l, LSE = ln2 * (c m + log2 l)
  __bf16* op = p.o + ((int64_t)bh * p.Sq + (int64_t)qt * TQ + wave * 32 * QB) * kHeadDim;
  float* lp = p.lse + (int64_t)bh * p.Sq + (int64_t)qt * TQ + wave * 32 * QB;
#pragma unroll
  for (int n = 0; n < QB; ++n) {
    const float l = sum_halves(l_run[n]);
    const float inv = l > 0.f ? 1.f / l : 0.f;
    if (h == 0) lp[32 * n + l32] = l > 0.f ? (m_run[n] * c + __builtin_log2f(l)) * 0.6931471805599453f : -INFINITY;
    __bf16* orow = op + (int64_t)(32 * n + l32) * kHeadDim;
#pragma unroll
    for (int mb = 0; mb < 4; ++mb)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const bf16x4 ov = pack4(acc_o[n][mb][4 * g + 0] * inv, acc_o[n][mb][4 * g + 1] * inv,
                                acc_o[n][mb][4 * g + 2] * inv, acc_o[n][mb][4 * g + 3] * inv);
        *reinterpret_cast<bf16x4*>(orow + 32 * mb + 8 * g + 4 * h) = ov;
      }
  }
}

template <int QB>
static hipError_t launch(const FwdParams& p, hipStream_t stream) {
  constexpr int kSmem = 2 * 2 * 64 * kRowBytes;
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&fwd_kernel<QB>), hipFuncAttributeMaxDynamicSharedMemorySize, kSmem);
  if (e != hipSuccess) return e;
  hipLaunchKernelGGL(fwd_kernel<QB>, dim3(p.items_per_xcd * kNumXcd), dim3(256), kSmem, stream, p);
  return hipGetLastError();
}

hipError_t launch_fwd(FwdParams p, int qb, hipStream_t stream) {
  const int tq = 128 * qb;
  p.num_items = p.B * p.Hq * (p.Sq / tq);
  p.items_per_xcd = (p.num_items + kNumXcd - 1) / kNumXcd;
  switch (qb) {
    case 1: return launch<1>(p, stream);
    case 2: return launch<2>(p, stream);
    case 3: return launch<3>(p, stream);
    default: return hipErrorInvalidValue;
  }
}

}  // namespace fba
