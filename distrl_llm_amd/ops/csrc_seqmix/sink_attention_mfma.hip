// Tiled MFMA forms of the sink attention for bf16: prompt portions (a tile =
// up to 64 queries of one head) and decode steps (HEADS: a tile = the heads
// of one token, the key range split over workgroups and merged afterwards).
//
// One workgroup (4 waves, or 8 when the value range is wider than 256
// columns: two sets of 4 that split the columns) per (tile of <= 64
// consecutive queries of one sequence, query head). Wave w of a set owns
// queries 16 w .. 16 w + 15 for the whole kernel: their scores, their online softmax and their value sums, so the
// waves only meet to stage a block of 64 keys: the head's K rows and the V
// rows (of every kv head when the weights are mixed across heads, of the
// head's own kv head otherwise) go through LDS once per 64 queries.
//   scores   MFMA 16x16x32: A = the wave's queries (registers, loaded once),
//            B = K rows from LDS
//   softmax  fp32 in the MFMA's result layout; cap and causal mask per score;
//            row reductions over the 16 lanes of a row; the sink enters the
//            denominator once, at the end
//   values   the fp32 weights go through a wave-private LDS tile to the A
//            layout and are split into two bf16 terms (p = hi + lo, error
//            <= 2^-17 p), so the weighted sum keeps fp32-grade weights on
//            bf16 MFMAs; B = V^T from LDS (staged transposed, so a lane's
//            eight keys of one value column are one 16-byte read)
// HEADS: wave w owns heads 16 w .. 16 w + 15 of one decoded token. Their kv
// heads differ, so the scores are taken per kv head (B = K rows straight from
// the cache: every K element feeds one MFMA only) and each row keeps the tile
// of its own kv head; the value sums always run over every kv head and the
// merge kernel keeps what the head needs.
#include <torch/extension.h>
#include <ATen/cuda/CUDAContext.h>
#include "seqmix_common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16v8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

namespace {

#define SAM_KB 64          // keys per block
#define SAM_QT 64          // queries per tile
#define SAM_VP 72          // v_lds row pitch (bf16): 64 keys + 8
#define SAM_PP 68          // p_lds row pitch (floats): 64 keys + 4
#define SAM_MAX_KSTEPS 8   // dk <= 256

// NT: 16-column value tiles held by a wave; WS: wave sets. Set s (waves 4 s ..
// 4 s + 3) sums value tiles s NT .. s NT + NT - 1 (NV <= 16 NT WS); with two
// sets both take the scores of the same rows, and the accumulators of a wide
// value range fit a register budget that lets two waves share a SIMD.
template <int NT, int WS, bool HEADS>
__global__ __launch_bounds__(256 * WS, 2) void sink_attention_mfma_kernel(
    const bf16_t* __restrict__ q,         // [Tn, H, dk]
    const bf16_t* __restrict__ cache,     // [rows, G (dk + vd)]
    const int* __restrict__ block_tables, int max_nb, int block_size,
    const int* __restrict__ positions,
    const int* __restrict__ tiles,        // query tiles, or tok_seq when HEADS
    int H, int G, int dk, int vd, float scale, float softcap,
    const float* __restrict__ sink, int all_groups,
    float* __restrict__ part,             // [Tn, H, NV]; HEADS: [Tn, H, ksplit, NV] unnormalised
    int ksplit, float* __restrict__ part_ml) {     // HEADS: [Tn, H, ksplit, 2] = (max, sum)
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int ksteps = (dk + 31) / 32;
  const int KP = HEADS ? 0 : ksteps * 32 + 8;      // k_lds row pitch (bf16)
  const int NV = (HEADS || all_groups) ? G * vd : vd;
  const int NVp = (NV + 15) / 16 * 16;
  bf16_t* k_lds = reinterpret_cast<bf16_t*>(smem);                 // [64][KP]
  bf16_t* v_lds = k_lds + SAM_KB * KP;                             // [NVp][SAM_VP]
  float* p_all = reinterpret_cast<float*>(v_lds + NVp * SAM_VP);   // [4 WS][16][SAM_PP]
  int* krow = reinterpret_cast<int*>(p_all + 4 * WS * 16 * SAM_PP);   // [64]
  constexpr int NTH = 256 * WS;

  const int tile = blockIdx.x;
  const int hd = HEADS ? 0 : blockIdx.y;
  const int b = HEADS ? tiles[tile] : tiles[3 * tile];
  const int t0 = HEADS ? tile : tiles[3 * tile + 1];
  const int nq = HEADS ? 1 : tiles[3 * tile + 2];
  const int tid = threadIdx.x, l = tid & 63, lrow = l & 15, lk = l >> 4;
  const int wave = (tid >> 6) & 3;                 // which 16 rows of the tile
  const int nt0 = (tid >> 8) * NT;                 // first value tile of the wave's set
  const int W = G * (dk + vd);
  const int rep = H / G;
  const int grp = hd / rep;
  const int koff = grp * dk;
  const int voff = G * dk + ((HEADS || all_groups) ? 0 : grp * vd);
  const int p0 = positions[t0];
  const int plast = p0 + nq - 1;
  const int nblk = plast / SAM_KB + 1;
  const int* bt = block_tables + (int64_t)b * max_nb;
  float* p_lds = p_all + (tid >> 6) * 16 * SAM_PP;
  // uniform per wave: it has rows (queries of the tile, or heads of the token)
  const bool active = HEADS ? (wave * 16 < H) : (wave * 16 < nq);
  const int wave_plast = HEADS ? plast : min(plast, p0 + wave * 16 + 15);
  const int kb_lo = HEADS ? (int)(((int64_t)nblk * blockIdx.y) / ksplit) : 0;
  const int kb_hi = HEADS ? (int)(((int64_t)nblk * (blockIdx.y + 1)) / ksplit) : nblk;

  // the wave's rows as A fragments: row lrow, k = ks * 32 + lk * 8 ..
  bf16v8 qf[SAM_MAX_KSTEPS];
  {
    const int qi = wave * 16 + lrow;
    const bool row_ok = HEADS ? (qi < H) : (qi < nq);
    const bf16_t* qp = HEADS ? q + ((int64_t)t0 * H + min(qi, H - 1)) * dk
                             : q + ((int64_t)(t0 + min(qi, nq - 1)) * H + hd) * dk;
    #pragma unroll
    for (int ks = 0; ks < SAM_MAX_KSTEPS; ++ks) {
      #pragma unroll
      for (int j = 0; j < 8; ++j) qf[ks][j] = (__bf16)0.0f;
      const int kk = ks * 32 + lk * 8;
      if (ks < ksteps && row_ok && kk < dk) qf[ks] = *reinterpret_cast<const bf16v8*>(qp + kk);
    }
  }
  // padding rows of v_lds (value columns NV .. NVp) stay zero
  for (int i = tid; i < (NVp - NV) * SAM_VP; i += NTH) v_lds[NV * SAM_VP + i] = __float2bfloat16(0.f);

  float m[4], lsum[4];
  f32x4 acc[NT];
  #pragma unroll
  for (int r = 0; r < 4; ++r) { m[r] = -INFINITY; lsum[r] = 0.f; }
  #pragma unroll
  for (int i = 0; i < NT; ++i) acc[i] = f32x4{0.f, 0.f, 0.f, 0.f};

  for (int kb = kb_lo; kb < kb_hi; ++kb) {
    const int j0 = kb * SAM_KB;
    __syncthreads();                               // the previous block's LDS reads are done
    if (tid < SAM_KB) {
      const int j = min(j0 + tid, plast);          // keys past the tile's last are masked below
      krow[tid] = bt[j / block_size] * block_size + j % block_size;
    }
    __syncthreads();
    // K rows: [key][dk], zero beyond dk
    if (!HEADS) for (int i = tid; i < SAM_KB * ksteps * 4; i += NTH) {
      const int key = i / (ksteps * 4), c = (i % (ksteps * 4)) * 8;
      bf16v8 v;
      if (c < dk) {
        v = *reinterpret_cast<const bf16v8*>(cache + (int64_t)krow[key] * W + koff + c);
      } else {
        #pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = (__bf16)0.0f;
      }
      *reinterpret_cast<bf16v8*>(k_lds + key * KP + c) = v;
    }
    // V rows, transposed: v_lds[column][key]
    for (int i = tid; i < SAM_KB * (NV / 8); i += NTH) {
      const int key = i % SAM_KB, c = (i / SAM_KB) * 8;
      const bf16v8 v = *reinterpret_cast<const bf16v8*>(cache + (int64_t)krow[key] * W + voff + c);
      #pragma unroll
      for (int j = 0; j < 8; ++j)
        *reinterpret_cast<__bf16*>(v_lds + (c + j) * SAM_VP + key) = v[j];
    }
    __syncthreads();
    if (!active || j0 > wave_plast) continue;      // no query of this wave sees the block

    // scores of the wave's 16 rows against the 64 keys
    f32x4 s[4];
    #pragma unroll
    for (int ct = 0; ct < 4; ++ct) s[ct] = f32x4{0.f, 0.f, 0.f, 0.f};
    if (HEADS) {
      const int c_hi = min(G - 1, (wave * 16 + 15) / rep);
      for (int c = (wave * 16) / rep; c <= c_hi; ++c) {
        #pragma unroll
        for (int ct = 0; ct < 4; ++ct) {
          f32x4 sc = f32x4{0.f, 0.f, 0.f, 0.f};
          const bf16_t* kp = cache + (int64_t)krow[ct * 16 + lrow] * W + c * dk + lk * 8;
          #pragma unroll
          for (int ks = 0; ks < SAM_MAX_KSTEPS; ++ks) {
            if (ks < ksteps) {
              bf16v8 kf;
              #pragma unroll
              for (int j = 0; j < 8; ++j) kf[j] = (__bf16)0.0f;
              if (ks * 32 + lk * 8 < dk) kf = *reinterpret_cast<const bf16v8*>(kp + ks * 32);
              sc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qf[ks], kf, sc, 0, 0, 0);
            }
          }
          #pragma unroll
          for (int r = 0; r < 4; ++r)
            if ((wave * 16 + lk * 4 + r) / rep == c) s[ct][r] = sc[r];
        }
      }
    } else {
      #pragma unroll
      for (int ct = 0; ct < 4; ++ct) {
        #pragma unroll
        for (int ks = 0; ks < SAM_MAX_KSTEPS; ++ks) {
          if (ks < ksteps) {
            const bf16v8 kf = *reinterpret_cast<const bf16v8*>(
                k_lds + (ct * 16 + lrow) * KP + ks * 32 + lk * 8);
            s[ct] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qf[ks], kf, s[ct], 0, 0, 0);
          }
        }
      }
    }
    // result layout: reg r -> query lk * 4 + r, lane column lrow -> key ct * 16 + lrow
    float cr[4];
    #pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int qi = wave * 16 + lk * 4 + r;
      const int prow = HEADS ? ((qi < H) ? p0 : -1) : ((qi < nq) ? p0 + qi : -1);
      float sv[4];
      float bm = -INFINITY;
      #pragma unroll
      for (int ct = 0; ct < 4; ++ct) {
        const int j = j0 + ct * 16 + lrow;
        float x = s[ct][r] * scale;
        if (softcap > 0.f) x = softcap * tanhf(x / softcap);
        sv[ct] = (j <= prow) ? x : -INFINITY;
        bm = fmaxf(bm, sv[ct]);
      }
      #pragma unroll
      for (int off = 8; off > 0; off >>= 1) bm = fmaxf(bm, __shfl_xor(bm, off, SM_WAVE));
      const float mn = fmaxf(m[r], bm);
      const float c = (mn == -INFINITY) ? 1.0f : expf(m[r] - mn);
      float ps = 0.f;
      #pragma unroll
      for (int ct = 0; ct < 4; ++ct) {
        const float pv = (sv[ct] == -INFINITY) ? 0.f : expf(sv[ct] - mn);
        ps += pv;
        p_lds[(lk * 4 + r) * SAM_PP + ct * 16 + lrow] = pv;
      }
      #pragma unroll
      for (int off = 8; off > 0; off >>= 1) ps += __shfl_xor(ps, off, SM_WAVE);
      lsum[r] = lsum[r] * c + ps;
      m[r] = mn;
      cr[r] = c;
    }
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_s_waitcnt(0xc07f);
    // weights as A fragments: row lrow, keys ks2 * 32 + lk * 8 ..
    bf16v8 a_hi[2], a_lo[2];
    #pragma unroll
    for (int ks2 = 0; ks2 < 2; ++ks2) {
      const float4 w0 = *reinterpret_cast<const float4*>(p_lds + lrow * SAM_PP + ks2 * 32 + lk * 8);
      const float4 w1 = *reinterpret_cast<const float4*>(p_lds + lrow * SAM_PP + ks2 * 32 + lk * 8 + 4);
      const float pv[8] = {w0.x, w0.y, w0.z, w0.w, w1.x, w1.y, w1.z, w1.w};
      #pragma unroll
      for (int j = 0; j < 8; ++j) {
        const __bf16 hi = (__bf16)pv[j];
        a_hi[ks2][j] = hi;
        a_lo[ks2][j] = (__bf16)(pv[j] - (float)hi);
      }
    }
    #pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      if ((nt0 + nt) * 16 < NV) {
        f32x4 a = acc[nt];
        #pragma unroll
        for (int r = 0; r < 4; ++r) a[r] *= cr[r];
        #pragma unroll
        for (int ks2 = 0; ks2 < 2; ++ks2) {
          const bf16v8 vf = *reinterpret_cast<const bf16v8*>(
              v_lds + ((nt0 + nt) * 16 + lrow) * SAM_VP + ks2 * 32 + lk * 8);
          a = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_hi[ks2], vf, a, 0, 0, 0);
          a = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_lo[ks2], vf, a, 0, 0, 0);
        }
        acc[nt] = a;
      }
    }
    __builtin_amdgcn_wave_barrier();               // p_lds is rewritten in the next block
  }

  if (!active) return;
  if (HEADS) {
    // unnormalised partial of this key range; the merge kernel adds the sink
    #pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int head = wave * 16 + lk * 4 + r;
      if (head >= H) continue;
      const int64_t o = ((int64_t)t0 * H + head) * ksplit + blockIdx.y;
      if (lrow == 0 && nt0 == 0) {
        part_ml[o * 2] = m[r];
        part_ml[o * 2 + 1] = lsum[r];
      }
      #pragma unroll
      for (int nt = 0; nt < NT; ++nt) {
        const int col = (nt0 + nt) * 16 + lrow;
        if (col < NV) part[o * NV + col] = acc[nt][r];
      }
    }
    return;
  }
  #pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int qi = wave * 16 + lk * 4 + r;
    if (qi >= nq) continue;
    float M = m[r], L = lsum[r], e = 1.0f;
    if (sink != nullptr) {
      const float sk = sink[hd];
      M = fmaxf(m[r], sk);
      e = expf(m[r] - M);
      L = lsum[r] * e + expf(sk - M);
    }
    const float f = e / L;
    float* dst = part + ((int64_t)(t0 + qi) * H + hd) * NV;
    #pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      const int col = (nt0 + nt) * 16 + lrow;
      if (col < NV) dst[col] = acc[nt][r] * f;
    }
  }
}

// Merge the key ranges of one (token, head): M = max(m_s, sink),
// L = sum_s l_s e^(m_s - M) + e^(sink - M), out = sum_s acc_s e^(m_s - M) / L,
// over every kv head's columns (all_groups) or the head's own.
__global__ __launch_bounds__(256) void sink_attention_merge_kernel(
    const float* __restrict__ pacc, const float* __restrict__ pml,
    const float* __restrict__ sink, int H, int G, int vd, int ksplit, int all_groups,
    float* __restrict__ part) {
  const int64_t t = blockIdx.x;
  const int h = blockIdx.y;
  const int NVin = G * vd;
  const int NVout = all_groups ? NVin : vd;
  const int c0 = all_groups ? 0 : (h / (H / G)) * vd;
  const float* ml = pml + ((t * H + h) * ksplit) * 2;
  float M = (sink != nullptr) ? sink[h] : -INFINITY;
  for (int s = 0; s < ksplit; ++s) M = fmaxf(M, ml[2 * s]);
  float L = (sink != nullptr) ? expf(sink[h] - M) : 0.f;
  for (int s = 0; s < ksplit; ++s)
    if (ml[2 * s] != -INFINITY) L += ml[2 * s + 1] * expf(ml[2 * s] - M);
  const float inv = 1.0f / L;
  for (int col = threadIdx.x; col < NVout; col += blockDim.x) {
    float a = 0.f;
    for (int s = 0; s < ksplit; ++s)
      if (ml[2 * s] != -INFINITY)
        a += pacc[((t * H + h) * ksplit + s) * NVin + c0 + col] * expf(ml[2 * s] - M);
    part[(t * H + h) * NVout + col] = a * inv;
  }
}

// wave sets by value range: one set up to 16 value tiles (two workgroups of
// four waves then share a CU and overlap their staging and MFMA phases), two
// beyond; every variant is held to 256 registers so two waves fit a SIMD
int sam_wave_sets(int NV) { return (NV + 15) / 16 > 16 ? 2 : 1; }

size_t sam_lds_bytes(int dk, int NV, bool heads) {
  const int ksteps = (dk + 31) / 32;
  const int NVp = (NV + 15) / 16 * 16;
  return (heads ? 0 : (size_t)SAM_KB * (ksteps * 32 + 8) * 2) + (size_t)NVp * SAM_VP * 2 +
         (size_t)4 * sam_wave_sets(NV) * 16 * SAM_PP * 4 + SAM_KB * 4;
}

}  // namespace

bool sink_attention_mfma_fits(int dk, int vd, int G, int all_groups) {
  const int NV = all_groups ? G * vd : vd;
  return dk % 8 == 0 && vd % 8 == 0 && dk <= 32 * SAM_MAX_KSTEPS && NV <= 768 &&
         sam_lds_bytes(dk, NV, false) <= 150 * 1024;
}

bool sink_attention_heads_fits(int H, int dk, int vd, int G) {
  return dk % 8 == 0 && vd % 8 == 0 && dk <= 32 * SAM_MAX_KSTEPS && G * vd <= 768 && H <= 64 &&
         sam_lds_bytes(dk, G * vd, true) <= 150 * 1024;
}

torch::Tensor sink_attention_mfma(torch::Tensor q, torch::Tensor cache, int H, int G, int dk, int vd,
                                  torch::Tensor block_tables, int block_size, torch::Tensor positions,
                                  float scale, float softcap, const float* sink, int all_groups,
                                  torch::Tensor tiles, torch::Tensor part) {
  const int NV = all_groups ? G * vd : vd;
  TORCH_CHECK(sink_attention_mfma_fits(dk, vd, G, all_groups), "sink_attention_mfma: sizes");
  const int ntiles = tiles.size(0);
  if (ntiles == 0) return part;
  const size_t lds = sam_lds_bytes(dk, NV, false);
  auto stream = at::cuda::getCurrentCUDAStream();
#define SAM_LAUNCH(N, WSETS)                                                               \
  do {                                                                                     \
    auto kern = sink_attention_mfma_kernel<N, WSETS, false>;                                           \
    static int raised = 0;     /* per variant; not repeated under graph capture */         \
    if (lds > 64 * 1024 && (int)lds > raised) {                                            \
      TORCH_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(kern),                 \
                      hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) == hipSuccess, \
                  "sink attention: cannot raise the LDS limit");                           \
      raised = (int)lds;                                                                   \
    }                                                                                      \
    kern<<<dim3(ntiles, H), 256 * WSETS, lds, stream>>>(                                           \
        reinterpret_cast<const bf16_t*>(q.data_ptr()),                                     \
        reinterpret_cast<const bf16_t*>(cache.data_ptr()), block_tables.data_ptr<int>(),   \
        (int)block_tables.size(1), block_size, positions.data_ptr<int>(),                  \
        tiles.data_ptr<int>(), H, G, dk, vd, scale, softcap, sink, all_groups,             \
        part.data_ptr<float>(), 1, nullptr);                                               \
  } while (0)
  const int nt = (NV + 15) / 16;
  if (nt <= 4) SAM_LAUNCH(4, 1);
  else if (nt <= 8) SAM_LAUNCH(8, 1);
  else if (nt <= 16) SAM_LAUNCH(16, 1);
  else if (nt <= 32) SAM_LAUNCH(16, 2);
  else SAM_LAUNCH(24, 2);
#undef SAM_LAUNCH
  SM_CHECK_LAUNCH();
  return part;
}

// Decode steps: every row of the step is one token. The key range of a token
// is split over ksplit workgroups, chosen from host-side sizes only (token
// count, block-table width) so that a captured step keeps its grid.
torch::Tensor sink_attention_heads(torch::Tensor q, torch::Tensor cache, int H, int G, int dk, int vd,
                                   torch::Tensor block_tables, int block_size, torch::Tensor tok_seq,
                                   torch::Tensor positions, float scale, float softcap,
                                   const float* sink, int all_groups, torch::Tensor part) {
  TORCH_CHECK(sink_attention_heads_fits(H, dk, vd, G), "sink_attention_heads: sizes");
  const int64_t Tn = q.size(0);
  if (Tn == 0) return part;
  const int NV = G * vd;
  const int64_t max_keys = block_tables.size(1) * (int64_t)block_size;
  const int max_blk = (int)std::max<int64_t>(1, SM_CDIV(max_keys, SAM_KB));
  const int ksplit = (int)std::min<int64_t>(max_blk, std::max<int64_t>(1, 1024 / Tn));
  auto f32 = q.options().dtype(at::kFloat);
  auto pacc = torch::empty({Tn, H, ksplit, NV}, f32);
  auto pml = torch::empty({Tn, H, ksplit, 2}, f32);
  const size_t lds = sam_lds_bytes(dk, NV, true);
  auto stream = at::cuda::getCurrentCUDAStream();
#define SAM_LAUNCH(N, WSETS)                                                               \
  do {                                                                                     \
    auto kern = sink_attention_mfma_kernel<N, WSETS, true>;                                     \
    static int raised = 0;                                                                 \
    if (lds > 64 * 1024 && (int)lds > raised) {                                            \
      TORCH_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(kern),                 \
                      hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) == hipSuccess, \
                  "sink attention: cannot raise the LDS limit");                           \
      raised = (int)lds;                                                                   \
    }                                                                                      \
    kern<<<dim3(Tn, ksplit), 256 * WSETS, lds, stream>>>(                                          \
        reinterpret_cast<const bf16_t*>(q.data_ptr()),                                     \
        reinterpret_cast<const bf16_t*>(cache.data_ptr()), block_tables.data_ptr<int>(),   \
        (int)block_tables.size(1), block_size, positions.data_ptr<int>(),                  \
        tok_seq.data_ptr<int>(), H, G, dk, vd, scale, softcap, sink, all_groups,           \
        pacc.data_ptr<float>(), ksplit, pml.data_ptr<float>());                            \
  } while (0)
  const int nt = (NV + 15) / 16;
  if (nt <= 4) SAM_LAUNCH(4, 1);
  else if (nt <= 8) SAM_LAUNCH(8, 1);
  else if (nt <= 16) SAM_LAUNCH(16, 1);
  else if (nt <= 32) SAM_LAUNCH(16, 2);
  else SAM_LAUNCH(24, 2);
#undef SAM_LAUNCH
  SM_CHECK_LAUNCH();
  sink_attention_merge_kernel<<<dim3(Tn, H), 256, 0, stream>>>(
      pacc.data_ptr<float>(), pml.data_ptr<float>(), sink, H, G, vd, ksplit, all_groups,
      part.data_ptr<float>());
  SM_CHECK_LAUNCH();
  return part;
}
