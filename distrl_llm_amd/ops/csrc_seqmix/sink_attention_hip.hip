#include "hip/hip_runtime.h"
// Grouped-query softmax attention over paged [k | v] rows with the extras of
// the sandwich designs: interleaved-pair rotary on the leading dims of every
// q/k head, value blending with an earlier layer's values at cache-write
// time, tanh-capped scores, a per-head sink in the softmax denominator and
// mixing of the heads' weights by a learned matrix.
//
// Head mixing without the T x T weights: with w_g = p_g / l_g the mixed
// output of head h is sum_g talk[h, g] * (sum_j w_g(j) v_c(h)(j)), so the
// attention kernels produce, per query head g, the normalised weighted value
// sums over EVERY kv head ("part" [T, H, G * vdim], fp32), and a small
// kernel mixes them. Without a mixing matrix only the head's own kv head is
// summed.
#include <torch/extension.h>
#include <ATen/hip/HIPContext.h>
#include "seqmix_common.h"

namespace {

// angle of pair i at position p: p * base^(-2 i / dims); the frequency is
// rounded once from double, the product and sin/cos are fp32
SM_INLINE void pair_cs(int p, int i, float base, int dims, float* c, float* s) {
  const float f = (float)pow((double)base, -2.0 * (double)i / (double)dims);
  sincosf((float)p * f, s, c);
}

// One workgroup per token. proj row = [q (H dk) | k (G dk) | v (G vd)], rows
// ldp apart. Writes rotated q (T dtype) and the cache row [k rotated | v].
template <typename T>
__global__ __launch_bounds__(256) void rope_kv_write_kernel(
    const T* __restrict__ proj, int64_t ldp, int H, int G, int dk, int vd,
    const int* __restrict__ positions, float base, int dims,
    const int* __restrict__ page_slot, T* __restrict__ cache,
    const float* __restrict__ vmix, const T* __restrict__ v_first, int64_t ldv,
    T* __restrict__ q_out) {
  const int64_t t = blockIdx.x;
  const T* row = proj + t * ldp;
  const int p = positions[t];
  const int W = G * (dk + vd);
  T* dst = cache + (int64_t)page_slot[t] * W;
  const int nq = H * dk, nk = G * dk, nv = G * vd;
  // rotated pairs of q heads then k heads
  const int rp = dims / 2;                 // rotated pairs per head
  for (int i = threadIdx.x; i < (H + G) * rp; i += blockDim.x) {
    const int hd = i / rp, pi = i % rp;
    float c, s;
    pair_cs(p, pi, base, dims, &c, &s);
    const T* src = row + (int64_t)hd * dk + 2 * pi;     // q heads and k heads are adjacent
    const float a = to_f(src[0]), b = to_f(src[1]);
    const T ra = from_f<T>(a * c - b * s), rb = from_f<T>(b * c + a * s);
    T* o = (hd < H) ? q_out + t * nq + hd * dk + 2 * pi
                    : dst + (hd - H) * dk + 2 * pi;
    o[0] = ra;
    o[1] = rb;
  }
  // unrotated tail of every head
  const int rest = dk - dims;
  for (int i = threadIdx.x; i < (H + G) * rest; i += blockDim.x) {
    const int hd = i / rest, k = dims + i % rest;
    const T v = row[(int64_t)hd * dk + k];
    if (hd < H) q_out[t * nq + hd * dk + k] = v;
    else dst[(hd - H) * dk + k] = v;
  }
  // values, blended with the first mixing layer's
  const float lam = (v_first != nullptr) ? vmix[0] : 0.f;
  for (int i = threadIdx.x; i < nv; i += blockDim.x) {
    float v = to_f(row[nq + nk + i]);
    if (v_first != nullptr) v = (1.0f - lam) * v + lam * to_f(v_first[t * ldv + i]);
    dst[nk + i] = from_f<T>(v);
  }
}

// One wave per (token, head). Keys 0..p of the token's sequence are taken 64
// at a time: lane l scores key l, an online softmax carries max and sum
// across chunks (started at the sink: m = sink, l = 1), then the lanes switch
// to the value axis and accumulate sum_j p_j v_j over NV = groups * vd dims.
#define SA_REGS 32   // value dims per lane: groups * vd <= 64 * 32
template <typename T>
__global__ __launch_bounds__(64) void sink_attention_kernel(
    const T* __restrict__ q,          // [Tn, H, dk]
    const T* __restrict__ cache,      // [rows, G (dk + vd)]
    const int* __restrict__ block_tables, int max_nb, int block_size,
    const int* __restrict__ tok_seq, const int* __restrict__ positions,
    int H, int G, int dk, int vd, float scale, float softcap,
    const float* __restrict__ sink, int all_groups,
    float* __restrict__ part) {       // [Tn, H, NV]
  extern __shared__ float lds[];
  float* qs = lds;                      // dk
  float* pw = lds + dk;                 // 64 weights
  int* krow = reinterpret_cast<int*>(pw + 64);
  const int t = blockIdx.x, hd = blockIdx.y, lane = threadIdx.x;
  const int W = G * (dk + vd);
  const int grp = hd / (H / G);
  const int NV = all_groups ? G * vd : vd;
  const int voff = G * dk + (all_groups ? 0 : grp * vd);
  for (int k = lane; k < dk; k += 64) qs[k] = to_f(q[((int64_t)t * H + hd) * dk + k]);
  const int b = tok_seq[t], p = positions[t];
  const int* bt = block_tables + (int64_t)b * max_nb;
  float m = (sink != nullptr) ? sink[hd] : -INFINITY;
  float l = (sink != nullptr) ? 1.f : 0.f;
  float acc[SA_REGS];
  #pragma unroll
  for (int i = 0; i < SA_REGS; ++i) acc[i] = 0.f;
  __syncthreads();
  for (int j0 = 0; j0 <= p; j0 += 64) {
    const int j = j0 + lane;
    float s = -INFINITY;
    int row = 0;
    if (j <= p) {
      row = bt[j / block_size] * block_size + j % block_size;
      const T* kr = cache + (int64_t)row * W + grp * dk;
      float dot = 0.f;
      for (int k = 0; k < dk; ++k) dot += qs[k] * to_f(kr[k]);
      s = dot * scale;
      if (softcap > 0.f) s = softcap * tanhf(s / softcap);
    }
    const float m_new = fmaxf(m, sm_wave_max(s));      // finite: key j0 always exists
    const float pj = (j <= p) ? expf(s - m_new) : 0.f;
    const float corr = expf(m - m_new);                // no sink, first chunk: exp(-inf) = 0
    l = l * corr + sm_wave_sum(pj);
    m = m_new;
    __syncthreads();
    pw[lane] = pj;
    krow[lane] = row;
    __syncthreads();
    const int nk = min(64, p - j0 + 1);
    #pragma unroll
    for (int i = 0; i < SA_REGS; ++i) {
      const int f = lane + 64 * i;
      if (f < NV) {
        float a = acc[i] * corr;
        for (int jj = 0; jj < nk; ++jj)
          a += pw[jj] * to_f(cache[(int64_t)krow[jj] * W + voff + f]);
        acc[i] = a;
      }
    }
  }
  const float inv = 1.0f / l;
  #pragma unroll
  for (int i = 0; i < SA_REGS; ++i) {
    const int f = lane + 64 * i;
    if (f < NV) part[((int64_t)t * H + hd) * NV + f] = acc[i] * inv;
  }
}

// out[t, h, d] = sum_g talk[h, g] * part[t, g, c(h) vd + d]  (talk given), or
// part[t, h, d] (no mixing: the part holds the head's own kv head only).
template <typename T>
__global__ __launch_bounds__(256) void head_mix_kernel(
    const float* __restrict__ part, const float* __restrict__ talk, int H, int G,
    int vd, T* __restrict__ out) {
  const int64_t t = blockIdx.x;
  const int rep = H / G;
  for (int i = threadIdx.x; i < H * vd; i += blockDim.x) {
    const int h = i / vd, d = i % vd;
    float a;
    if (talk != nullptr) {
      const float* src = part + t * H * G * vd + (h / rep) * vd + d;
      a = 0.f;
      for (int g = 0; g < H; ++g) a += talk[h * H + g] * src[(int64_t)g * G * vd];
    } else {
      a = part[(t * H + h) * vd + d];
    }
    out[t * H * vd + i] = from_f<T>(a);
  }
}

}  // namespace

torch::Tensor rope_kv_write(torch::Tensor proj, int64_t heads, int64_t kv_heads,
                            int64_t dim, int64_t vdim, torch::Tensor positions,
                            double rope_base, int64_t rope_dims, torch::Tensor page_slot,
                            torch::Tensor cache, c10::optional<torch::Tensor> vmix,
                            c10::optional<torch::Tensor> v_first) {
  TORCH_CHECK(proj.is_cuda() && proj.dim() == 2 && proj.stride(1) == 1, "rope_kv_write: proj must be row-major");
  SM_CHECK_CUDA(positions); SM_CHECK_I32(positions); SM_CHECK_CUDA(page_slot); SM_CHECK_I32(page_slot);
  SM_CHECK_CUDA(cache);
  const int64_t T = proj.size(0);
  const int H = heads, G = kv_heads, dk = dim, vd = vdim;
  const int W = G * (dk + vd);
  TORCH_CHECK(G >= 1 && H % G == 0, "rope_kv_write: heads must be a multiple of kv_heads");
  TORCH_CHECK(proj.size(1) == H * dk + W, "rope_kv_write: projection width");
  TORCH_CHECK(cache.dim() == 2 && cache.size(1) == W && cache.scalar_type() == proj.scalar_type(),
              "rope_kv_write: cache layout");
  TORCH_CHECK(rope_dims >= 0 && rope_dims <= dk && rope_dims % 2 == 0, "rope_kv_write: rope dims");
  TORCH_CHECK(positions.numel() == T && page_slot.numel() == T, "rope_kv_write: per-token inputs");
  const void* vf = nullptr;
  int64_t ldv = 0;
  const float* lam = nullptr;
  if (v_first.has_value()) {
    TORCH_CHECK(vmix.has_value(), "rope_kv_write: v_first needs vmix");
    SM_CHECK_CUDA(*vmix); SM_CHECK_F32(*vmix);
    TORCH_CHECK(v_first->is_cuda() && v_first->dim() == 2 && v_first->stride(1) == 1 &&
                v_first->size(0) == T && v_first->size(1) == G * vd &&
                v_first->scalar_type() == proj.scalar_type(), "rope_kv_write: v_first layout");
    vf = v_first->data_ptr();
    ldv = v_first->stride(0);
    lam = vmix->data_ptr<float>();
  }
  auto q = torch::empty({T, H, dk}, proj.options());
  if (T == 0) return q;
  auto stream = at::hip::getCurrentHIPStreamMasqueradingAsCUDA();
  if (proj.scalar_type() == at::kBFloat16)
   hipLaunchKernelGGL(( rope_kv_write_kernel<bf16_t>), dim3(T), dim3(256), 0, stream, 
        reinterpret_cast<const bf16_t*>(proj.data_ptr()), proj.stride(0), H, G, dk, vd,
        positions.data_ptr<int>(), (float)rope_base, (int)rope_dims, page_slot.data_ptr<int>(),
        reinterpret_cast<bf16_t*>(cache.data_ptr()), lam, reinterpret_cast<const bf16_t*>(vf), ldv,
        reinterpret_cast<bf16_t*>(q.data_ptr()));
  else {
    SM_CHECK_F32(proj);
   hipLaunchKernelGGL(( rope_kv_write_kernel<float>), dim3(T), dim3(256), 0, stream, 
        proj.data_ptr<float>(), proj.stride(0), H, G, dk, vd, positions.data_ptr<int>(),
        (float)rope_base, (int)rope_dims, page_slot.data_ptr<int>(), cache.data_ptr<float>(), lam,
        reinterpret_cast<const float*>(vf), ldv, q.data_ptr<float>());
  }
  SM_CHECK_LAUNCH();
  return q;
}

torch::Tensor sink_attention_mfma(torch::Tensor q, torch::Tensor cache, int H, int G, int dk, int vd,
                                  torch::Tensor block_tables, int block_size, torch::Tensor positions,
                                  float scale, float softcap, const float* sink, int all_groups,
                                  torch::Tensor tiles, torch::Tensor part);
bool sink_attention_mfma_fits(int dk, int vd, int G, int all_groups);
torch::Tensor sink_attention_heads(torch::Tensor q, torch::Tensor cache, int H, int G, int dk, int vd,
                                   torch::Tensor block_tables, int block_size, torch::Tensor tok_seq,
                                   torch::Tensor positions, float scale, float softcap,
                                   const float* sink, int all_groups, torch::Tensor part);
bool sink_attention_heads_fits(int H, int dk, int vd, int G);

torch::Tensor sink_attention(torch::Tensor q, torch::Tensor cache, int64_t heads,
                             int64_t kv_heads, int64_t dim, int64_t vdim,
                             torch::Tensor block_tables, int64_t block_size,
                             torch::Tensor tok_seq, torch::Tensor positions, double scale,
                             double softcap, c10::optional<torch::Tensor> sink,
                             c10::optional<torch::Tensor> talk,
                             c10::optional<torch::Tensor> tiles, int64_t max_tile_queries) {
  SM_CHECK_CUDA(q); SM_CHECK_CUDA(cache);
  SM_CHECK_CUDA(block_tables); SM_CHECK_I32(block_tables);
  SM_CHECK_CUDA(tok_seq); SM_CHECK_I32(tok_seq); SM_CHECK_CUDA(positions); SM_CHECK_I32(positions);
  const int H = heads, G = kv_heads, dk = dim, vd = vdim;
  const int64_t Tn = q.size(0);
  TORCH_CHECK(G >= 1 && H % G == 0, "sink_attention: heads must be a multiple of kv_heads");
  TORCH_CHECK(q.dim() == 3 && q.size(1) == H && q.size(2) == dk, "sink_attention: q is [T, H, dim]");
  TORCH_CHECK(cache.dim() == 2 && cache.size(1) == G * (dk + vd) && cache.scalar_type() == q.scalar_type(),
              "sink_attention: cache layout");
  TORCH_CHECK(block_tables.dim() == 2 && tok_seq.numel() == Tn && positions.numel() == Tn && block_size >= 1,
              "sink_attention: batch layout");
  const float* sinkp = nullptr;
  if (sink.has_value()) {
    SM_CHECK_CUDA(*sink); SM_CHECK_F32(*sink);
    TORCH_CHECK(sink->numel() == H, "sink_attention: one sink per head");
    sinkp = sink->data_ptr<float>();
  }
  const float* talkp = nullptr;
  if (talk.has_value()) {
    SM_CHECK_CUDA(*talk); SM_CHECK_F32(*talk);
    TORCH_CHECK(talk->dim() == 2 && talk->size(0) == H && talk->size(1) == H, "sink_attention: talk is [H, H]");
    talkp = talk->data_ptr<float>();
  }
  const int all_groups = (talkp != nullptr && G > 1) ? 1 : 0;
  const int NV = all_groups ? G * vd : vd;
  TORCH_CHECK(NV <= 64 * SA_REGS, "sink_attention: kv_heads * vdim too large");
  auto out = torch::empty({Tn, (int64_t)H * vd}, q.options());
  if (Tn == 0) return out;
  auto part = torch::empty({Tn, H, NV}, q.options().dtype(at::kFloat));
  auto stream = at::hip::getCurrentHIPStreamMasqueradingAsCUDA();
  const bool bf16 = q.scalar_type() == at::kBFloat16;
  if (bf16 && tiles.has_value() && max_tile_queries > 1 && sink_attention_mfma_fits(dk, vd, G, all_groups)) {
    SM_CHECK_CUDA(*tiles); SM_CHECK_I32(*tiles);
    TORCH_CHECK(tiles->dim() == 2 && tiles->size(1) == 3 && max_tile_queries <= 64, "sink_attention: tiles");
    sink_attention_mfma(q, cache, H, G, dk, vd, block_tables, (int)block_size, positions, (float)scale,
                        (float)softcap, sinkp, all_groups, *tiles, part);
  } else if (bf16 && tiles.has_value() && max_tile_queries == 1 &&
             sink_attention_heads_fits(H, dk, vd, G)) {
    // a decode step: one token per row
    sink_attention_heads(q, cache, H, G, dk, vd, block_tables, (int)block_size, tok_seq, positions,
                         (float)scale, (float)softcap, sinkp, all_groups, part);
  } else {
    const size_t lds = (dk + 64) * sizeof(float) + 64 * sizeof(int);
    dim3 grid(Tn, H);
    if (bf16)
     hipLaunchKernelGGL(( sink_attention_kernel<bf16_t>), dim3(grid), dim3(64), lds, stream, 
          reinterpret_cast<const bf16_t*>(q.data_ptr()), reinterpret_cast<const bf16_t*>(cache.data_ptr()),
          block_tables.data_ptr<int>(), (int)block_tables.size(1), (int)block_size,
          tok_seq.data_ptr<int>(), positions.data_ptr<int>(), H, G, dk, vd, (float)scale,
          (float)softcap, sinkp, all_groups, part.data_ptr<float>());
    else {
      SM_CHECK_F32(q);
     hipLaunchKernelGGL(( sink_attention_kernel<float>), dim3(grid), dim3(64), lds, stream, 
          q.data_ptr<float>(), cache.data_ptr<float>(), block_tables.data_ptr<int>(),
          (int)block_tables.size(1), (int)block_size, tok_seq.data_ptr<int>(),
          positions.data_ptr<int>(), H, G, dk, vd, (float)scale, (float)softcap, sinkp, all_groups,
          part.data_ptr<float>());
    }
    SM_CHECK_LAUNCH();
  }
  // with one kv head the part of head g is already over "every" kv head
  const float* mixp = talkp;
  if (bf16)
   hipLaunchKernelGGL(( head_mix_kernel<bf16_t>), dim3(Tn), dim3(256), 0, stream, part.data_ptr<float>(), mixp, H, all_groups ? G : 1, vd,
                                                    reinterpret_cast<bf16_t*>(out.data_ptr()));
  else
   hipLaunchKernelGGL(( head_mix_kernel<float>), dim3(Tn), dim3(256), 0, stream, part.data_ptr<float>(), mixp, H, all_groups ? G : 1, vd,
                                                   out.data_ptr<float>());
  SM_CHECK_LAUNCH();
  return out;
}
