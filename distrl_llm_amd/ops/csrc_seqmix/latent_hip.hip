#include "hip/hip_runtime.h"
// Latent attention: cache write (latent RMS norm + rotated shared key part),
// query rotation, and windowed softmax attention in latent space over the
// paged cache. Prompt portions and single decode tokens run in the same
// launch: one wave per (token, head).
#include <torch/extension.h>
#include <ATen/hip/HIPContext.h>
#include "seqmix_common.h"

namespace {

// angle of pair i at position p: p * base^(-2 i / dims), all fp32
SM_INLINE void rot_cs(int p, int i, float base, int dims, float* c, float* s) {
  const float f = powf(base, -2.0f * (float)i / (float)dims);
  sincosf((float)p * f, s, c);
}

// One workgroup per token. proj row = [q (H * (dn + rd)) | d (r + rd)].
template <typename T>
__global__ __launch_bounds__(256) void latent_prepare_kernel(
    const T* __restrict__ proj, int P, int H, int dn, int rd, int r, int own,
    const float* __restrict__ norm_w, float eps, const int* __restrict__ positions,
    float base, int dims, const int* __restrict__ page_slot, T* __restrict__ cache,
    float* __restrict__ q_rot) {
  __shared__ float red[4];
  const int64_t t = blockIdx.x;
  const T* row = proj + t * P;
  const int p = positions[t];
  const int half = dims / 2;
  // rotated query part of every head
  for (int i = threadIdx.x; i < H * rd; i += blockDim.x) {
    const int hd = i / rd, k = i % rd;
    const T* qr = row + hd * (dn + rd) + dn;
    float v;
    if (k < dims) {
      const int pi = (k < half) ? k : k - half;
      float c, s;
      rot_cs(p, pi, base, dims, &c, &s);
      const float a = to_f(qr[pi]), b = to_f(qr[pi + half]);
      v = (k < half) ? a * c - b * s : b * c + a * s;
    } else {
      v = to_f(qr[k]);
    }
    q_rot[(t * H + hd) * rd + k] = v;
  }
  if (!own) return;
  const T* d = row + H * (dn + rd);
  float ss = 0.f;
  for (int k = threadIdx.x; k < r; k += blockDim.x) {
    const float v = to_f(d[k]);
    ss += v * v;
  }
  ss = sm_block_sum(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)r + eps);
  T* dst = cache + (int64_t)page_slot[t] * (r + rd);
  for (int k = threadIdx.x; k < r; k += blockDim.x)
    dst[k] = from_f<T>(to_f(d[k]) * inv * norm_w[k]);
  for (int k = threadIdx.x; k < rd; k += blockDim.x) {
    float v;
    if (k < dims) {
      const int pi = (k < half) ? k : k - half;
      float c, s;
      rot_cs(p, pi, base, dims, &c, &s);
      const float a = to_f(d[r + pi]), b = to_f(d[r + pi + half]);
      v = (k < half) ? a * c - b * s : b * c + a * s;
    } else {
      v = to_f(d[r + k]);
    }
    dst[r + k] = from_f<T>(v);
  }
}

// One wave per (token, head). Keys lo..p of the token's sequence are taken
// 64 at a time: lane l scores key l (dot over the whole cache row), an
// online softmax carries max and sum across chunks, then the lanes switch
// to the latent axis and accumulate sum_j p_j c_j.
#define SM_LAT_REGS 16   // latent dims per lane: kv_rank <= 64 * 16
template <typename T>
__global__ __launch_bounds__(64) void latent_attention_kernel(
    const T* __restrict__ q_lat,      // [H, Tn, r]
    const float* __restrict__ q_rot,  // [Tn, H, rd]
    const T* __restrict__ cache,      // [rows, r + rd]
    const int* __restrict__ block_tables, int max_nb, int block_size,
    const int* __restrict__ tok_seq, const int* __restrict__ positions,
    int Tn, int H, int r, int rd, int window, float scale,
    T* __restrict__ out) {            // [H, Tn, r]
  extern __shared__ float lds[];
  float* q = lds;                       // r + rd
  float* pw = lds + r + rd;             // 64 weights
  int* krow = reinterpret_cast<int*>(pw + 64);   // 64 cache rows
  const int t = blockIdx.x, hd = blockIdx.y, lane = threadIdx.x;
  const int W = r + rd;
  for (int k = lane; k < r; k += 64) q[k] = to_f(q_lat[((int64_t)hd * Tn + t) * r + k]);
  for (int k = lane; k < rd; k += 64) q[r + k] = q_rot[((int64_t)t * H + hd) * rd + k];
  const int b = tok_seq[t], p = positions[t];
  const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
  const int* bt = block_tables + (int64_t)b * max_nb;
  float m = -INFINITY, l = 0.f;
  float acc[SM_LAT_REGS];
  #pragma unroll
  for (int i = 0; i < SM_LAT_REGS; ++i) acc[i] = 0.f;
  __syncthreads();
  for (int j0 = lo; j0 <= p; j0 += 64) {
    const int j = j0 + lane;
    float s = -INFINITY;
    int row = 0;
    if (j <= p) {
      row = bt[j / block_size] * block_size + j % block_size;
      const T* kv = cache + (int64_t)row * W;
      float dot = 0.f;
      for (int k = 0; k < W; ++k) dot += q[k] * to_f(kv[k]);
      s = dot * scale;
    }
    const float m_new = fmaxf(m, sm_wave_max(s));
    const float pj = (j <= p) ? expf(s - m_new) : 0.f;
    const float corr = expf(m - m_new);          // first chunk: exp(-inf) = 0
    l = l * corr + sm_wave_sum(pj);
    m = m_new;
    __syncthreads();
    pw[lane] = pj;
    krow[lane] = row;
    __syncthreads();
    const int nk = min(64, p - j0 + 1);
    #pragma unroll
    for (int i = 0; i < SM_LAT_REGS; ++i) {
      const int k = lane + 64 * i;
      if (k < r) {
        float a = acc[i] * corr;
        for (int jj = 0; jj < nk; ++jj)
          a += pw[jj] * to_f(cache[(int64_t)krow[jj] * W + k]);
        acc[i] = a;
      }
    }
  }
  const float invl = 1.0f / l;
  #pragma unroll
  for (int i = 0; i < SM_LAT_REGS; ++i) {
    const int k = lane + 64 * i;
    if (k < r) out[((int64_t)hd * Tn + t) * r + k] = from_f<T>(acc[i] * invl);
  }
}

}  // namespace

torch::Tensor latent_prepare(torch::Tensor proj, int64_t heads, int64_t dim,
                             int64_t rot_dim, int64_t kv_rank, bool own_cache,
                             c10::optional<torch::Tensor> norm_w, double eps,
                             torch::Tensor positions, double rope_base,
                             int64_t rope_dims, torch::Tensor page_slot,
                             torch::Tensor cache) {
  SM_CHECK_CUDA(proj); SM_CHECK_CUDA(positions); SM_CHECK_I32(positions);
  SM_CHECK_CUDA(page_slot); SM_CHECK_I32(page_slot); SM_CHECK_CUDA(cache);
  const int64_t T = proj.size(0);
  const int P = proj.size(1);
  const int64_t qs = heads * (dim + rot_dim);
  TORCH_CHECK(P == qs + (own_cache ? kv_rank + rot_dim : 0), "latent_prepare: projection width");
  TORCH_CHECK(rope_dims % 2 == 0 && rope_dims <= rot_dim, "latent_prepare: rope dims");
  TORCH_CHECK(positions.numel() == T && page_slot.numel() == T, "latent_prepare: batch layout");
  TORCH_CHECK(cache.dim() == 2 && cache.size(1) == kv_rank + rot_dim &&
              cache.scalar_type() == proj.scalar_type(), "latent_prepare: cache shape/dtype");
  const float* nw = nullptr;
  if (own_cache) {
    TORCH_CHECK(norm_w.has_value(), "latent_prepare: norm weight missing");
    SM_CHECK_CUDA(*norm_w); SM_CHECK_F32(*norm_w);
    TORCH_CHECK(norm_w->numel() == kv_rank, "latent_prepare: norm weight size");
    nw = norm_w->data_ptr<float>();
  }
  auto q_rot = torch::empty({T, heads, rot_dim}, proj.options().dtype(at::kFloat));
  if (T == 0) return q_rot;
  auto stream = at::hip::getCurrentHIPStreamMasqueradingAsCUDA();
  if (proj.scalar_type() == at::kBFloat16)
   hipLaunchKernelGGL(( latent_prepare_kernel<bf16_t>), dim3(T), dim3(256), 0, stream, 
        reinterpret_cast<const bf16_t*>(proj.data_ptr()), P, heads, dim, rot_dim, kv_rank,
        own_cache ? 1 : 0, nw, (float)eps, positions.data_ptr<int>(), (float)rope_base,
        (int)rope_dims, page_slot.data_ptr<int>(), reinterpret_cast<bf16_t*>(cache.data_ptr()),
        q_rot.data_ptr<float>());
  else {
    SM_CHECK_F32(proj);
   hipLaunchKernelGGL(( latent_prepare_kernel<float>), dim3(T), dim3(256), 0, stream, 
        proj.data_ptr<float>(), P, heads, dim, rot_dim, kv_rank, own_cache ? 1 : 0, nw,
        (float)eps, positions.data_ptr<int>(), (float)rope_base, (int)rope_dims,
        page_slot.data_ptr<int>(), cache.data_ptr<float>(), q_rot.data_ptr<float>());
  }
  SM_CHECK_LAUNCH();
  return q_rot;
}

torch::Tensor latent_window_attention(torch::Tensor q_lat, torch::Tensor q_rot,
                                      torch::Tensor cache, int64_t kv_rank,
                                      torch::Tensor block_tables, int64_t block_size,
                                      torch::Tensor tok_seq, torch::Tensor positions,
                                      int64_t window, double scale) {
  SM_CHECK_CUDA(q_lat); SM_CHECK_CUDA(q_rot); SM_CHECK_F32(q_rot); SM_CHECK_CUDA(cache);
  SM_CHECK_CUDA(block_tables); SM_CHECK_I32(block_tables);
  SM_CHECK_CUDA(tok_seq); SM_CHECK_I32(tok_seq); SM_CHECK_CUDA(positions); SM_CHECK_I32(positions);
  TORCH_CHECK(q_lat.dim() == 3 && q_rot.dim() == 3 && block_tables.dim() == 2, "latent attention: ranks");
  const int H = q_lat.size(0);
  const int64_t T = q_lat.size(1);
  const int r = q_lat.size(2);
  const int rd = q_rot.size(2);
  TORCH_CHECK(r == kv_rank && r <= 64 * SM_LAT_REGS, "latent attention: kv_rank unsupported");
  TORCH_CHECK(q_rot.size(0) == T && q_rot.size(1) == H, "latent attention: q_rot shape");
  TORCH_CHECK(cache.size(1) == r + rd && cache.scalar_type() == q_lat.scalar_type(),
              "latent attention: cache shape/dtype");
  TORCH_CHECK(tok_seq.numel() == T && positions.numel() == T && block_size > 0, "latent attention: batch layout");
  auto out = torch::empty_like(q_lat);
  if (T == 0) return out;
  auto stream = at::hip::getCurrentHIPStreamMasqueradingAsCUDA();
  const size_t lds = (size_t)(r + rd + 64) * sizeof(float) + 64 * sizeof(int);
  dim3 grid(T, H);
  if (q_lat.scalar_type() == at::kBFloat16)
   hipLaunchKernelGGL(( latent_attention_kernel<bf16_t>), dim3(grid), dim3(64), lds, stream, 
        reinterpret_cast<const bf16_t*>(q_lat.data_ptr()), q_rot.data_ptr<float>(),
        reinterpret_cast<const bf16_t*>(cache.data_ptr()), block_tables.data_ptr<int>(),
        (int)block_tables.size(1), (int)block_size, tok_seq.data_ptr<int>(),
        positions.data_ptr<int>(), (int)T, H, r, rd, (int)window, (float)scale,
        reinterpret_cast<bf16_t*>(out.data_ptr()));
  else {
    SM_CHECK_F32(q_lat);
   hipLaunchKernelGGL(( latent_attention_kernel<float>), dim3(grid), dim3(64), lds, stream, 
        q_lat.data_ptr<float>(), q_rot.data_ptr<float>(), cache.data_ptr<float>(),
        block_tables.data_ptr<int>(), (int)block_tables.size(1), (int)block_size,
        tok_seq.data_ptr<int>(), positions.data_ptr<int>(), (int)T, H, r, rd,
        (int)window, (float)scale, out.data_ptr<float>());
  }
  SM_CHECK_LAUNCH();
  return out;
}
