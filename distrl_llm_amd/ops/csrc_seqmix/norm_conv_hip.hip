#include "hip/hip_runtime.h"
// Offset-weight RMS norm, short causal depthwise convolution with per-slot
// tails, and the gated parallel-residual update (alone, and fused with the
// next layer's norm). One workgroup per token row for the row-wise ops.
#include <torch/extension.h>
#include <ATen/hip/HIPContext.h>
#include "seqmix_common.h"

namespace {

// h = x / sqrt(mean(x^2) + eps) * (1 + w); written as fp32 and (if hb) as T.
template <typename Tin, typename T>
__global__ __launch_bounds__(256) void offset_rmsnorm_kernel(
    const Tin* __restrict__ x, const float* __restrict__ w, float eps, int D,
    float* __restrict__ h32, T* __restrict__ hb) {
  __shared__ float red[4];
  const int64_t row = blockIdx.x;
  const Tin* xr = x + row * D;
  float ss = 0.f;
  for (int d = threadIdx.x; d < D; d += blockDim.x) {
    const float v = to_f(xr[d]);
    ss += v * v;
  }
  ss = sm_block_sum(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)D + eps);
  for (int d = threadIdx.x; d < D; d += blockDim.x) {
    const float v = to_f(xr[d]) * inv * (1.0f + w[d]);
    h32[row * D + d] = v;
    if (hb != nullptr) hb[row * D + d] = from_f<T>(v);
  }
}

// x += mult * (mix * sigmoid(g1 + b1) + ff * sigmoid(g2 + b2)); optionally
// followed by the next offset RMS norm of the new row.
template <typename T>
__global__ __launch_bounds__(256) void gated_residual_kernel(
    float* __restrict__ x, const T* __restrict__ mix, const float* __restrict__ ff,
    const T* __restrict__ gates, const float* __restrict__ gate_b, float mult,
    int D, int G, const float* __restrict__ next_w, float eps,
    float* __restrict__ h32, T* __restrict__ hb) {
  __shared__ float red[4];
  const int64_t row = blockIdx.x;
  float ss = 0.f;
  for (int d = threadIdx.x; d < D; d += blockDim.x) {
    float acc = to_f(mix[row * D + d]) * sm_sigmoid(to_f(gates[row * G + d]) + gate_b[d]);
    if (ff != nullptr)
      acc += ff[row * D + d] * sm_sigmoid(to_f(gates[row * G + D + d]) + gate_b[D + d]);
    const float v = x[row * D + d] + mult * acc;
    x[row * D + d] = v;
    ss += v * v;
  }
  if (next_w == nullptr) return;
  ss = sm_block_sum(ss, red);   // also orders the row's writes before the re-read
  const float inv = 1.0f / sqrtf(ss / (float)D + eps);
  for (int d = threadIdx.x; d < D; d += blockDim.x) {
    const float v = x[row * D + d] * inv * (1.0f + next_w[d]);
    h32[row * D + d] = v;
    if (hb != nullptr) hb[row * D + d] = from_f<T>(v);
  }
}

// out[t] = h[t] + sum_j w[:, j] * h[t - taps + 1 + j] within the row's
// sequence; inputs before the portion come from tails[slot].
template <typename T>
__global__ __launch_bounds__(256) void tap_conv_kernel(
    const float* __restrict__ h, const float* __restrict__ w,
    const float* __restrict__ tails, const int* __restrict__ cu,
    const int* __restrict__ tok_seq, const int* __restrict__ slots, int D,
    int taps, T* __restrict__ out) {
  const int t = blockIdx.x;
  const int d = blockIdx.y * blockDim.x + threadIdx.x;
  if (d >= D) return;
  const int b = tok_seq[t];
  const int start = cu[b];
  const int rel = t - start;
  const int64_t slot = slots[b];
  float acc = h[(int64_t)t * D + d];
  for (int j = 0; j < taps; ++j) {
    const int src = rel - taps + 1 + j;
    const float v = (src >= 0)
        ? h[(int64_t)(start + src) * D + d]
        : tails[(slot * (taps - 1) + (taps - 1 + src)) * D + d];
    acc += w[d * taps + j] * v;
  }
  out[(int64_t)t * D + d] = from_f<T>(acc);
}

// Advance tails[slot] to the last taps-1 inputs of the row's sequence.
#define SM_MAX_TAILS 15
__global__ __launch_bounds__(256) void tap_tail_kernel(
    const float* __restrict__ h, float* __restrict__ tails,
    const int* __restrict__ cu, const int* __restrict__ slots, int D, int taps) {
  const int b = blockIdx.x;
  const int d = blockIdx.y * blockDim.x + threadIdx.x;
  if (d >= D) return;
  const int start = cu[b], n = cu[b + 1] - start;
  if (n == 0) return;
  const int64_t slot = slots[b];
  const int keep = taps - 1;
  float nv[SM_MAX_TAILS];
  #pragma unroll
  for (int k = 0; k < SM_MAX_TAILS; ++k) {
    if (k < keep) {
      const int src = n - keep + k;
      nv[k] = (src >= 0) ? h[(int64_t)(start + src) * D + d]
                         : tails[(slot * keep + (k + n)) * D + d];
    }
  }
  #pragma unroll
  for (int k = 0; k < SM_MAX_TAILS; ++k)
    if (k < keep) tails[(slot * keep + k) * D + d] = nv[k];
}

}  // namespace

std::vector<torch::Tensor> offset_rmsnorm(torch::Tensor x, torch::Tensor w,
                                          double eps, bool out_bf16) {
  SM_CHECK_CUDA(x); SM_CHECK_CUDA(w); SM_CHECK_F32(w);
  TORCH_CHECK(x.dim() == 2 && w.numel() == x.size(1), "offset_rmsnorm: shapes");
  const int64_t T = x.size(0);
  const int D = x.size(1);
  auto h32 = torch::empty({T, D}, x.options().dtype(at::kFloat));
  torch::Tensor hb = out_bf16 ? torch::empty({T, D}, x.options().dtype(at::kBFloat16)) : h32;
  if (T == 0) return {h32, hb};
  auto stream = at::hip::getCurrentHIPStreamMasqueradingAsCUDA();
  bf16_t* hbp = out_bf16 ? reinterpret_cast<bf16_t*>(hb.data_ptr()) : nullptr;
  if (x.scalar_type() == at::kBFloat16) {
   hipLaunchKernelGGL(( offset_rmsnorm_kernel<bf16_t, bf16_t>), dim3(T), dim3(256), 0, stream, 
        reinterpret_cast<const bf16_t*>(x.data_ptr()), w.data_ptr<float>(),
        (float)eps, D, h32.data_ptr<float>(), hbp);
  } else {
    SM_CHECK_F32(x);
   hipLaunchKernelGGL(( offset_rmsnorm_kernel<float, bf16_t>), dim3(T), dim3(256), 0, stream, 
        x.data_ptr<float>(), w.data_ptr<float>(), (float)eps, D,
        h32.data_ptr<float>(), hbp);
  }
  SM_CHECK_LAUNCH();
  return {h32, hb};
}

static std::vector<torch::Tensor> gated_residual_impl(
    torch::Tensor x, torch::Tensor mix, c10::optional<torch::Tensor> ff,
    torch::Tensor gates, torch::Tensor gate_b, double mult,
    c10::optional<torch::Tensor> next_w, double eps, bool out_bf16) {
  SM_CHECK_CUDA(x); SM_CHECK_F32(x); SM_CHECK_CUDA(mix); SM_CHECK_CUDA(gates);
  SM_CHECK_CUDA(gate_b); SM_CHECK_F32(gate_b);
  const int64_t T = x.size(0);
  const int D = x.size(1);
  const int G = gates.size(1);
  TORCH_CHECK(mix.size(0) == T && mix.size(1) == D && gates.size(0) == T, "gated_residual: shapes");
  TORCH_CHECK(G == (ff.has_value() ? 2 * D : D) && gate_b.numel() == G, "gated_residual: gate width");
  TORCH_CHECK(mix.scalar_type() == gates.scalar_type(), "gated_residual: dtypes");
  const float* ffp = nullptr;
  if (ff.has_value()) {
    SM_CHECK_CUDA(*ff); SM_CHECK_F32(*ff);
    TORCH_CHECK(ff->size(0) == T && ff->size(1) == D, "gated_residual: ff shape");
    ffp = ff->data_ptr<float>();
  }
  torch::Tensor h32, hb;
  const float* nw = nullptr;
  if (next_w.has_value()) {
    SM_CHECK_CUDA(*next_w); SM_CHECK_F32(*next_w);
    TORCH_CHECK(next_w->numel() == D, "gated_residual: norm weight");
    nw = next_w->data_ptr<float>();
    h32 = torch::empty({T, D}, x.options());
    hb = out_bf16 ? torch::empty({T, D}, x.options().dtype(at::kBFloat16)) : h32;
  }
  if (T == 0) return {h32, hb};
  auto stream = at::hip::getCurrentHIPStreamMasqueradingAsCUDA();
  float* h32p = next_w.has_value() ? h32.data_ptr<float>() : nullptr;
  if (mix.scalar_type() == at::kBFloat16) {
    bf16_t* hbp = (next_w.has_value() && out_bf16) ? reinterpret_cast<bf16_t*>(hb.data_ptr()) : nullptr;
   hipLaunchKernelGGL(( gated_residual_kernel<bf16_t>), dim3(T), dim3(256), 0, stream, 
        x.data_ptr<float>(), reinterpret_cast<const bf16_t*>(mix.data_ptr()), ffp,
        reinterpret_cast<const bf16_t*>(gates.data_ptr()), gate_b.data_ptr<float>(),
        (float)mult, D, G, nw, (float)eps, h32p, hbp);
  } else {
    SM_CHECK_F32(mix);
    TORCH_CHECK(!out_bf16, "gated_residual: bf16 output needs bf16 inputs");
   hipLaunchKernelGGL(( gated_residual_kernel<float>), dim3(T), dim3(256), 0, stream, 
        x.data_ptr<float>(), mix.data_ptr<float>(), ffp, gates.data_ptr<float>(),
        gate_b.data_ptr<float>(), (float)mult, D, G, nw, (float)eps, h32p, nullptr);
  }
  SM_CHECK_LAUNCH();
  return {h32, hb};
}

void gated_residual_add(torch::Tensor x, torch::Tensor mix,
                        c10::optional<torch::Tensor> ff, torch::Tensor gates,
                        torch::Tensor gate_b, double mult) {
  gated_residual_impl(x, mix, ff, gates, gate_b, mult, c10::nullopt, 0.0, false);
}

std::vector<torch::Tensor> gated_residual_norm(
    torch::Tensor x, torch::Tensor mix, c10::optional<torch::Tensor> ff,
    torch::Tensor gates, torch::Tensor gate_b, double mult, torch::Tensor next_w,
    double eps, bool out_bf16) {
  return gated_residual_impl(x, mix, ff, gates, gate_b, mult, next_w, eps, out_bf16);
}

torch::Tensor causal_tap_conv(torch::Tensor h, torch::Tensor w, torch::Tensor tails,
                              torch::Tensor cu, torch::Tensor tok_seq,
                              torch::Tensor slots, bool out_bf16) {
  SM_CHECK_CUDA(h); SM_CHECK_F32(h); SM_CHECK_CUDA(w); SM_CHECK_F32(w);
  SM_CHECK_CUDA(tails); SM_CHECK_F32(tails);
  SM_CHECK_CUDA(cu); SM_CHECK_I32(cu); SM_CHECK_CUDA(tok_seq); SM_CHECK_I32(tok_seq);
  SM_CHECK_CUDA(slots); SM_CHECK_I32(slots);
  const int64_t T = h.size(0);
  const int D = h.size(1);
  const int taps = w.size(1);
  const int B = slots.numel();
  TORCH_CHECK(w.size(0) == D && taps >= 1 && taps - 1 <= SM_MAX_TAILS, "tap conv: weight shape");
  TORCH_CHECK(tails.dim() == 3 && tails.size(1) == taps - 1 && tails.size(2) == D, "tap conv: tails shape");
  TORCH_CHECK(cu.numel() == B + 1 && tok_seq.numel() == T, "tap conv: batch layout");
  auto out = torch::empty({T, D}, h.options().dtype(out_bf16 ? at::kBFloat16 : at::kFloat));
  if (T == 0) return out;
  auto stream = at::hip::getCurrentHIPStreamMasqueradingAsCUDA();
  dim3 grid(T, SM_CDIV(D, 256));
  if (out_bf16)
   hipLaunchKernelGGL(( tap_conv_kernel<bf16_t>), dim3(grid), dim3(256), 0, stream, 
        h.data_ptr<float>(), w.data_ptr<float>(), tails.data_ptr<float>(),
        cu.data_ptr<int>(), tok_seq.data_ptr<int>(), slots.data_ptr<int>(), D, taps,
        reinterpret_cast<bf16_t*>(out.data_ptr()));
  else
   hipLaunchKernelGGL(( tap_conv_kernel<float>), dim3(grid), dim3(256), 0, stream, 
        h.data_ptr<float>(), w.data_ptr<float>(), tails.data_ptr<float>(),
        cu.data_ptr<int>(), tok_seq.data_ptr<int>(), slots.data_ptr<int>(), D, taps,
        out.data_ptr<float>());
  SM_CHECK_LAUNCH();
  if (taps > 1) {
    dim3 g2(B, SM_CDIV(D, 256));
   hipLaunchKernelGGL(( tap_tail_kernel), dim3(g2), dim3(256), 0, stream, h.data_ptr<float>(), tails.data_ptr<float>(),
                                            cu.data_ptr<int>(), slots.data_ptr<int>(), D, taps);
    SM_CHECK_LAUNCH();
  }
  return out;
}
