// Tiled MFMA form of the sink attention for bf16 prompt portions.
#include <torch/extension.h>
#include <ATen/hip/HIPContext.h>
#include "seqmix_common.h"

bool sink_attention_mfma_fits(int dk, int vd, int G, int all_groups) { return false; }

torch::Tensor sink_attention_mfma(torch::Tensor q, torch::Tensor cache, int H, int G, int dk, int vd,
                                  torch::Tensor block_tables, int block_size, torch::Tensor positions,
                                  float scale, float softcap, const float* sink, int all_groups,
                                  torch::Tensor tiles, torch::Tensor part) {
  TORCH_CHECK(false, "sink_attention_mfma: not available");
  return part;
}
