#include <torch/extension.h>
#include "seqmix_common.h"
bool sigmoid_attention_mfma_fits(int dk, int vd) { return false; }
torch::Tensor sigmoid_attention_mfma(torch::Tensor q, torch::Tensor cache, int H, int G, int dk,
                                     int vd, torch::Tensor block_tables, int block_size,
                                     torch::Tensor positions, float scale, int window, int keep,
                                     torch::Tensor slopes, torch::Tensor pos_bias,
                                     torch::Tensor tiles) {
  TORCH_CHECK(false, "not built yet");
  return q;
}
