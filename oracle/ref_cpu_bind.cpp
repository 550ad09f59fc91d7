// Registers the reference's two CPU operators on the quantized-linear path under
// this repository's own op namespace, so the checker can call the reference's
// unmodified CPU kernels (compiled from where they lie in the reference checkout)
// from Python:
//
//   torch.ops.oq_ref_cpu.matmul_packed_weight(out, x, packed, row_norms, centroids,
//                                             bias, has_bias, bits, N, K, bm, bn, bk)
//   torch.ops.oq_ref_cpu.quantize_activations_cpu(out, x, perm, signs, centroids,
//                                                 boundaries, eps, inv_sqrt_block, block)
//
// The functions themselves are declared by the reference's torch_binding.h
// (native-kernels/orbitquant-packed-matmul/torch-ext/torch_binding.h:11-37) and
// defined in orbitquant_packed_matmul_cpu/{packed_matmul_cpu,quantize_activations_cpu}.cpp.
// TEST INFRASTRUCTURE ONLY: the built library stays under oracle/_ref/.
#include <torch/csrc/stable/library.h>

#include "torch_binding.h"

STABLE_TORCH_LIBRARY(oq_ref_cpu, m) {
  m.def(
      "matmul_packed_weight(Tensor(a!) out, Tensor x, Tensor packed_weight_indices, Tensor row_norms, "
      "Tensor centroids, Tensor bias, bool has_bias, int bits, int out_features, int in_features, "
      "int block_m, int block_n, int block_k) -> ()");
  m.def(
      "quantize_activations_cpu(Tensor(a!) out, Tensor x, Tensor permutation, Tensor signs, "
      "Tensor centroids, Tensor boundaries, float eps, float inv_sqrt_block, int block_size) -> ()");
}

STABLE_TORCH_LIBRARY_IMPL(oq_ref_cpu, CPU, m) {
  m.impl("matmul_packed_weight", TORCH_BOX(&matmul_packed_weight));
  m.impl("quantize_activations_cpu", TORCH_BOX(&quantize_activations_cpu));
}
