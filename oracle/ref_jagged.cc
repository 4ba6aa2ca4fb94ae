// TEST INFRASTRUCTURE, NOT PRODUCT CODE.
//
// C entry points over the reference's own jagged pooling loops, compiled in place from the
// reference tree (never copied): pytorch/py/jagged_ops.cc. Its only dependency outside the
// C++ standard library is PyTorch's C++ headers, which this image ships with its torch
// wheel. Built without -mavx2, i.e. the portable loops; the AVX2 specialisations do the same
// fp32 operations eight at a time. Used to check the plain-C restatement of the same loops.
#include "pytorch/py/jagged_ops.cc"

extern "C" {

void ref_jagged_sum_forward(const float* v, int64_t col, const int64_t* offsets, int64_t k,
                            float patch_value, float* out) {
  kraken::py::jagged::SumForwardImpl<float>(v, col, offsets, k, patch_value, out);
}

void ref_jagged_mean_forward(const float* v, int64_t col, const int64_t* offsets, int64_t k,
                             float patch_value, float* out) {
  kraken::py::jagged::MeanForwardImpl<float>(v, col, offsets, k, patch_value, out);
}

void ref_jagged_sum_backward(const int64_t* offsets, int64_t k, const float* grads, int64_t col,
                             float* vgrads) {
  kraken::py::jagged::SumBackwardImpl<float>(offsets, k, grads, col, vgrads);
}

void ref_jagged_mean_backward(const int64_t* offsets, int64_t k, const float* grads, int64_t col,
                              float* vgrads) {
  kraken::py::jagged::MeanBackwardImpl<float>(offsets, k, grads, col, vgrads);
}

}  // extern "C"
