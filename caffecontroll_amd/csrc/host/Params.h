// Plain structs standing in for the protobuf messages the reference's bridges read
// (src/parser/cnn.proto: LayerParameter, ConvolutionParameter, PoolingParameter, LRNParameter,
// DropoutParameter, InnerProductParameter, FillerParameter, SolverParameter).  Accessor names
// are kept so bridge code reads like the reference's; only the fields this path uses exist.
#pragma once
#include <cstdint>
#include <string>

namespace cct {
namespace cnn {

struct FillerParameter {
  std::string type_ = "constant";
  float value_ = 0.f, mean_ = 0.f, std_ = 1.f;
  const std::string &type() const { return type_; }
  float value() const { return value_; }
  float mean() const { return mean_; }
  float std() const { return std_; }
};

struct ConvolutionParameter {
  uint32_t num_output_ = 0, kernel_size_ = 0, stride_ = 1, pad_ = 0, group_ = 1;
  bool bias_term_ = true;
  FillerParameter weight_filler_, bias_filler_;
  uint32_t num_output() const { return num_output_; }
  uint32_t kernel_size() const { return kernel_size_; }
  uint32_t stride() const { return stride_; }
  uint32_t pad() const { return pad_; }
  uint32_t group() const { return group_; }
  bool bias_term() const { return bias_term_; }
  const FillerParameter &weight_filler() const { return weight_filler_; }
  const FillerParameter &bias_filler() const { return bias_filler_; }
};

struct InnerProductParameter {
  uint32_t num_output_ = 0;
  bool bias_term_ = true;
  FillerParameter weight_filler_, bias_filler_;
  uint32_t num_output() const { return num_output_; }
  bool bias_term() const { return bias_term_; }
  const FillerParameter &weight_filler() const { return weight_filler_; }
  const FillerParameter &bias_filler() const { return bias_filler_; }
};

struct PoolingParameter {
  uint32_t kernel_size_ = 0, stride_ = 1, pad_ = 0;
  uint32_t kernel_size() const { return kernel_size_; }
  uint32_t stride() const { return stride_; }
  uint32_t pad() const { return pad_; }
};

struct LRNParameter {
  uint32_t local_size_ = 5;
  float alpha_ = 1.f, beta_ = 0.75f;
  uint32_t local_size() const { return local_size_; }
  float alpha() const { return alpha_; }
  float beta() const { return beta_; }
};

struct DropoutParameter {
  float dropout_ratio_ = 0.5f;
  float dropout_ratio() const { return dropout_ratio_; }
};

struct LayerParameter {
  ConvolutionParameter convolution_param_;
  InnerProductParameter inner_product_param_;
  PoolingParameter pooling_param_;
  LRNParameter lrn_param_;
  DropoutParameter dropout_param_;
  // blobs_lr / weight_decay multipliers (cnn.proto blobs_lr, weight_decay): [0] weights, [1] bias
  float blobs_lr_[2] = {1.f, 1.f};
  float weight_decay_[2] = {1.f, 1.f};
  // device placement as in cnn.proto:249-256; 1.0 selects the (single) GPU partition
  float gpu_0_batch_proportion_ = 1.f;
  const ConvolutionParameter &convolution_param() const { return convolution_param_; }
  const InnerProductParameter &inner_product_param() const { return inner_product_param_; }
  const PoolingParameter &pooling_param() const { return pooling_param_; }
  const LRNParameter &lrn_param() const { return lrn_param_; }
  const DropoutParameter &dropout_param() const { return dropout_param_; }
  float blobs_lr(int i) const { return blobs_lr_[i]; }
  float weight_decay(int i) const { return weight_decay_[i]; }
  float gpu_0_batch_proportion() const { return gpu_0_batch_proportion_; }
};

struct SolverParameter {
  float base_lr_ = 0.01f, momentum_ = 0.f, gamma_ = 0.1f, power_ = 0.f, weight_decay_ = 0.f;
  int stepsize_ = 100000, max_iter_ = 0, random_seed_ = -1;
  std::string lr_policy_ = "fixed", regularization_type_ = "L2";
  float base_lr() const { return base_lr_; }
  float momentum() const { return momentum_; }
  float gamma() const { return gamma_; }
  float power() const { return power_; }
  float weight_decay() const { return weight_decay_; }
  int stepsize() const { return stepsize_; }
  int max_iter() const { return max_iter_; }
  int random_seed() const { return random_seed_; }
  const std::string &lr_policy() const { return lr_policy_; }
  const std::string &regularization_type() const { return regularization_type_; }
};

}  // namespace cnn
}  // namespace cct
