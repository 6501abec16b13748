// tiny_dnn_hip.h — host side of the MI355X hot path in the reference's own language.
//
// A thin, header-only C++14 mirror of the part of tiny-dnn's API that drives the training hot
// path, with the same names, argument meaning and error behaviour, sitting on the C ABI of
// libtdh.so (include/tdh.h). It is not a copy of tiny-dnn: no CPU kernels, no serialization,
// no graph networks — only what a program needs to switch this path to the GPU:
//
//   * vec_t / tensor_t / shape3d / padding / nn_error      (tiny_dnn/util/util.h, nn_error.h)
//   * core::backend_t with the added value `hip`           (tiny_dnn/core/backend.h:30)
//   * core::Params, conv_params, fully_params, maxpool_params, avepool_params (new)
//   * core::OpKernelConstruction / OpKernelContext / OpKernel
//                                                          (tiny_dnn/core/framework/op_kernel.h)
//   * Conv2dOp, Conv2dGradOp, FullyConnectedOp, FullyConnectedGradOp, MaxPoolOp, MaxPoolGradOp
//     and the new AvePoolOp / AvePoolGradOp, whose compute(OpKernelContext&) dispatch to libtdh
//   * gradient_descent / momentum / adam with the reference's members and update() signature
//   * network<sequential> with operator<<, fit<Loss>, train<Loss>, predict — the whole step stays
//     on the device (tdh_net_*)
//
// Per-operator calls take host tensors, as the OpKernelContext contract requires: compute()
// uploads its inputs, runs the kernels and downloads its outputs. Device residency across
// forward, backward and update is what network<sequential> provides.
//
// Differences from the reference that a caller can observe (all follow from the C ABI):
//   * the HIP engine takes UNPADDED convolution tensors (padding::same is applied in the
//     kernels), so input(0)/input_grad(0) of the conv ops are the layer's edge tensors;
//   * weight/bias gradients are produced reduced over the batch and ADDED into sample slot 0 of
//     the gradient tensor; the other slots are left untouched (zero after clear_grads), so
//     edge::merge_grads (tiny_dnn/node.h:89-103) sees the same sum.
#pragma once

#include <algorithm>
#include <cmath>
#include <cstddef>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <exception>
#include <fstream>
#include <iomanip>
#include <istream>
#include <limits>
#include <map>
#include <ostream>
#include <random>
#include <memory>
#include <string>
#include <vector>

#include "tdh.h"

namespace tiny_dnn {

typedef float float_t;                    // tiny_dnn/config.h:88-92
typedef std::vector<float_t> vec_t;       // tiny_dnn/util/util.h:64
typedef std::vector<vec_t> tensor_t;      // tiny_dnn/util/util.h:66
typedef size_t label_t;

// tiny_dnn/util/nn_error.h:19-26
class nn_error : public std::exception {
 public:
  explicit nn_error(const std::string &msg) : msg_(msg) {}
  const char *what() const throw() override { return msg_.c_str(); }

 private:
  std::string msg_;
};

enum class padding { valid, same };       // tiny_dnn/util/util.h:73-76

// tiny_dnn/util/util.h:149-182
template <typename T>
struct index3d {
  index3d() : width_(0), height_(0), depth_(0) {}
  index3d(T width, T height, T depth) : width_(width), height_(height), depth_(depth) {}
  T get_index(T x, T y, T channel) const { return (height_ * channel + y) * width_ + x; }
  T area() const { return width_ * height_; }
  T size() const { return width_ * height_ * depth_; }
  T width_, height_, depth_;
};
typedef index3d<size_t> shape3d;

namespace detail {

inline void check(int rc) {
  if (rc != TDH_OK) throw nn_error(std::string("tdh: ") + tdh_last_error());
}

// the library is initialised on first use, on device 0 unless tdh_init was called before
inline void ensure_init() {
  static bool done = false;
  if (!done) {
    check(tdh_init(0));
    done = true;
  }
}

// A device buffer holding the contiguous image of a host tensor_t ([sample][flat]).
class device_tensor {
 public:
  device_tensor() = default;
  device_tensor(const device_tensor &) = delete;
  device_tensor &operator=(const device_tensor &) = delete;
  ~device_tensor() {
    if (ptr_) tdh_free(ptr_);
  }
  float *resize(size_t floats) {
    if (floats > cap_) {
      if (ptr_) check(tdh_free(ptr_));
      ptr_ = nullptr;
      void *p = nullptr;
      check(tdh_malloc(&p, floats * sizeof(float)));
      ptr_ = static_cast<float *>(p);
      cap_ = floats;
    }
    return ptr_;
  }
  // rows [0, samples) of t, each `len` floats
  float *upload(const tensor_t &t, size_t samples, size_t len) {
    resize(samples * len);
    stage_.resize(samples * len);
    for (size_t s = 0; s < samples; ++s) {
      if (t[s].size() < len) throw nn_error("tensor row shorter than the layer shape");
      std::memcpy(stage_.data() + s * len, t[s].data(), len * sizeof(float));
    }
    if (samples * len > 0) check(tdh_memcpy_h2d(ptr_, stage_.data(), samples * len * sizeof(float)));
    return ptr_;
  }
  float *upload(const vec_t &v, size_t len) {
    resize(len);
    if (v.size() < len) throw nn_error("vector shorter than the layer shape");
    if (len) check(tdh_memcpy_h2d(ptr_, v.data(), len * sizeof(float)));
    return ptr_;
  }
  void download(tensor_t &t, size_t samples, size_t len) {
    stage_.resize(samples * len);
    if (samples * len > 0) check(tdh_memcpy_d2h(stage_.data(), ptr_, samples * len * sizeof(float)));
    for (size_t s = 0; s < samples; ++s) {
      if (t[s].size() < len) t[s].resize(len);
      std::memcpy(t[s].data(), stage_.data() + s * len, len * sizeof(float));
    }
  }
  // adds the device vector into `row` (the reference's `+=` into gradient slot 0)
  void download_add(vec_t &row, size_t len) {
    stage_.resize(len);
    if (len) check(tdh_memcpy_d2h(stage_.data(), ptr_, len * sizeof(float)));
    if (row.size() < len) row.resize(len);
    for (size_t i = 0; i < len; ++i) row[i] += stage_[i];
  }
  float *get() const { return ptr_; }

 private:
  float *ptr_  = nullptr;
  size_t cap_  = 0;
  std::vector<float> stage_;
};

}  // namespace detail

namespace core {

// tiny_dnn/core/backend.h:30, plus the engine this library adds
enum class backend_t { internal, nnpack, libdnn, avx, opencl, cblas, intel_mkl, hip };
inline backend_t default_engine() { return backend_t::hip; }

class conv_params;
class fully_params;
class maxpool_params;
class avepool_params;

// tiny_dnn/core/params/params.h:22-33
class Params {
 public:
  Params() {}
  conv_params &conv();
  fully_params &fully();
  maxpool_params &maxpool();
  avepool_params &avepool();
};

// tiny_dnn/core/params/conv_params.h:25-61
struct connection_table {
  connection_table() : rows_(0), cols_(0) {}
  connection_table(const bool *ar, size_t rows, size_t cols)
    : connected_(ar, ar + rows * cols), rows_(rows), cols_(cols) {}
  bool is_connected(size_t x, size_t y) const { return is_empty() ? true : connected_[y * cols_ + x]; }
  bool is_empty() const { return rows_ == 0 && cols_ == 0; }
  std::vector<bool> connected_;
  size_t rows_, cols_;
};

// tiny_dnn/core/params/conv_params.h:63-90
class conv_params : public Params {
 public:
  connection_table tbl;
  shape3d in, in_padded, out, weight;
  bool has_bias;
  padding pad_type;
  size_t w_stride, h_stride, w_dilation, h_dilation;
};
// tiny_dnn/core/params/fully_params.h:15-20
class fully_params : public Params {
 public:
  size_t in_size_, out_size_;
  bool has_bias_;
};
// tiny_dnn/core/params/maxpool_params.h:17-34 (out2inmax holds the argmax per sample)
class maxpool_params : public Params {
 public:
  shape3d in, out;
  size_t pool_size_x, pool_size_y, stride_x, stride_y;
  bool ceil_mode;
  padding pad_type;
  std::vector<std::vector<size_t>> out2inmax;
};
// new: the constructor arguments of average_pooling_layer
// (tiny_dnn/layers/average_pooling_layer.h:180-228)
class avepool_params : public Params {
 public:
  shape3d in, out;
  size_t pool_size_x, pool_size_y, stride_x, stride_y;
  bool ceil_mode;
  padding pad_type;
};

inline conv_params &Params::conv() { return *static_cast<conv_params *>(this); }
inline fully_params &Params::fully() { return *static_cast<fully_params *>(this); }
inline maxpool_params &Params::maxpool() { return *static_cast<maxpool_params *>(this); }
inline avepool_params &Params::avepool() { return *static_cast<avepool_params *>(this); }

class Device;  // the reference's OpenCL device registry has no counterpart here

// tiny_dnn/core/framework/op_kernel.h:22-37
class OpKernelConstruction {
 public:
  OpKernelConstruction() {}
  explicit OpKernelConstruction(Device *device, Params *params) : device_(device), params_(params) {}
  Device *device() const { return device_; }
  Params *params() const { return params_; }

 private:
  Device *device_ = nullptr;
  Params *params_ = nullptr;
};

// tiny_dnn/core/framework/op_kernel.h:39-127: borrows the caller's vectors of tensor pointers
class OpKernelContext {
 public:
  OpKernelContext() {}
  void set_in_out(const std::vector<tensor_t *> &in_data, std::vector<tensor_t *> &out_data) {
    in_data_  = const_cast<std::vector<tensor_t *> *>(&in_data);
    out_data_ = &out_data;
  }
  void set_in_out(const std::vector<tensor_t *> &in_data, const std::vector<tensor_t *> &out_data,
                  std::vector<tensor_t *> &out_grad, std::vector<tensor_t *> &in_grad) {
    in_data_  = const_cast<std::vector<tensor_t *> *>(&in_data);
    out_data_ = const_cast<std::vector<tensor_t *> *>(&out_data);
    out_grad_ = &out_grad;
    in_grad_  = &in_grad;
  }
  tensor_t &input(const int idx) { return *(*in_data_)[idx]; }
  tensor_t &output(const int idx) { return *(*out_data_)[idx]; }
  tensor_t &input_grad(const int idx) { return *(*in_grad_)[idx]; }
  tensor_t &output_grad(const int idx) { return *(*out_grad_)[idx]; }
  void setParams(Params *params) { params_ = params; }
  Params *params() const { return params_; }
  void setParallelize(const bool parallelize) { parallelize_ = parallelize; }
  bool parallelize() const { return parallelize_; }
  void setDevice(Device *device) { device_ = device; }
  Device *device() const { return device_; }
  backend_t engine() const { return engine_; }
  void setEngine(const backend_t engine) { engine_ = engine; }

 private:
  std::vector<tensor_t *> *in_data_ = nullptr, *out_data_ = nullptr, *out_grad_ = nullptr,
                          *in_grad_ = nullptr;
  Params *params_   = nullptr;
  Device *device_   = nullptr;
  bool parallelize_ = false;
  backend_t engine_ = default_engine();
};

// tiny_dnn/core/framework/op_kernel.h:129-142
class OpKernel {
 public:
  OpKernel() {}
  explicit OpKernel(const OpKernelConstruction &context)
    : device_(context.device()), params_(context.params()) {}
  virtual ~OpKernel() {}
  virtual void compute(OpKernelContext &context) = 0;

 protected:
  Device *device_ = nullptr;
  Params *params_ = nullptr;
};

}  // namespace core

namespace detail {

inline void require_hip(core::backend_t engine) {
  if (engine != core::backend_t::hip)
    throw nn_error("Not supported engine: " + std::to_string(static_cast<int>(engine)));
}

struct conv_desc_holder {
  tdh_conv_desc d;
  std::vector<uint8_t> tbl;
  explicit conv_desc_holder(const core::conv_params &p) {
    d.in_w = static_cast<int32_t>(p.in.width_); d.in_h = static_cast<int32_t>(p.in.height_);
    d.in_c = static_cast<int32_t>(p.in.depth_);
    d.k_w = static_cast<int32_t>(p.weight.width_); d.k_h = static_cast<int32_t>(p.weight.height_);
    d.out_c = static_cast<int32_t>(p.out.depth_);
    d.w_stride = static_cast<int32_t>(p.w_stride); d.h_stride = static_cast<int32_t>(p.h_stride);
    d.w_dilation = static_cast<int32_t>(p.w_dilation); d.h_dilation = static_cast<int32_t>(p.h_dilation);
    d.pad_same = p.pad_type == padding::same; d.has_bias = p.has_bias;
    d.tbl = nullptr;
    if (!p.tbl.is_empty()) {
      tbl.resize(p.tbl.rows_ * p.tbl.cols_);
      for (size_t i = 0; i < tbl.size(); ++i) tbl[i] = p.tbl.connected_[i];
      d.tbl = tbl.data();
    }
  }
};

template <typename P>
inline tdh_pool_desc pool_desc(const P &p) {
  tdh_pool_desc d;
  d.in_w = static_cast<int32_t>(p.in.width_); d.in_h = static_cast<int32_t>(p.in.height_);
  d.in_c = static_cast<int32_t>(p.in.depth_);
  d.pool_w = static_cast<int32_t>(p.pool_size_x); d.pool_h = static_cast<int32_t>(p.pool_size_y);
  d.stride_w = static_cast<int32_t>(p.stride_x); d.stride_h = static_cast<int32_t>(p.stride_y);
  d.pad_same = p.pad_type == padding::same; d.ceil_mode = p.ceil_mode;
  return d;
}

}  // namespace detail

// ---- operators: same class names and compute() contract as tiny_dnn/core/kernels/*_op.h ----

// tiny_dnn/core/kernels/conv2d_op.h:18-52
class Conv2dOp : public core::OpKernel {
 public:
  explicit Conv2dOp(const core::OpKernelConstruction &context) : core::OpKernel(context) {}
  void compute(core::OpKernelContext &context) override {
    detail::require_hip(context.engine());
    detail::ensure_init();
    auto &params = OpKernel::params_->conv();
    detail::conv_desc_holder h(params);
    const tensor_t &in = context.input(0);
    const tensor_t &W  = context.input(1);
    tensor_t &out      = context.output(0);
    const size_t n = in.size();
    float *bias = params.has_bias ? b_.upload(context.input(2)[0], params.out.depth_) : nullptr;
    y_.resize(n * params.out.size());
    detail::check(tdh_conv2d_fwd(&h.d, static_cast<int>(n), x_.upload(in, n, params.in.size()),
                                 w_.upload(W[0], params.weight.size()), bias, y_.get()));
    y_.download(out, n, params.out.size());
  }

 private:
  detail::device_tensor x_, w_, b_, y_;
};

// tiny_dnn/core/kernels/conv2d_grad_op.h:17-51
class Conv2dGradOp : public core::OpKernel {
 public:
  explicit Conv2dGradOp(const core::OpKernelConstruction &context) : core::OpKernel(context) {}
  void compute(core::OpKernelContext &context) override {
    detail::require_hip(context.engine());
    detail::ensure_init();
    auto &params = OpKernel::params_->conv();
    detail::conv_desc_holder h(params);
    const tensor_t &prev_out = context.input(0);
    const tensor_t &W        = context.input(1);
    tensor_t &dW             = context.input_grad(1);
    tensor_t &prev_delta     = context.input_grad(0);
    tensor_t &curr_delta     = context.output_grad(0);
    const size_t n = prev_out.size();
    dx_.resize(n * params.in.size());
    dw_.resize(params.weight.size());
    db_.resize(params.out.depth_);
    detail::check(tdh_conv2d_bwd(&h.d, static_cast<int>(n),
                                 x_.upload(prev_out, n, params.in.size()),
                                 w_.upload(W[0], params.weight.size()),
                                 dy_.upload(curr_delta, n, params.out.size()), dx_.get(), dw_.get(),
                                 params.has_bias ? db_.get() : nullptr, /*accumulate=*/0));
    dx_.download(prev_delta, n, params.in.size());   // dX is overwritten (conv2d_grad_op.h:34)
    dw_.download_add(dW[0], params.weight.size());   // dW, db accumulate
    if (params.has_bias) db_.download_add(context.input_grad(2)[0], params.out.depth_);
  }

 private:
  detail::device_tensor x_, w_, dy_, dx_, dw_, db_;
};

// tiny_dnn/core/kernels/fully_connected_op.h:20-65
class FullyConnectedOp : public core::OpKernel {
 public:
  explicit FullyConnectedOp(const core::OpKernelConstruction &context) : core::OpKernel(context) {}
  void compute(core::OpKernelContext &context) override {
    detail::require_hip(context.engine());
    detail::ensure_init();
    auto &params = OpKernel::params_->fully();
    const tensor_t &in = context.input(0);
    const size_t n = in.size();
    float *bias = params.has_bias_ ? b_.upload(context.input(2)[0], params.out_size_) : nullptr;
    y_.resize(n * params.out_size_);
    detail::check(tdh_fc_fwd(static_cast<int>(params.in_size_), static_cast<int>(params.out_size_),
                             params.has_bias_, static_cast<int>(n),
                             x_.upload(in, n, params.in_size_),
                             w_.upload(context.input(1)[0], params.in_size_ * params.out_size_), bias,
                             y_.get()));
    y_.download(context.output(0), n, params.out_size_);
  }

 private:
  detail::device_tensor x_, w_, b_, y_;
};

// tiny_dnn/core/kernels/fully_connected_grad_op.h:17-53
class FullyConnectedGradOp : public core::OpKernel {
 public:
  explicit FullyConnectedGradOp(const core::OpKernelConstruction &context) : core::OpKernel(context) {}
  void compute(core::OpKernelContext &context) override {
    detail::require_hip(context.engine());
    detail::ensure_init();
    auto &params = OpKernel::params_->fully();
    const tensor_t &prev_out = context.input(0);
    const size_t n = prev_out.size(), in = params.in_size_, out = params.out_size_;
    dx_.resize(n * in);
    dw_.resize(in * out);
    db_.resize(out);
    detail::check(tdh_fc_bwd(static_cast<int>(in), static_cast<int>(out), params.has_bias_,
                             static_cast<int>(n), x_.upload(prev_out, n, in),
                             w_.upload(context.input(1)[0], in * out),
                             dy_.upload(context.output_grad(0), n, out), dx_.get(), dw_.get(),
                             params.has_bias_ ? db_.get() : nullptr, 0));
    dx_.download(context.input_grad(0), n, in);
    dw_.download_add(context.input_grad(1)[0], in * out);
    if (params.has_bias_) db_.download_add(context.input_grad(2)[0], out);
  }

 private:
  detail::device_tensor x_, w_, dy_, dx_, dw_, db_;
};

// tiny_dnn/core/kernels/maxpool_op.h:18-63; params.out2inmax receives the argmax indices
class MaxPoolOp : public core::OpKernel {
 public:
  explicit MaxPoolOp(const core::OpKernelConstruction &context) : core::OpKernel(context) {}
  void compute(core::OpKernelContext &context) override {
    detail::require_hip(context.engine());
    detail::ensure_init();
    auto &params = OpKernel::params_->maxpool();
    const tdh_pool_desc d = detail::pool_desc(params);
    const tensor_t &in = context.input(0);
    const size_t n = in.size(), osz = params.out.size();
    y_.resize(n * osz);
    idx_.resize(n * osz);
    detail::check(tdh_maxpool_fwd(&d, static_cast<int>(n), x_.upload(in, n, params.in.size()),
                                  y_.get(), reinterpret_cast<int32_t *>(idx_.get())));
    y_.download(context.output(0), n, osz);
    std::vector<int32_t> host(n * osz);
    if (n * osz > 0) detail::check(tdh_memcpy_d2h(host.data(), idx_.get(), host.size() * sizeof(int32_t)));
    params.out2inmax.resize(n);
    for (size_t s = 0; s < n; ++s) params.out2inmax[s].assign(host.begin() + s * osz, host.begin() + (s + 1) * osz);
  }

 private:
  detail::device_tensor x_, y_, idx_;
};

// tiny_dnn/core/kernels/maxpool_grad_op.h:17-47
class MaxPoolGradOp : public core::OpKernel {
 public:
  explicit MaxPoolGradOp(const core::OpKernelConstruction &context) : core::OpKernel(context) {}
  void compute(core::OpKernelContext &context) override {
    detail::require_hip(context.engine());
    detail::ensure_init();
    auto &params = OpKernel::params_->maxpool();
    const tdh_pool_desc d = detail::pool_desc(params);
    tensor_t &prev_delta = context.input_grad(0);
    const tensor_t &curr_delta = context.output_grad(0);
    const size_t n = curr_delta.size(), osz = params.out.size();
    if (params.out2inmax.size() < n) throw nn_error("max-pool backward without a recorded forward pass");
    std::vector<int32_t> host(n * osz);
    for (size_t s = 0; s < n; ++s)
      for (size_t i = 0; i < osz; ++i) host[s * osz + i] = static_cast<int32_t>(params.out2inmax[s][i]);
    idx_.resize(n * osz);
    if (n * osz > 0) detail::check(tdh_memcpy_h2d(idx_.get(), host.data(), host.size() * sizeof(int32_t)));
    dx_.resize(n * params.in.size());
    detail::check(tdh_maxpool_bwd(&d, static_cast<int>(n), dy_.upload(curr_delta, n, osz),
                                  reinterpret_cast<const int32_t *>(idx_.get()), dx_.get()));
    dx_.download(prev_delta, n, params.in.size());
  }

 private:
  detail::device_tensor dy_, dx_, idx_;
};

// new operators with MaxPool's contract for tiny_average_pooling_kernel / _back_kernel
// (tiny_dnn/layers/average_pooling_layer.h:25-106): input(0)=X, input(1)=W, input(2)=b
class AvePoolOp : public core::OpKernel {
 public:
  explicit AvePoolOp(const core::OpKernelConstruction &context) : core::OpKernel(context) {}
  void compute(core::OpKernelContext &context) override {
    detail::require_hip(context.engine());
    detail::ensure_init();
    auto &params = OpKernel::params_->avepool();
    const tdh_pool_desc d = detail::pool_desc(params);
    const tensor_t &in = context.input(0);
    const size_t n = in.size(), c = params.in.depth_;
    y_.resize(n * params.out.size());
    detail::check(tdh_avepool_fwd(&d, static_cast<int>(n), x_.upload(in, n, params.in.size()),
                                  w_.upload(context.input(1)[0], c), b_.upload(context.input(2)[0], c),
                                  y_.get()));
    y_.download(context.output(0), n, params.out.size());
  }

 private:
  detail::device_tensor x_, w_, b_, y_;
};

class AvePoolGradOp : public core::OpKernel {
 public:
  explicit AvePoolGradOp(const core::OpKernelConstruction &context) : core::OpKernel(context) {}
  void compute(core::OpKernelContext &context) override {
    detail::require_hip(context.engine());
    detail::ensure_init();
    auto &params = OpKernel::params_->avepool();
    const tdh_pool_desc d = detail::pool_desc(params);
    const tensor_t &prev_out = context.input(0);
    const size_t n = prev_out.size(), c = params.in.depth_;
    dx_.resize(n * params.in.size());
    dw_.resize(c);
    db_.resize(c);
    detail::check(tdh_avepool_bwd(&d, static_cast<int>(n), x_.upload(prev_out, n, params.in.size()),
                                  w_.upload(context.input(1)[0], c),
                                  dy_.upload(context.output_grad(0), n, params.out.size()), dx_.get(),
                                  dw_.get(), db_.get(), 0));
    dx_.download(context.input_grad(0), n, params.in.size());
    dw_.download_add(context.input_grad(1)[0], c);
    db_.download_add(context.input_grad(2)[0], c);
  }

 private:
  detail::device_tensor x_, w_, dy_, dx_, dw_, db_;
};

// ---- loss functions (type tags; tiny_dnn/lossfunctions/loss_function.h) ----
struct mse { static const int kind = TDH_LOSS_MSE; };
struct cross_entropy { static const int kind = TDH_LOSS_CE; };
struct cross_entropy_multiclass { static const int kind = TDH_LOSS_CE_MULTICLASS; };

// ---- optimizers: the reference's members and update(dW, W, parallelize) signature
// (tiny_dnn/optimizers/optimizer.h). State vectors live on the device, keyed by &W like the
// reference's unordered_map (optimizer.h:35-48). ----
struct optimizer {
  virtual ~optimizer() {}
  virtual void update(const vec_t &dW, vec_t &W, bool parallelize) = 0;
  virtual void reset() {}
  virtual tdh_opt descriptor() const = 0;       // hyper-parameters + running powers
  virtual void absorb(const tdh_opt &) {}        // takes the advanced powers back
};

namespace detail {
struct device_optimizer : public optimizer {
  void update(const vec_t &dW, vec_t &W, bool /*parallelize*/) override {
    ensure_init();
    tdh_opt o = descriptor();
    state &st = states_[&W];
    const size_t n = W.size();
    if (st.n != n) {
      st.s0.resize(n); st.s1.resize(n); st.n = n;
      if (n) { check(tdh_fill_zero(st.s0.get(), n * sizeof(float))); check(tdh_fill_zero(st.s1.get(), n * sizeof(float))); }
    }
    float *g = g_.upload(dW, n), *w = w_.upload(W, n);
    check(tdh_opt_update(&o, n, g, 1.0f, w, st.s0.get(), st.s1.get()));
    if (n) check(tdh_memcpy_d2h(W.data(), w, n * sizeof(float)));
    absorb(o);
  }
  void reset() override { states_.clear(); }

 private:
  struct state {
    device_tensor s0, s1;
    size_t n = 0;
  };
  std::map<const vec_t *, state> states_;
  device_tensor g_, w_;
};
}  // namespace detail

// tiny_dnn/optimizers/optimizer.h:182-192
struct gradient_descent : public detail::device_optimizer {
  gradient_descent() : alpha(float_t(0.01)), lambda(float_t(0)) {}
  tdh_opt descriptor() const override {
    tdh_opt o; tdh_opt_default(&o, TDH_OPT_SGD); o.alpha = alpha; o.lambda = lambda; return o;
  }
  float_t alpha, lambda;
};
// tiny_dnn/optimizers/optimizer.h:201-218
struct momentum : public detail::device_optimizer {
  momentum() : alpha(float_t(0.01)), lambda(float_t(0)), mu(float_t(0.9)) {}
  tdh_opt descriptor() const override {
    tdh_opt o; tdh_opt_default(&o, TDH_OPT_MOMENTUM); o.alpha = alpha; o.lambda = lambda; o.mu = mu; return o;
  }
  float_t alpha, lambda, mu;
};
// tiny_dnn/optimizers/optimizer.h:103-137 (b1_t, b2_t advance once per update() call)
struct adam : public detail::device_optimizer {
  adam() : alpha(float_t(0.001)), b1(float_t(0.9)), b2(float_t(0.999)), b1_t(float_t(0.9)), b2_t(float_t(0.999)) {}
  tdh_opt descriptor() const override {
    tdh_opt o; tdh_opt_default(&o, TDH_OPT_ADAM);
    o.alpha = alpha; o.b1 = b1; o.b2 = b2; o.b1_t = b1_t; o.b2_t = b2_t; return o;
  }
  void absorb(const tdh_opt &o) override { b1_t = o.b1_t; b2_t = o.b2_t; }
  float_t alpha, b1, b2, b1_t, b2_t;
};

// tiny_dnn/optimizers/optimizer.h:57-71
struct adagrad : public detail::device_optimizer {
  adagrad() : alpha(float_t(0.01)) {}
  tdh_opt descriptor() const override {
    tdh_opt o; tdh_opt_default(&o, TDH_OPT_ADAGRAD); o.alpha = alpha; return o;
  }
  float_t alpha;
};
// tiny_dnn/optimizers/optimizer.h:79-95
struct RMSprop : public detail::device_optimizer {
  RMSprop() : alpha(float_t(0.0001)), mu(float_t(0.99)) {}
  tdh_opt descriptor() const override {
    tdh_opt o; tdh_opt_default(&o, TDH_OPT_RMSPROP); o.alpha = alpha; o.mu = mu; return o;
  }
  float_t alpha, mu;
};
// tiny_dnn/optimizers/optimizer.h:145-175 (only b1_t advances)
struct adamax : public detail::device_optimizer {
  adamax() : alpha(float_t(0.002)), b1(float_t(0.9)), b2(float_t(0.999)), b1_t(b1) {}
  tdh_opt descriptor() const override {
    tdh_opt o; tdh_opt_default(&o, TDH_OPT_ADAMAX);
    o.alpha = alpha; o.b1 = b1; o.b2 = b2; o.b1_t = b1_t; return o;
  }
  void absorb(const tdh_opt &o) override { b1_t = o.b1_t; }
  float_t alpha, b1, b2, b1_t;
};
// tiny_dnn/optimizers/optimizer.h:227-245
struct nesterov_momentum : public detail::device_optimizer {
  nesterov_momentum() : alpha(float_t(0.01)), lambda(float_t(0)), mu(float_t(0.9)) {}
  tdh_opt descriptor() const override {
    tdh_opt o; tdh_opt_default(&o, TDH_OPT_NESTEROV); o.alpha = alpha; o.lambda = lambda; o.mu = mu; return o;
  }
  float_t alpha, lambda, mu;
};

// ---- layers: constructor arguments as in tiny_dnn/layers/*.h; they only describe the layer,
// network<sequential> turns the descriptions into one device-resident tdh_net ----
struct layer_desc {
  tdh_layer l;
  std::vector<uint8_t> tbl;
};

class layer {
 public:
  virtual ~layer() {}
  virtual layer_desc describe(const shape3d &prev_out) const = 0;
  virtual std::string layer_type() const = 0;
};

// tiny_dnn/layers/convolutional_layer.h:64-100
class convolutional_layer : public layer {
 public:
  convolutional_layer(size_t in_width, size_t in_height, size_t window_size, size_t in_channels,
                      size_t out_channels, padding pad_type = padding::valid, bool has_bias = true,
                      size_t w_stride = 1, size_t h_stride = 1, size_t w_dilation = 1,
                      size_t h_dilation = 1, core::backend_t backend_type = core::default_engine())
    : convolutional_layer(in_width, in_height, window_size, window_size, in_channels, out_channels,
                          core::connection_table(), pad_type, has_bias, w_stride, h_stride,
                          w_dilation, h_dilation, backend_type) {}
  convolutional_layer(size_t in_width, size_t in_height, size_t window_width, size_t window_height,
                      size_t in_channels, size_t out_channels,
                      const core::connection_table &connection_table,
                      padding pad_type = padding::valid, bool has_bias = true, size_t w_stride = 1,
                      size_t h_stride = 1, size_t w_dilation = 1, size_t h_dilation = 1,
                      core::backend_t backend_type = core::default_engine()) {
    detail::require_hip(backend_type);
    params_.in = shape3d(in_width, in_height, in_channels);
    params_.weight = shape3d(window_width, window_height, in_channels * out_channels);
    params_.has_bias = has_bias; params_.pad_type = pad_type;
    params_.w_stride = w_stride; params_.h_stride = h_stride;
    params_.w_dilation = w_dilation; params_.h_dilation = h_dilation;
    params_.tbl = connection_table;
    detail::conv_desc_holder h(with_out(out_channels));
    params_.out = shape3d(tdh_conv_out_w(&h.d), tdh_conv_out_h(&h.d), out_channels);
    params_.in_padded = pad_type == padding::same
                          ? shape3d(in_width + window_width - 1, in_height + window_height - 1, in_channels)
                          : params_.in;
    kernel_fwd_.reset(new Conv2dOp(core::OpKernelConstruction(nullptr, &params_)));
    kernel_back_.reset(new Conv2dGradOp(core::OpKernelConstruction(nullptr, &params_)));
  }
  std::string layer_type() const override { return "conv"; }
  std::vector<shape3d> in_shape() const {
    return {params_.in, shape3d(params_.weight.width_, params_.weight.height_, params_.weight.depth_),
            shape3d(1, 1, params_.out.depth_)};
  }
  std::vector<shape3d> out_shape() const { return {params_.out}; }
  // layer::forward_propagation / back_propagation (convolutional_layer.h:283-337) on the HIP
  // engine: the unpadded edge tensors go straight to the operators
  void forward_propagation(const std::vector<tensor_t *> &in_data, std::vector<tensor_t *> &out_data) {
    core::OpKernelContext ctx;
    ctx.set_in_out(in_data, out_data);
    ctx.setEngine(core::backend_t::hip);
    kernel_fwd_->compute(ctx);
  }
  void back_propagation(const std::vector<tensor_t *> &in_data, const std::vector<tensor_t *> &out_data,
                        std::vector<tensor_t *> &out_grad, std::vector<tensor_t *> &in_grad) {
    core::OpKernelContext ctx;
    ctx.set_in_out(in_data, out_data, out_grad, in_grad);
    ctx.setParams(&params_);
    ctx.setEngine(core::backend_t::hip);
    kernel_back_->compute(ctx);
  }
  layer_desc describe(const shape3d &) const override {
    layer_desc r;
    detail::conv_desc_holder h(params_);
    std::memset(&r.l, 0, sizeof(r.l));
    r.l.kind = TDH_L_CONV;
    r.l.conv = h.d;
    r.tbl    = h.tbl;
    return r;
  }
  const core::conv_params &params() const { return params_; }

 private:
  core::conv_params with_out(size_t out_channels) {
    core::conv_params p = params_;
    p.out = shape3d(0, 0, out_channels);
    return p;
  }
  core::conv_params params_;
  std::shared_ptr<core::OpKernel> kernel_fwd_, kernel_back_;
};

// tiny_dnn/layers/fully_connected_layer.h:32-41
class fully_connected_layer : public layer {
 public:
  fully_connected_layer(size_t in_dim, size_t out_dim, bool has_bias = true,
                        core::backend_t backend_type = core::default_engine()) {
    detail::require_hip(backend_type);
    params_.in_size_ = in_dim; params_.out_size_ = out_dim; params_.has_bias_ = has_bias;
    kernel_fwd_.reset(new FullyConnectedOp(core::OpKernelConstruction(nullptr, &params_)));
    kernel_back_.reset(new FullyConnectedGradOp(core::OpKernelConstruction(nullptr, &params_)));
  }
  std::string layer_type() const override { return "fully-connected"; }
  void forward_propagation(const std::vector<tensor_t *> &in_data, std::vector<tensor_t *> &out_data) {
    core::OpKernelContext ctx;
    ctx.set_in_out(in_data, out_data);
    ctx.setEngine(core::backend_t::hip);
    kernel_fwd_->compute(ctx);
  }
  void back_propagation(const std::vector<tensor_t *> &in_data, const std::vector<tensor_t *> &out_data,
                        std::vector<tensor_t *> &out_grad, std::vector<tensor_t *> &in_grad) {
    core::OpKernelContext ctx;
    ctx.set_in_out(in_data, out_data, out_grad, in_grad);
    ctx.setEngine(core::backend_t::hip);
    kernel_back_->compute(ctx);
  }
  layer_desc describe(const shape3d &) const override {
    layer_desc r;
    std::memset(&r.l, 0, sizeof(r.l));
    r.l.kind = TDH_L_FC;
    r.l.fc_in = static_cast<int32_t>(params_.in_size_);
    r.l.fc_out = static_cast<int32_t>(params_.out_size_);
    r.l.fc_bias = params_.has_bias_;
    return r;
  }

 private:
  core::fully_params params_;
  std::shared_ptr<core::OpKernel> kernel_fwd_, kernel_back_;
};

namespace detail {
template <typename P>
inline void set_pool_params(P &p, size_t in_width, size_t in_height, size_t in_channels, size_t px,
                            size_t py, size_t sx, size_t sy, bool ceil_mode, padding pad_type) {
  p.in = shape3d(in_width, in_height, in_channels);
  p.pool_size_x = px; p.pool_size_y = py; p.stride_x = sx; p.stride_y = sy;
  p.ceil_mode = ceil_mode; p.pad_type = pad_type;
  const tdh_pool_desc d = pool_desc(p);
  p.out = shape3d(tdh_pool_out_w(&d), tdh_pool_out_h(&d), in_channels);
}
}  // namespace detail

// tiny_dnn/layers/max_pooling_layer.h:40-118
class max_pooling_layer : public layer {
 public:
  max_pooling_layer(size_t in_width, size_t in_height, size_t in_channels, size_t pooling_size,
                    bool ceil_mode = false, core::backend_t backend_type = core::default_engine())
    : max_pooling_layer(in_width, in_height, in_channels, pooling_size,
                        (in_height == 1 ? 1 : pooling_size), pooling_size, pooling_size, ceil_mode,
                        padding::valid, backend_type) {}
  max_pooling_layer(size_t in_width, size_t in_height, size_t in_channels, size_t pooling_size_x,
                    size_t pooling_size_y, size_t stride_x, size_t stride_y, bool ceil_mode = false,
                    padding pad_type = padding::valid,
                    core::backend_t backend_type = core::default_engine()) {
    detail::require_hip(backend_type);
    detail::set_pool_params(params_, in_width, in_height, in_channels, pooling_size_x,
                            pooling_size_y, stride_x, stride_y, ceil_mode, pad_type);
    kernel_fwd_.reset(new MaxPoolOp(core::OpKernelConstruction(nullptr, &params_)));
    kernel_back_.reset(new MaxPoolGradOp(core::OpKernelConstruction(nullptr, &params_)));
  }
  std::string layer_type() const override { return "max-pool"; }
  std::vector<shape3d> out_shape() const { return {params_.out}; }
  void forward_propagation(const std::vector<tensor_t *> &in_data, std::vector<tensor_t *> &out_data) {
    core::OpKernelContext ctx;
    ctx.set_in_out(in_data, out_data);
    ctx.setEngine(core::backend_t::hip);
    kernel_fwd_->compute(ctx);
  }
  void back_propagation(const std::vector<tensor_t *> &in_data, const std::vector<tensor_t *> &out_data,
                        std::vector<tensor_t *> &out_grad, std::vector<tensor_t *> &in_grad) {
    core::OpKernelContext ctx;
    ctx.set_in_out(in_data, out_data, out_grad, in_grad);
    ctx.setEngine(core::backend_t::hip);
    kernel_back_->compute(ctx);
  }
  layer_desc describe(const shape3d &) const override {
    layer_desc r;
    std::memset(&r.l, 0, sizeof(r.l));
    r.l.kind = TDH_L_MAXPOOL;
    r.l.pool = detail::pool_desc(params_);
    return r;
  }

 private:
  core::maxpool_params params_;
  std::shared_ptr<core::OpKernel> kernel_fwd_, kernel_back_;
};

// tiny_dnn/layers/average_pooling_layer.h:123-228; throws like the reference when the input is
// not a multiple of the window (:216-218)
class average_pooling_layer : public layer {
 public:
  average_pooling_layer(size_t in_width, size_t in_height, size_t in_channels, size_t pool_size,
                        bool ceil_mode = false)
    : average_pooling_layer(in_width, in_height, in_channels, pool_size,
                            (in_height == 1 ? 1 : pool_size), pool_size, pool_size, ceil_mode,
                            padding::valid) {}
  average_pooling_layer(size_t in_width, size_t in_height, size_t in_channels, size_t pool_size_x,
                        size_t pool_size_y, size_t stride_x, size_t stride_y, bool ceil_mode = false,
                        padding pad_type = padding::valid) {
    if ((in_width % pool_size_x) || (in_height % pool_size_y))
      throw nn_error("width/height not multiples of pooling size");
    detail::set_pool_params(params_, in_width, in_height, in_channels, pool_size_x, pool_size_y,
                            stride_x, stride_y, ceil_mode, pad_type);
    kernel_fwd_.reset(new AvePoolOp(core::OpKernelConstruction(nullptr, &params_)));
    kernel_back_.reset(new AvePoolGradOp(core::OpKernelConstruction(nullptr, &params_)));
  }
  std::string layer_type() const override { return "ave-pool"; }
  std::vector<shape3d> out_shape() const { return {params_.out}; }
  void forward_propagation(const std::vector<tensor_t *> &in_data, std::vector<tensor_t *> &out_data) {
    core::OpKernelContext ctx;
    ctx.set_in_out(in_data, out_data);
    ctx.setEngine(core::backend_t::hip);
    kernel_fwd_->compute(ctx);
  }
  void back_propagation(const std::vector<tensor_t *> &in_data, const std::vector<tensor_t *> &out_data,
                        std::vector<tensor_t *> &out_grad, std::vector<tensor_t *> &in_grad) {
    core::OpKernelContext ctx;
    ctx.set_in_out(in_data, out_data, out_grad, in_grad);
    ctx.setEngine(core::backend_t::hip);
    kernel_back_->compute(ctx);
  }
  layer_desc describe(const shape3d &) const override {
    layer_desc r;
    std::memset(&r.l, 0, sizeof(r.l));
    r.l.kind = TDH_L_AVEPOOL;
    r.l.pool = detail::pool_desc(params_);
    return r;
  }

 private:
  core::avepool_params params_;
  std::shared_ptr<core::OpKernel> kernel_fwd_, kernel_back_;
};

// activation layers (tiny_dnn/activations/*.h): shape is inherited from the previous layer;
// forward_activation / backward_activation keep the reference's signatures
// (activation_layer.h:93-112) on single samples
class activation_layer : public layer {
 public:
  std::string layer_type() const override { return type_; }
  layer_desc describe(const shape3d &) const override {
    layer_desc r;
    std::memset(&r.l, 0, sizeof(r.l));
    r.l.kind     = TDH_L_ACT;
    r.l.act      = kind_;
    r.l.act_p[0] = p_[0];
    r.l.act_p[1] = p_[1];
    return r;
  }
  void forward_activation(const vec_t &x, vec_t &y) {
    detail::ensure_init();
    const int n = static_cast<int>(x.size());
    y.resize(x.size());
    buffers &s = scratch();
    s.b.resize(x.size());
    detail::check(tdh_act_fwd_p(kind_, p_, 1, n, s.a.upload(x, x.size()), s.b.get()));
    if (n) detail::check(tdh_memcpy_d2h(y.data(), s.b.get(), x.size() * sizeof(float)));
  }
  void backward_activation(const vec_t &x, const vec_t &y, vec_t &dx, const vec_t &dy) {
    detail::ensure_init();
    const int n = static_cast<int>(y.size());
    dx.resize(y.size());
    buffers &s = scratch();
    s.d.resize(y.size());
    detail::check(tdh_act_bwd_p(kind_, p_, 1, n, s.a.upload(x, x.size()), s.b.upload(y, y.size()),
                                s.c.upload(dy, dy.size()), s.d.get()));
    if (n) detail::check(tdh_memcpy_d2h(dx.data(), s.d.get(), y.size() * sizeof(float)));
  }

 protected:
  activation_layer(int kind, const char *type, float p0 = 0.f, float p1 = 0.f)
    : kind_(kind), type_(type) {
    p_[0] = p0;
    p_[1] = p1;
  }
  int kind_;
  const char *type_;
  float p_[2];

 private:
  struct buffers {
    detail::device_tensor a, b, c, d;
  };
  buffers &scratch() {
    if (!buf_) buf_.reset(new buffers());
    return *buf_;
  }
  std::shared_ptr<buffers> buf_;  // copies of a layer share their device scratch, like the ops
};
struct tanh_layer : activation_layer { tanh_layer() : activation_layer(TDH_ACT_TANH, "tanh-activation") {} };
struct relu_layer : activation_layer { relu_layer() : activation_layer(TDH_ACT_RELU, "relu-activation") {} };
struct softmax_layer : activation_layer { softmax_layer() : activation_layer(TDH_ACT_SOFTMAX, "softmax-activation") {} };
struct sigmoid_layer : activation_layer { sigmoid_layer() : activation_layer(TDH_ACT_SIGMOID, "sigmoid-activation") {} };
// leaky_relu_layer.h:25, elu_layer.h:18, selu_layer.h:26-27, softplus_layer.h:26-27
struct leaky_relu_layer : activation_layer {
  explicit leaky_relu_layer(const float_t epsilon = float_t(0.01))
    : activation_layer(TDH_ACT_LEAKY_RELU, "leaky-relu-activation", epsilon) {}
  float_t epsilon_value() const { return p_[0]; }
};
struct elu_layer : activation_layer {
  explicit elu_layer(const float_t alpha = float_t(1.0)) : activation_layer(TDH_ACT_ELU, "elu-activation", alpha) {}
};
struct selu_layer : activation_layer {
  explicit selu_layer(const float_t lambda = float_t(1.05070), const float_t alpha = float_t(1.67326))
    : activation_layer(TDH_ACT_SELU, "selu-activation", lambda, alpha) {}
};
struct softplus_layer : activation_layer {
  explicit softplus_layer(const float_t beta = float_t(1.0), const float_t threshold = float_t(20.0))
    : activation_layer(TDH_ACT_SOFTPLUS, "softplus-activation", beta, threshold) {}
};
struct softsign_layer : activation_layer { softsign_layer() : activation_layer(TDH_ACT_SOFTSIGN, "softsign-activation") {} };
struct asinh_layer : activation_layer { asinh_layer() : activation_layer(TDH_ACT_ASINH, "asinh-activation") {} };
struct tanh_p1m2_layer : activation_layer { tanh_p1m2_layer() : activation_layer(TDH_ACT_TANH_P1M2, "tanh-scaled-activation") {} };

// ---- the reference's random source (tiny_dnn/util/random.h:19-69): one std::mt19937 for the
// whole process, seeded with 1 until set_random_seed is called; bernoulli(p) is one draw of
// uniform_real_distribution<float_t>(0, 1) compared with p ----
class random_generator {
 public:
  static random_generator &get_instance() {
    static random_generator g;
    return g;
  }
  std::mt19937 &operator()() { return engine_; }
  void set_seed(unsigned int seed) { engine_.seed(seed); }

 private:
  random_generator() : engine_(1) {}
  std::mt19937 engine_;
};
inline void set_random_seed(unsigned int seed) { random_generator::get_instance().set_seed(seed); }
inline bool bernoulli(float_t p) {
  std::uniform_real_distribution<float_t> unit(float_t(0), float_t(1));
  return unit(random_generator::get_instance()()) <= p;
}

enum class net_phase { train, test };  // tiny_dnn/util/util.h:71

// The two layers below run on the device through their own operators. The device-resident
// train step of network<sequential> does not include them (describe() says so); they are used
// the way the reference's tests use a single layer: forward_propagation / back_propagation on
// host tensors.
namespace detail {
struct norm_buffers {
  device_tensor x, y, dy, dx, mean, var, stddev, mean_cur, var_cur;
  void *mask     = nullptr;
  size_t mask_cap = 0;
  ~norm_buffers() {
    if (mask) tdh_free(mask);
  }
  void *mask_upload(const std::vector<uint8_t> &m) {
    if (m.size() > mask_cap) {
      if (mask) check(tdh_free(mask));
      mask = nullptr;
      check(tdh_malloc(&mask, m.size()));
      mask_cap = m.size();
    }
    if (!m.empty()) check(tdh_memcpy_h2d(mask, m.data(), m.size()));
    return mask;
  }
};
inline void download_vec(vec_t &v, const float *dev, size_t n) {
  v.resize(n);
  if (n) check(tdh_memcpy_d2h(v.data(), dev, n * sizeof(float)));
}
}  // namespace detail

// tiny_dnn/layers/batch_normalization_layer.h:54-72 (the constructor that takes the shape)
class batch_normalization_layer : public layer {
 public:
  batch_normalization_layer(size_t in_spatial_size, size_t in_channels, float_t epsilon = 1e-5,
                            float_t momentum = 0.999, net_phase phase = net_phase::train)
    : channels_(in_channels), spatial_(in_spatial_size), phase_(phase), momentum_(momentum),
      eps_(epsilon), update_immidiately_(false), mean_(in_channels), variance_(in_channels),
      mean_current_(in_channels), variance_current_(in_channels), stddev_(in_channels),
      buf_(new detail::norm_buffers()) {}

  std::string layer_type() const override { return "batch-norm"; }
  layer_desc describe(const shape3d &) const override {
    throw nn_error("batch_normalization_layer is not part of the device-resident train step");
  }
  std::vector<shape3d> in_shape() const { return {shape3d(spatial_, 1, channels_)}; }
  std::vector<shape3d> out_shape() const { return {shape3d(spatial_, 1, channels_)}; }

  // batch_normalization_layer.h:127-169
  void forward_propagation(const std::vector<tensor_t *> &in_data, std::vector<tensor_t *> &out_data) {
    detail::ensure_init();
    const tensor_t &in = *in_data[0];
    tensor_t &out      = *out_data[0];
    const size_t n = in.size(), len = channels_ * spatial_;
    const bool train = phase_ == net_phase::train;
    detail::norm_buffers &b = *buf_;
    float *mean = train ? b.mean_cur.resize(channels_) : b.mean.upload(mean_, channels_);
    float *var  = train ? b.var_cur.resize(channels_) : b.var.upload(variance_, channels_);
    b.y.resize(n * len);
    detail::check(tdh_batchnorm_fwd(static_cast<int>(channels_), static_cast<int>(spatial_),
                                    static_cast<int>(n), eps_, train ? 1 : 0, b.x.upload(in, n, len),
                                    mean, var, b.stddev.resize(channels_), b.y.get()));
    out.resize(n);
    b.y.download(out, n, len);
    detail::download_vec(stddev_, b.stddev.get(), channels_);
    if (train) {
      detail::download_vec(mean_current_, mean, channels_);
      detail::download_vec(variance_current_, var, channels_);
      if (update_immidiately_) {
        mean_     = mean_current_;
        variance_ = variance_current_;
      }
    }
  }

  // batch_normalization_layer.h:87-125
  void back_propagation(const std::vector<tensor_t *> &, const std::vector<tensor_t *> &out_data,
                        std::vector<tensor_t *> &out_grad, std::vector<tensor_t *> &in_grad) {
    detail::ensure_init();
    const tensor_t &curr_out = *out_data[0];
    tensor_t &prev_delta     = *in_grad[0];
    const size_t n = curr_out.size(), len = channels_ * spatial_;
    detail::norm_buffers &b = *buf_;
    b.dx.resize(n * len);
    detail::check(tdh_batchnorm_bwd(static_cast<int>(channels_), static_cast<int>(spatial_),
                                    static_cast<int>(n), b.y.upload(curr_out, n, len),
                                    b.dy.upload(*out_grad[0], n, len),
                                    b.stddev.upload(stddev_, channels_), b.dx.get()));
    prev_delta.resize(n);
    b.dx.download(prev_delta, n, len);
  }

  void set_context(net_phase ctx) { phase_ = ctx; }
  // batch_normalization_layer.h:171-177
  void post_update() {
    detail::ensure_init();
    detail::norm_buffers &b = *buf_;
    detail::check(tdh_batchnorm_update_moving(
      static_cast<int>(channels_), momentum_, b.mean_cur.upload(mean_current_, channels_),
      b.var_cur.upload(variance_current_, channels_), b.mean.upload(mean_, channels_),
      b.var.upload(variance_, channels_)));
    detail::download_vec(mean_, b.mean.get(), channels_);
    detail::download_vec(variance_, b.var.get(), channels_);
  }
  // batch_normalization_layer.h:179-202: the moving averages follow the (absent) weights
  void save(std::ostream &os, const int precision = std::numeric_limits<float_t>::digits10 + 2) const {
    os << std::setprecision(precision);
    for (auto m : mean_) os << m << " ";
    for (auto v : variance_) os << v << " ";
  }
  void load(std::istream &is) {
    for (auto &m : mean_) is >> m;
    for (auto &v : variance_) is >> v;
  }
  void update_immidiately(bool update) { update_immidiately_ = update; }
  void set_stddev(const vec_t &stddev) { stddev_ = stddev; }
  void set_mean(const vec_t &mean) { mean_ = mean; }
  void set_variance(const vec_t &variance) {
    variance_ = variance;
    for (size_t i = 0; i < channels_; ++i) stddev_[i] = std::sqrt(variance_[i] + eps_);
  }
  const vec_t &mean() const { return mean_; }
  const vec_t &variance() const { return variance_; }
  float_t epsilon() const { return eps_; }
  float_t momentum() const { return momentum_; }

 private:
  size_t channels_, spatial_;
  net_phase phase_;
  float_t momentum_, eps_;
  bool update_immidiately_;
  vec_t mean_, variance_, mean_current_, variance_current_, stddev_;
  std::shared_ptr<detail::norm_buffers> buf_;
};

// tiny_dnn/layers/dropout_layer.h:22-147
class dropout_layer : public layer {
 public:
  dropout_layer(size_t in_dim, float_t dropout_rate, net_phase phase = net_phase::train)
    : phase_(phase), dropout_rate_(dropout_rate), scale_(float_t(1) / (float_t(1) - dropout_rate)),
      in_size_(in_dim), mask_(1, std::vector<uint8_t>(in_dim)), buf_(new detail::norm_buffers()) {}

  std::string layer_type() const override { return "dropout"; }
  layer_desc describe(const shape3d &) const override {
    throw nn_error("dropout_layer is not part of the device-resident train step");
  }
  std::vector<shape3d> in_shape() const { return {shape3d(in_size_, 1, 1)}; }
  std::vector<shape3d> out_shape() const { return {shape3d(in_size_, 1, 1)}; }
  void set_dropout_rate(float_t rate) {
    dropout_rate_ = rate;
    scale_        = float_t(1) / (float_t(1) - dropout_rate_);
  }
  float_t dropout_rate() const { return dropout_rate_; }

  // dropout_layer.h:84-117: in the train phase every element of every sample draws its own
  // bernoulli(rate), sample after sample; the products run on the device
  void forward_propagation(const std::vector<tensor_t *> &in_data, std::vector<tensor_t *> &out_data) {
    detail::ensure_init();
    const tensor_t &in = *in_data[0];
    tensor_t &out      = *out_data[0];
    const size_t n = in.size();
    if (mask_.size() < n) mask_.resize(n, mask_[0]);
    const bool train = phase_ == net_phase::train;
    detail::norm_buffers &b = *buf_;
    void *mask = nullptr;
    if (train) {
      flat_.resize(n * in_size_);
      for (size_t s = 0; s < n; ++s) {
        for (size_t i = 0; i < in_size_; ++i) mask_[s][i] = bernoulli(dropout_rate_);
        std::memcpy(flat_.data() + s * in_size_, mask_[s].data(), in_size_);
      }
      mask = b.mask_upload(flat_);
    }
    b.y.resize(n * in_size_);
    detail::check(tdh_dropout_fwd(static_cast<int>(n), static_cast<int>(in_size_), train ? 1 : 0, scale_,
                                  static_cast<const uint8_t *>(mask), b.x.upload(in, n, in_size_), b.y.get()));
    out.resize(n);
    b.y.download(out, n, in_size_);
  }

  // dropout_layer.h:62-82
  void back_propagation(const std::vector<tensor_t *> &, const std::vector<tensor_t *> &,
                        std::vector<tensor_t *> &out_grad, std::vector<tensor_t *> &in_grad) {
    detail::ensure_init();
    const tensor_t &curr_delta = *out_grad[0];
    tensor_t &prev_delta       = *in_grad[0];
    const size_t n = curr_delta.size();
    if (n > mask_.size()) throw nn_error("dropout_layer: backward over more samples than forward");
    detail::norm_buffers &b = *buf_;
    flat_.resize(n * in_size_);
    for (size_t s = 0; s < n; ++s) std::memcpy(flat_.data() + s * in_size_, mask_[s].data(), in_size_);
    b.dx.resize(n * in_size_);
    detail::check(tdh_dropout_bwd(static_cast<int>(n), static_cast<int>(in_size_),
                                  static_cast<const uint8_t *>(b.mask_upload(flat_)),
                                  b.dy.upload(curr_delta, n, in_size_), b.dx.get()));
    prev_delta.resize(n);
    b.dx.download(prev_delta, n, in_size_);
  }

  void set_context(net_phase ctx) { phase_ = ctx; }
  const std::vector<uint8_t> &get_mask(size_t sample_index) const { return mask_[sample_index]; }
  void clear_mask() {
    for (auto &sample : mask_) std::fill(sample.begin(), sample.end(), 0);
  }

 private:
  net_phase phase_;
  float_t dropout_rate_, scale_;
  size_t in_size_;
  std::vector<std::vector<uint8_t>> mask_;
  std::vector<uint8_t> flat_;
  std::shared_ptr<detail::norm_buffers> buf_;
};

namespace detail {
// RAII handle of a tdh_feeder plus the flattening of vector-of-vectors batches
class feeder {
 public:
  feeder(size_t x_len, size_t t_len, size_t max_batch) : x_len_(x_len), t_len_(t_len) {
    check(tdh_feeder_create(x_len, t_len, static_cast<int>(max_batch), &f_));
    x_.resize(x_len * max_batch);
    t_.resize(t_len * max_batch);
  }
  feeder(const feeder &) = delete;
  feeder &operator=(const feeder &) = delete;
  ~feeder() {
    if (f_) tdh_feeder_destroy(f_);
  }
  void stage(const std::vector<vec_t> &x, const std::vector<vec_t> &t, size_t first, size_t n) {
    for (size_t s = 0; s < n; ++s) {
      if (x[first + s].size() < x_len_ || t[first + s].size() < t_len_)
        throw nn_error("fit: sample shorter than the network's input / output");
      std::memcpy(x_.data() + s * x_len_, x[first + s].data(), x_len_ * sizeof(float));
      std::memcpy(t_.data() + s * t_len_, t[first + s].data(), t_len_ * sizeof(float));
    }
    check(tdh_feeder_stage(f_, static_cast<int>(n), x_.data(), t_.data()));
  }
  tdh_feeder *get() const { return f_; }

 private:
  tdh_feeder *f_ = nullptr;
  size_t x_len_, t_len_;
  std::vector<float> x_, t_;
};
}  // namespace detail

struct sequential {};

// network<sequential> (tiny_dnn/network.h:148-1105): operator<<, fit, train, predict. Weights
// live on the device; weights()/set_weights() copy one parameter tensor at a time.
template <typename NetType>
class network;

template <>
class network<sequential> {
 public:
  network() {}
  network(const network &) = delete;
  network &operator=(const network &) = delete;
  ~network() {
    if (net_) tdh_net_destroy(net_);
  }

  template <typename Layer>
  network &add(Layer &&l) {
    layers_.emplace_back(new typename std::decay<Layer>::type(std::forward<Layer>(l)));
    drop();
    return *this;
  }
  size_t layer_size() const { return layers_.size(); }
  size_t depth() const { return layer_size(); }
  const layer *operator[](size_t index) const { return layers_[index].get(); }

  size_t in_data_size() { return build(1), tdh_net_in_size(net_); }
  size_t out_data_size() { return build(1), tdh_net_out_size(net_); }

  // trainable tensors of layer `index`: which = 0 weight, 1 bias
  vec_t weights(size_t index, int which) {
    build(max_batch_ ? max_batch_ : 1);
    vec_t v(tdh_net_param_size(net_, static_cast<int>(index), which));
    detail::check(tdh_net_get_param(net_, static_cast<int>(index), which, v.data()));
    return v;
  }
  void set_weights(size_t index, int which, const vec_t &v) {
    build(max_batch_ ? max_batch_ : 1);
    if (v.size() != tdh_net_param_size(net_, static_cast<int>(index), which))
      throw nn_error("set_weights: size mismatch");
    detail::check(tdh_net_set_param(net_, static_cast<int>(index), which, v.data()));
    initialized_ = true;
  }

  // network::fit (tiny_dnn/network.h:368-386, 840-879): epochs over mini-batches of
  // fprop + loss gradient + bprop + update_weights; the last batch may be short
  template <typename Error, typename Optimizer>
  bool fit(Optimizer &opt, const std::vector<vec_t> &inputs, const std::vector<vec_t> &desired_outputs,
           size_t batch_size, int epoch) {
    return fit<Error>(opt, inputs, desired_outputs, batch_size, epoch, []() {}, []() {});
  }
  template <typename Error, typename Optimizer, typename OnBatch, typename OnEpoch>
  bool fit(Optimizer &opt, const std::vector<vec_t> &inputs, const std::vector<vec_t> &desired_outputs,
           size_t batch_size, int epoch, OnBatch on_batch_enumerate, OnEpoch on_epoch_enumerate) {
    if (inputs.size() != desired_outputs.size() || inputs.empty() || batch_size == 0) return false;
    build(batch_size);
    if (!initialized_) throw nn_error("fit: weights have not been set (set_weights)");
    const size_t in_len = tdh_net_in_size(net_), out_len = tdh_net_out_size(net_);
    opt.reset();  // network.h:856; the device copy of the state vectors is cleared with it
    detail::check(tdh_net_reset_optimizer(net_));
    tdh_opt o = opt.descriptor();
    // batches travel double-buffered: while a step runs, the next batch is flattened, copied
    // to pinned memory and uploaded
    detail::feeder feed(in_len, out_len, batch_size);
    const size_t per_epoch = (inputs.size() + batch_size - 1) / batch_size;
    const size_t total     = per_epoch * static_cast<size_t>(epoch);
    auto stage = [&](size_t k) {
      const size_t i = (k % per_epoch) * batch_size;
      const size_t n = std::min(batch_size, inputs.size() - i);
      feed.stage(inputs, desired_outputs, i, n);
    };
    if (total) stage(0);
    for (size_t k = 0; k < total; ++k) {
      const float *xd = nullptr, *td = nullptr;
      int n = 0;
      detail::check(tdh_feeder_acquire(feed.get(), &xd, &td, &n));
      if (k + 1 < total) stage(k + 1);  // the feeder's thread copies while this one launches
      detail::check(tdh_net_train_step(net_, &o, Error::kind, n, xd, td, 1));
      on_batch_enumerate();
      if ((k + 1) % per_epoch == 0) on_epoch_enumerate();
    }
    opt.absorb(o);
    return true;
  }

  // network::train (tiny_dnn/network.h:284-308): labels become one-hot targets {0,1}
  // (nodes::label2vec with the default out_value_range, tiny_dnn/nodes.h:180-189)
  template <typename Error, typename Optimizer>
  bool train(Optimizer &opt, const std::vector<vec_t> &inputs, const std::vector<label_t> &class_labels,
             size_t batch_size, int epoch) {
    if (inputs.size() != class_labels.size() || inputs.size() < batch_size) return false;
    build(batch_size);
    const size_t out_len = tdh_net_out_size(net_);
    std::vector<vec_t> t(class_labels.size(), vec_t(out_len, float_t(0)));
    for (size_t i = 0; i < class_labels.size(); ++i) {
      if (class_labels[i] >= out_len) throw nn_error("label out of range");
      t[i][class_labels[i]] = float_t(1);
    }
    return fit<Error>(opt, inputs, t, batch_size, epoch);
  }

  // Weights as text, the reference's stream format (network::save / load, tiny_dnn/network.h:
  // 762-771; layer::save / load, tiny_dnn/layers/layer.h:361-385): every trainable vector of
  // every layer in order, each value printed with 8 significant digits and followed by a
  // blank. An average-pooling layer's weight vector has pool_w*pool_h*channels entries in the
  // reference's files although only the first `channels` are ever read
  // (average_pooling_layer.h:222-226): the extra ones are written as 0 and skipped on load.
  void save(std::ostream &os) {
    build(max_batch_ ? max_batch_ : 1);
    os << std::setprecision(std::numeric_limits<float_t>::digits10 + 2);
    for (size_t i = 0; i < layers_.size(); ++i)
      for (int which = 0; which < 2; ++which) {
        const vec_t v = weights(i, which);
        for (float_t w : v) os << w << " ";
        for (size_t k = v.size(); k < file_length(i, which); ++k) os << float_t(0) << " ";
      }
  }
  void load(std::istream &is) {
    build(max_batch_ ? max_batch_ : 1);
    for (size_t i = 0; i < layers_.size(); ++i)
      for (int which = 0; which < 2; ++which) {
        vec_t v(tdh_net_param_size(net_, static_cast<int>(i), which));
        for (float_t &w : v) is >> w;
        float_t skipped;
        for (size_t k = v.size(); k < file_length(i, which); ++k) is >> skipped;
        if (is.fail()) throw nn_error("load: the stream holds fewer weights than the network");
        if (!v.empty()) set_weights(i, which, v);
      }
    initialized_ = true;
  }
  // network::fast_load (tiny_dnn/network.h:777-785): the same file through fscanf
  void fast_load(const char *filepath) {
    FILE *stream = std::fopen(filepath, "r");
    if (!stream) throw nn_error(std::string("failed to open file:") + filepath);
    std::vector<float_t> data;
    double temp;
    while (std::fscanf(stream, "%lf", &temp) > 0) data.push_back(float_t(temp));
    std::fclose(stream);
    build(max_batch_ ? max_batch_ : 1);
    size_t idx = 0;
    for (size_t i = 0; i < layers_.size(); ++i)
      for (int which = 0; which < 2; ++which) {
        const size_t n = tdh_net_param_size(net_, static_cast<int>(i), which), len = file_length(i, which);
        if (idx + len > data.size()) throw nn_error("fast_load: the file holds fewer weights than the network");
        if (n) set_weights(i, which, vec_t(data.begin() + idx, data.begin() + idx + n));
        idx += len;
      }
    initialized_ = true;
  }

  // network::predict (tiny_dnn/network.h:226-230)
  vec_t predict(const vec_t &in) {
    build(max_batch_ ? max_batch_ : 1);
    tensor_t xb{in};
    const size_t in_len = tdh_net_in_size(net_), out_len = tdh_net_out_size(net_);
    detail::check(tdh_net_forward(net_, 1, x_.upload(xb, 1, in_len)));
    vec_t out(out_len);
    detail::check(tdh_memcpy_d2h(out.data(), tdh_net_layer_out(net_, static_cast<int>(layers_.size()) - 1),
                                 out_len * sizeof(float)));
    return out;
  }

 private:
  // entries of trainable vector `which` of layer i in a weight file
  size_t file_length(size_t i, int which) {
    const size_t n = tdh_net_param_size(net_, static_cast<int>(i), which);
    const layer_desc d = layers_[i]->describe(shape3d());
    if (d.l.kind == TDH_L_AVEPOOL && which == 0) return n * d.l.pool.pool_w * d.l.pool.pool_h;
    return n;
  }
  void drop() {
    if (net_) tdh_net_destroy(net_);
    net_ = nullptr;
    max_batch_ = 0;
  }
  // (re)creates the device network when the batch capacity grows; parameters are carried over
  void build(size_t batch) {
    detail::ensure_init();
    if (net_ && batch <= max_batch_) return;
    if (layers_.empty()) throw nn_error("network has no layers");
    std::vector<layer_desc> descs;
    shape3d prev;
    for (auto &l : layers_) descs.push_back(l->describe(prev));
    std::vector<tdh_layer> raw(descs.size());
    for (size_t i = 0; i < descs.size(); ++i) {
      raw[i] = descs[i].l;
      if (!descs[i].tbl.empty()) raw[i].conv.tbl = descs[i].tbl.data();
    }
    tdh_net *fresh = nullptr;
    detail::check(tdh_net_create(raw.data(), static_cast<int>(raw.size()), static_cast<int>(batch),
                                 TDH_NET_FUSE_ACT_GRAD | TDH_NET_GRAPH, &fresh));
    if (net_) {
      for (size_t i = 0; i < layers_.size(); ++i)
        for (int which = 0; which < 2; ++which) {
          vec_t v(tdh_net_param_size(net_, static_cast<int>(i), which));
          if (v.empty()) continue;
          detail::check(tdh_net_get_param(net_, static_cast<int>(i), which, v.data()));
          detail::check(tdh_net_set_param(fresh, static_cast<int>(i), which, v.data()));
        }
      tdh_net_destroy(net_);
    }
    net_       = fresh;
    max_batch_ = batch;
  }

  std::vector<std::unique_ptr<layer>> layers_;
  tdh_net *net_     = nullptr;
  size_t max_batch_ = 0;
  bool initialized_ = false;
  detail::device_tensor x_, t_;
};

template <typename Layer>
network<sequential> &operator<<(network<sequential> &n, Layer &&l) {
  return n.add(std::forward<Layer>(l));
}
// tiny_dnn/network.h:1153-1165
inline std::ostream &operator<<(std::ostream &os, network<sequential> &n) {
  n.save(os);
  return os;
}
inline std::istream &operator>>(std::istream &is, network<sequential> &n) {
  n.load(is);
  return is;
}

// ---- data ingest: the reference's dataset readers (tiny_dnn/io/mnist_parser.h,
// tiny_dnn/io/cifar10_parser.h) with their signatures, scaling arithmetic and errors; the
// batches they produce travel to the device through network::fit's double-buffered feeder.
namespace detail {
inline std::vector<uint8_t> read_file(const std::string &path) {
  std::ifstream ifs(path.c_str(), std::ios::in | std::ios::binary);
  if (ifs.bad() || ifs.fail()) throw nn_error("failed to open file:" + path);
  return std::vector<uint8_t>((std::istreambuf_iterator<char>(ifs)), std::istreambuf_iterator<char>());
}
// big-endian 32-bit field at byte `at`; bytes past the end read as 0, like a failed ifstream::read
inline uint32_t be32(const std::vector<uint8_t> &b, size_t at) {
  uint32_t v = 0;
  for (size_t i = 0; i < 4; ++i) v = (v << 8) | (at + i < b.size() ? b[at + i] : 0u);
  return v;
}
}  // namespace detail

// mnist_parser.h:77-102: idx1 file, magic 0x00000801
inline void parse_mnist_labels(const std::string &label_file, std::vector<label_t> *labels) {
  const std::vector<uint8_t> b = detail::read_file(label_file);
  const uint32_t magic = detail::be32(b, 0), num_items = detail::be32(b, 4);
  if (magic != 0x00000801 || num_items <= 0) throw nn_error("MNIST label-file format error");
  labels->resize(num_items);
  for (uint32_t i = 0; i < num_items; ++i)
    (*labels)[i] = static_cast<label_t>(8 + static_cast<size_t>(i) < b.size() ? b[8 + i] : 0);
}

// mnist_parser.h:121-147 (+ :26-75): idx3 file, magic 0x00000803; pixel p becomes
// (p / 255) * (scale_max - scale_min) + scale_min, the border added by the paddings scale_min
inline void parse_mnist_images(const std::string &image_file, std::vector<vec_t> *images,
                               float_t scale_min, float_t scale_max, int x_padding, int y_padding) {
  if (x_padding < 0 || y_padding < 0) throw nn_error("padding size must not be negative");
  if (scale_min >= scale_max) throw nn_error("scale_max must be greater than scale_min");
  const std::vector<uint8_t> b = detail::read_file(image_file);
  const uint32_t magic = detail::be32(b, 0), num_items = detail::be32(b, 4);
  const uint32_t rows = detail::be32(b, 8), cols = detail::be32(b, 12);
  if (magic != 0x00000803 || num_items <= 0) throw nn_error("MNIST label-file format error");
  const size_t width = cols + 2 * static_cast<size_t>(x_padding), height = rows + 2 * static_cast<size_t>(y_padding);
  images->resize(num_items);
  for (uint32_t i = 0; i < num_items; ++i) {
    vec_t &dst = (*images)[i];
    dst.assign(width * height, scale_min);
    const size_t base = 16 + static_cast<size_t>(i) * rows * cols;
    for (uint32_t y = 0; y < rows; ++y)
      for (uint32_t x = 0; x < cols; ++x) {
        const size_t at = base + static_cast<size_t>(y) * cols + x;
        const uint8_t p = at < b.size() ? b[at] : 0;
        dst[width * (y + y_padding) + x + x_padding] = (p / float_t(255)) * (scale_max - scale_min) + scale_min;
      }
  }
}

// cifar10_parser.h:38-86: records of one label byte and 3 x 32 x 32 pixel bytes, appended to
// the vectors; pixel c becomes scale_min + (scale_max - scale_min) * c / 255
inline void parse_cifar10(const std::string &filename, std::vector<vec_t> *train_images,
                          std::vector<label_t> *train_labels, float_t scale_min, float_t scale_max,
                          int x_padding, int y_padding) {
  if (x_padding < 0 || y_padding < 0) throw nn_error("padding size must not be negative");
  if (scale_min >= scale_max) throw nn_error("scale_max must be greater than scale_min");
  const std::vector<uint8_t> b = detail::read_file(filename);
  const size_t depth = 3, side = 32, area = side * side, record = 1 + depth * area;
  const size_t w = side + 2 * static_cast<size_t>(x_padding), h = side + 2 * static_cast<size_t>(y_padding);
  for (size_t at = 0; at + record <= b.size(); at += record) {
    vec_t img(w * h * depth, scale_min);
    for (size_t c = 0; c < depth; ++c)
      for (size_t y = 0; y < side; ++y)
        for (size_t x = 0; x < side; ++x)
          img[c * w * h + (y + y_padding) * w + x + x_padding] =
            scale_min + (scale_max - scale_min) * b[at + 1 + c * area + y * side + x] / 255;
    train_images->push_back(std::move(img));
    train_labels->push_back(b[at]);
  }
}

}  // namespace tiny_dnn
