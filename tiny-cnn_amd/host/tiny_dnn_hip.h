// tiny_dnn_hip.h — host side of the MI355X hot path in the reference's own language.
//
// A thin, header-only C++14 mirror of the part of tiny-dnn's API that drives the training hot
// path, with the same names, argument meaning and error behaviour, sitting on the C ABI of
// libtdh.so (include/tdh.h). It is not a copy of tiny-dnn: no CPU kernels, no model
// serialization, no graph networks — only what a program needs to switch this path to the GPU:
//
//   * vec_t / tensor_t / shape3d / padding / nn_error      (tiny_dnn/util/util.h, nn_error.h)
//   * core::backend_t with the added value `hip`           (tiny_dnn/core/backend.h:30)
//   * core::Params, conv_params, fully_params, maxpool_params, avepool_params (new)
//   * core::OpKernelConstruction / OpKernelContext / OpKernel
//                                                          (tiny_dnn/core/framework/op_kernel.h)
//   * Conv2dOp, Conv2dGradOp, FullyConnectedOp, FullyConnectedGradOp, MaxPoolOp, MaxPoolGradOp
//     and the new AvePoolOp / AvePoolGradOp, whose compute(OpKernelContext&) dispatch to libtdh
//   * gradient_descent / momentum / adam with the reference's members and update() signature
//   * node / edge / layer with forward(), backward(), setup(), update_weight(), connect() and the
//     `sequential` container (tiny_dnn/node.h, layers/layer.h, nodes.h): the reference's call
//     chain from network::train down to OpKernel::compute, with the edges' tensors resident on
//     the device between the layers
//   * network<sequential> with operator<<, fit<Loss>, train<Loss>, predict, save / load — by
//     default the whole step is one fused, graph-replayed device program (tdh_net_*);
//     set_execution(layer_by_layer) runs the layer chain instead
//
// compute() takes host tensors, as the OpKernelContext contract requires. Tensors that belong to
// an edge stay on the device until host code asks for them; tensors a caller built by hand are
// uploaded and downloaded around every compute() unless set_device_resident(true) is in force.
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

// ---- device mirror of host tensors ------------------------------------------------------
// tiny-dnn's tensors are owned by edges (tiny_dnn/node.h:130-135) and only borrowed by
// OpKernel::compute (tiny_dnn/core/framework/op_kernel.h:74-96). The operators below keep a
// device image of every tensor they are handed, in a table keyed by the address of the host
// tensor_t, with one valid bit per side:
//
//   tensors of an edge (class edge below) are ADOPTED by the mirror for the edge's lifetime and
//     always resident: an input is uploaded only when the host side is the newer one, outputs
//     stay on the device, and edge::get_data() / get_gradient() bring the host copy up to date
//     when host code asks for it (the non-const forms also mark the host side as the newer
//     one). Weights, activations and gradients so stay on the device across layer::forward,
//     layer::backward and layer::update_weight without the caller doing anything;
//   loose tensors (handed to compute() by a caller that built the pointer vectors itself) are
//     write-through by default: compute() uploads its inputs and downloads its outputs, so a
//     caller sees exactly what the reference's CPU kernels leave in the host vectors. With
//     set_device_resident(true) they are treated like edge tensors, and the host says
//     to_host(t) / host_modified(t) itself. A loose tensor is recognised by its address and the
//     address of its first row's values; when another tensor turns up at a known address, the
//     image held for the old one is dropped, never used and never copied into the new one.
//     (A new tensor whose first row also lands at the old row's address cannot be told apart:
//     release_device_copy(t) before destroying a loose tensor in resident mode, or use edges.)
struct transfer_counters {
  size_t h2d_calls = 0, h2d_bytes = 0, d2h_calls = 0, d2h_bytes = 0;
};
inline transfer_counters &transfers() {
  static transfer_counters c;
  return c;
}

class mirror {
 public:
  static mirror &get() {
    static mirror m;
    return m;
  }
  bool resident = false;  // loose tensors; adopted ones always are

  // an edge's tensor: identity is certain until release(), residency does not depend on the mode
  void adopt(const tensor_t &t) {
    entry &e = table_[&t];
    e.owned = true;
    e.seen  = true;
    remember(e, t);
  }
  bool is_resident(const tensor_t &t) const {
    auto it = table_.find(&t);
    return resident || (it != table_.end() && it->second.owned);
  }
  // the device holds values of t that the host copy does not
  bool device_is_newer(const tensor_t &t) const {
    auto it = table_.find(&t);
    return it != table_.end() && it->second.dev_valid && !it->second.host_valid;
  }

  // device image of rows [0, rows) x len of t, for reading
  const float *read(const tensor_t &t, size_t rows, size_t len) {
    entry &e = find(t, rows, len);
    if (!e.dev_valid || !(resident || e.owned)) upload(e, t, rows, len);
    return e.dev;
  }
  // ... for overwriting: nothing is uploaded; the host copy is stale until to_host / commit
  float *write(tensor_t &t, size_t rows, size_t len) {
    entry &e = find(t, rows, len);
    reserve(e, rows * len);
    e.rows = rows; e.len = len;
    e.dev_valid = true; e.host_valid = false;
    return e.dev;
  }
  // ... for adding to (weight and bias gradients: the reference's +=)
  float *update(tensor_t &t, size_t rows, size_t len) {
    entry &e = find(t, rows, len);
    if (!e.dev_valid || !(resident || e.owned)) upload(e, t, rows, len);
    e.host_valid = false;
    return e.dev;
  }
  // after a compute(): write-through brings the host copy up to date now
  void commit(tensor_t &t) {
    if (!is_resident(t)) to_host(t);
  }
  void to_host(tensor_t &t) {
    auto it = table_.find(&t);
    if (it == table_.end() || it->second.host_valid || !it->second.dev_valid) return;
    entry &e = it->second;
    const size_t rows = e.rows, len = e.len;
    e.stage.resize(rows * len);
    if (rows * len > 0) {
      check(tdh_memcpy_d2h(e.stage.data(), e.dev, rows * len * sizeof(float)));
      transfers().d2h_calls++; transfers().d2h_bytes += rows * len * sizeof(float);
    }
    if (t.size() < rows) t.resize(rows);
    for (size_t s = 0; s < rows; ++s) {
      if (t[s].size() < len) t[s].resize(len);
      std::memcpy(t[s].data(), e.stage.data() + s * len, len * sizeof(float));
    }
    e.host_valid = true;
    remember(e, t);
  }
  void host_modified(const tensor_t &t) {
    auto it = table_.find(&t);
    if (it != table_.end()) { it->second.dev_valid = false; it->second.host_valid = true; }
  }
  // zero on both sides without a transfer (edge::clear_grads, tiny_dnn/node.h:105-111)
  void clear(tensor_t &t) {
    for (auto &row : t) std::fill(row.begin(), row.end(), float_t(0));
    auto it = table_.find(&t);
    if (it == table_.end()) return;
    entry &e = it->second;
    if (e.dev && e.rows * e.len > 0) check(tdh_fill_zero(e.dev, e.rows * e.len * sizeof(float)));
    e.dev_valid = e.dev != nullptr; e.host_valid = true;
  }
  void release(const tensor_t &t) {
    auto it = table_.find(&t);
    if (it == table_.end()) return;
    if (it->second.dev) tdh_free(it->second.dev);
    rows_.erase(it->second.row0_vec);
    table_.erase(it);
  }
  // floats per sample of t: of the device image where that is the newer side (the host rows
  // of a resident tensor may never have been filled), else of the host rows
  size_t row_length(const tensor_t &t) const {
    auto it = table_.find(&t);
    if (it != table_.end() && !it->second.host_valid && it->second.dev_valid) return it->second.len;
    return t.empty() ? 0 : t[0].size();
  }
  // the tensor whose only mirrored row is this vector (optimizer::update is handed rows)
  tensor_t *owner_of(const vec_t &row) {
    auto it = rows_.find(&row);
    return it == rows_.end() ? nullptr : const_cast<tensor_t *>(it->second);
  }
  ~mirror() {
    for (auto &kv : table_)
      if (kv.second.dev) tdh_free(kv.second.dev);
  }

 private:
  struct entry {
    float *dev = nullptr;
    size_t cap = 0, rows = 0, len = 0;
    const float *row0 = nullptr;     // data() of row 0 when the host side was last seen
    const vec_t *row0_vec = nullptr;
    bool host_valid = true, dev_valid = false;
    bool owned = false;              // adopted by an edge: the address cannot be reused meanwhile
    bool seen  = false;              // a tensor has been met at this address before
    std::vector<float> stage;
  };
  void reserve(entry &e, size_t floats) {
    if (floats <= e.cap && e.dev) return;
    if (e.dev) check(tdh_free(e.dev));
    e.dev = nullptr;
    void *p = nullptr;
    check(tdh_malloc(&p, std::max<size_t>(floats, 1) * sizeof(float)));
    e.dev = static_cast<float *>(p);
    e.cap = std::max<size_t>(floats, 1);
  }
  void remember(entry &e, const tensor_t &t) {
    if (e.row0_vec) rows_.erase(e.row0_vec);
    e.row0     = t.empty() ? nullptr : t[0].data();
    e.row0_vec = t.empty() ? nullptr : &t[0];
    if (e.row0_vec) rows_[e.row0_vec] = &t;
  }
  entry &find(const tensor_t &t, size_t rows, size_t len) {
    entry &e = table_[&t];
    const float *r0 = t.empty() ? nullptr : t[0].data();
    // the tensor this entry was made for? An adopted one always; a loose one when its first
    // row's values still lie where they were last seen
    const bool known = e.owned || (e.seen && r0 == e.row0);
    e.seen = true;
    if (!known) {
      // another tensor lives at this address now: the image belonged to one that is gone
      e.dev_valid  = false;
      e.host_valid = true;
    }
    const bool same = known && e.rows == rows && e.len == len;
    if (!same && e.host_valid) e.dev_valid = false;
    if (!same && !e.host_valid && (e.rows < rows || e.len != len)) {
      // the device holds the newer values of a smaller image: save them before it is replaced
      to_host(const_cast<tensor_t &>(t));
      e.dev_valid = false;
    }
    if (e.row0_vec == nullptr || (!t.empty() && &t[0] != e.row0_vec)) remember(e, t);
    return e;
  }
  void upload(entry &e, const tensor_t &t, size_t rows, size_t len) {
    if (!e.host_valid) {  // the device is newer: nothing to send
      if (e.rows >= rows && e.len == len) return;
      throw nn_error("device mirror: a tensor was resized while its newest values were on the device");
    }
    if (t.size() < rows) throw nn_error("tensor has fewer samples than the call needs");
    reserve(e, rows * len);
    e.stage.resize(rows * len);
    for (size_t s = 0; s < rows; ++s) {
      if (t[s].size() < len) throw nn_error("tensor row shorter than the layer shape");
      std::memcpy(e.stage.data() + s * len, t[s].data(), len * sizeof(float));
    }
    if (rows * len > 0) {
      check(tdh_memcpy_h2d(e.dev, e.stage.data(), rows * len * sizeof(float)));
      transfers().h2d_calls++; transfers().h2d_bytes += rows * len * sizeof(float);
    }
    e.rows = rows; e.len = len; e.dev_valid = true;
    remember(e, t);
  }
  std::map<const tensor_t *, entry> table_;
  std::map<const vec_t *, const tensor_t *> rows_;
};

// device argmax records of a max-pool layer, shared by its forward and backward operators
// (the reference keeps them in maxpool_params::out2inmax)
struct argmax_store {
  device_tensor idx;
  size_t samples = 0;
  bool host_valid = true;
};
inline argmax_store &argmax_of(const void *params) {
  static std::map<const void *, std::shared_ptr<argmax_store>> table;
  std::shared_ptr<argmax_store> &p = table[params];
  if (!p) p.reset(new argmax_store());
  return *p;
}

}  // namespace detail

// ---- the host's side of the mirror protocol (see detail::mirror) ----
inline void set_device_resident(bool on) { detail::mirror::get().resident = on; }
inline bool device_resident() { return detail::mirror::get().resident; }
// brings the host copy of t up to date (a download only if the device holds newer values)
inline void to_host(tensor_t &t) { detail::mirror::get().to_host(t); }
// the host has written t: the device copy is stale
inline void host_modified(const tensor_t &t) { detail::mirror::get().host_modified(t); }
// edge::clear_grads (tiny_dnn/node.h:105-111) on both sides, without a transfer
inline void clear_grads(tensor_t &t) { detail::mirror::get().clear(t); }
// frees the device image of a tensor that is about to be destroyed
inline void release_device_copy(const tensor_t &t) { detail::mirror::get().release(t); }
// host<->device copies made by the mirror since the last reset (for tests of residency)
inline detail::transfer_counters transfer_stats() { return detail::transfers(); }
inline void reset_transfer_stats() { detail::transfers() = detail::transfer_counters(); }

class layer;

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
  const tensor_t &input(const int idx) const { return *(*in_data_)[idx]; }
  tensor_t &output(const int idx) { return *(*out_data_)[idx]; }
  const tensor_t &output(const int idx) const { return *(*out_data_)[idx]; }
  tensor_t &input_grad(const int idx) { return *(*in_grad_)[idx]; }
  const tensor_t &input_grad(const int idx) const { return *(*in_grad_)[idx]; }
  tensor_t &output_grad(const int idx) { return *(*out_grad_)[idx]; }
  const tensor_t &output_grad(const int idx) const { return *(*out_grad_)[idx]; }
  void setLayer(layer *l) { layer_ = l; }   // op_kernel.h:112-114
  layer *Layer() const { return layer_; }
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
  layer *layer_     = nullptr;
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

// Every compute() takes its tensors through the device mirror (detail::mirror): inputs are
// uploaded only when the device does not hold their newest values, outputs stay on the device in
// resident mode and are written through to the host vectors otherwise.

// tiny_dnn/core/kernels/conv2d_op.h:18-52
class Conv2dOp : public core::OpKernel {
 public:
  explicit Conv2dOp(const core::OpKernelConstruction &context) : core::OpKernel(context) {}
  void compute(core::OpKernelContext &context) override {
    detail::require_hip(context.engine());
    detail::ensure_init();
    auto &params = OpKernel::params_->conv();
    detail::conv_desc_holder h(params);
    detail::mirror &m = detail::mirror::get();
    const tensor_t &in = context.input(0);
    tensor_t &out      = context.output(0);
    const size_t n = in.size();
    const float *bias = params.has_bias ? m.read(context.input(2), 1, params.out.depth_) : nullptr;
    const float *x = m.read(in, n, params.in.size());
    const float *w = m.read(context.input(1), 1, params.weight.size());
    if (out.size() < n) out.resize(n);
    detail::check(tdh_conv2d_fwd(&h.d, static_cast<int>(n), x, w, bias, m.write(out, n, params.out.size())));
    m.commit(out);
  }
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
    detail::mirror &m = detail::mirror::get();
    const tensor_t &prev_out = context.input(0);
    tensor_t &dW             = context.input_grad(1);
    tensor_t &prev_delta     = context.input_grad(0);
    const size_t n = prev_out.size();
    const float *x  = m.read(prev_out, n, params.in.size());
    const float *w  = m.read(context.input(1), 1, params.weight.size());
    const float *dy = m.read(context.output_grad(0), n, params.out.size());
    if (prev_delta.size() < n) prev_delta.resize(n);
    // dX is overwritten (conv2d_grad_op.h:34); dW and db are added to, reduced over the batch,
    // in sample slot 0 of the gradient tensors
    float *dx = m.write(prev_delta, n, params.in.size());
    float *dw = m.update(dW, 1, params.weight.size());
    float *db = params.has_bias ? m.update(context.input_grad(2), 1, params.out.depth_) : nullptr;
    detail::check(tdh_conv2d_bwd(&h.d, static_cast<int>(n), x, w, dy, dx, dw, db, /*accumulate=*/1));
    m.commit(prev_delta);
    m.commit(dW);
    if (params.has_bias) m.commit(context.input_grad(2));
  }
};

// tiny_dnn/core/kernels/fully_connected_op.h:20-65
class FullyConnectedOp : public core::OpKernel {
 public:
  explicit FullyConnectedOp(const core::OpKernelConstruction &context) : core::OpKernel(context) {}
  void compute(core::OpKernelContext &context) override {
    detail::require_hip(context.engine());
    detail::ensure_init();
    auto &params = OpKernel::params_->fully();
    detail::mirror &m = detail::mirror::get();
    const tensor_t &in = context.input(0);
    tensor_t &out      = context.output(0);
    const size_t n = in.size();
    const float *bias = params.has_bias_ ? m.read(context.input(2), 1, params.out_size_) : nullptr;
    const float *x = m.read(in, n, params.in_size_);
    const float *w = m.read(context.input(1), 1, params.in_size_ * params.out_size_);
    if (out.size() < n) out.resize(n);
    detail::check(tdh_fc_fwd(static_cast<int>(params.in_size_), static_cast<int>(params.out_size_),
                             params.has_bias_, static_cast<int>(n), x, w, bias,
                             m.write(out, n, params.out_size_)));
    m.commit(out);
  }
};

// tiny_dnn/core/kernels/fully_connected_grad_op.h:17-53
class FullyConnectedGradOp : public core::OpKernel {
 public:
  explicit FullyConnectedGradOp(const core::OpKernelConstruction &context) : core::OpKernel(context) {}
  void compute(core::OpKernelContext &context) override {
    detail::require_hip(context.engine());
    detail::ensure_init();
    auto &params = OpKernel::params_->fully();
    detail::mirror &m = detail::mirror::get();
    const tensor_t &prev_out = context.input(0);
    tensor_t &prev_delta     = context.input_grad(0);
    const size_t n = prev_out.size(), in = params.in_size_, out = params.out_size_;
    const float *x  = m.read(prev_out, n, in);
    const float *w  = m.read(context.input(1), 1, in * out);
    const float *dy = m.read(context.output_grad(0), n, out);
    if (prev_delta.size() < n) prev_delta.resize(n);
    float *dx = m.write(prev_delta, n, in);
    float *dw = m.update(context.input_grad(1), 1, in * out);
    float *db = params.has_bias_ ? m.update(context.input_grad(2), 1, out) : nullptr;
    detail::check(tdh_fc_bwd(static_cast<int>(in), static_cast<int>(out), params.has_bias_,
                             static_cast<int>(n), x, w, dy, dx, dw, db, 1));
    m.commit(prev_delta);
    m.commit(context.input_grad(1));
    if (params.has_bias_) m.commit(context.input_grad(2));
  }
};

namespace detail {
// maxpool_params::out2inmax from the device records (a download; resident callers ask for it
// through max_pooling_layer::out2inmax())
inline void argmax_to_host(core::maxpool_params &params) {
  argmax_store &a = argmax_of(&params);
  if (a.host_valid) return;
  const size_t n = a.samples, osz = params.out.size();
  std::vector<int32_t> host(n * osz);
  if (n * osz > 0) {
    check(tdh_memcpy_d2h(host.data(), a.idx.get(), host.size() * sizeof(int32_t)));
    transfers().d2h_calls++; transfers().d2h_bytes += host.size() * sizeof(int32_t);
  }
  params.out2inmax.resize(n);
  for (size_t s = 0; s < n; ++s) params.out2inmax[s].assign(host.begin() + s * osz, host.begin() + (s + 1) * osz);
  a.host_valid = true;
}
}  // namespace detail

// tiny_dnn/core/kernels/maxpool_op.h:18-63; the argmax records stay on the device for the
// backward operator and reach params.out2inmax in write-through mode or on request
class MaxPoolOp : public core::OpKernel {
 public:
  explicit MaxPoolOp(const core::OpKernelConstruction &context) : core::OpKernel(context) {}
  void compute(core::OpKernelContext &context) override {
    detail::require_hip(context.engine());
    detail::ensure_init();
    auto &params = OpKernel::params_->maxpool();
    const tdh_pool_desc d = detail::pool_desc(params);
    detail::mirror &m = detail::mirror::get();
    const tensor_t &in = context.input(0);
    tensor_t &out      = context.output(0);
    const size_t n = in.size(), osz = params.out.size();
    detail::argmax_store &a = detail::argmax_of(&params);
    a.idx.resize(n * osz);
    const float *x = m.read(in, n, params.in.size());
    if (out.size() < n) out.resize(n);
    detail::check(tdh_maxpool_fwd(&d, static_cast<int>(n), x, m.write(out, n, osz),
                                  reinterpret_cast<int32_t *>(a.idx.get())));
    a.samples = n;
    a.host_valid = false;
    m.commit(out);
    if (!m.is_resident(out)) detail::argmax_to_host(params);
  }
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
    detail::mirror &m = detail::mirror::get();
    tensor_t &prev_delta = context.input_grad(0);
    const tensor_t &curr_delta = context.output_grad(0);
    const size_t n = curr_delta.size(), osz = params.out.size();
    detail::argmax_store &a = detail::argmax_of(&params);
    if (a.host_valid) {
      // the host's records are the current ones (a caller wrote out2inmax, or no forward pass
      // has run on the device yet)
      if (params.out2inmax.size() < n) throw nn_error("max-pool backward without a recorded forward pass");
      std::vector<int32_t> host(n * osz);
      for (size_t s = 0; s < n; ++s)
        for (size_t i = 0; i < osz; ++i) host[s * osz + i] = static_cast<int32_t>(params.out2inmax[s][i]);
      a.idx.resize(n * osz);
      if (n * osz > 0) {
        detail::check(tdh_memcpy_h2d(a.idx.get(), host.data(), host.size() * sizeof(int32_t)));
        detail::transfers().h2d_calls++; detail::transfers().h2d_bytes += host.size() * sizeof(int32_t);
      }
      a.samples = n;
    } else if (a.samples < n) {
      throw nn_error("max-pool backward over more samples than the forward pass");
    }
    const float *dy = m.read(curr_delta, n, osz);
    if (prev_delta.size() < n) prev_delta.resize(n);
    detail::check(tdh_maxpool_bwd(&d, static_cast<int>(n), dy, reinterpret_cast<const int32_t *>(a.idx.get()),
                                  m.write(prev_delta, n, params.in.size())));
    m.commit(prev_delta);
  }
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
    detail::mirror &m = detail::mirror::get();
    const tensor_t &in = context.input(0);
    tensor_t &out      = context.output(0);
    const size_t n = in.size(), c = params.in.depth_;
    const float *x = m.read(in, n, params.in.size());
    const float *w = m.read(context.input(1), 1, c);
    const float *b = m.read(context.input(2), 1, c);
    if (out.size() < n) out.resize(n);
    detail::check(tdh_avepool_fwd(&d, static_cast<int>(n), x, w, b, m.write(out, n, params.out.size())));
    m.commit(out);
  }
};

class AvePoolGradOp : public core::OpKernel {
 public:
  explicit AvePoolGradOp(const core::OpKernelConstruction &context) : core::OpKernel(context) {}
  void compute(core::OpKernelContext &context) override {
    detail::require_hip(context.engine());
    detail::ensure_init();
    auto &params = OpKernel::params_->avepool();
    const tdh_pool_desc d = detail::pool_desc(params);
    detail::mirror &m = detail::mirror::get();
    const tensor_t &prev_out = context.input(0);
    tensor_t &prev_delta     = context.input_grad(0);
    const size_t n = prev_out.size(), c = params.in.depth_;
    const float *x  = m.read(prev_out, n, params.in.size());
    const float *w  = m.read(context.input(1), 1, c);
    const float *dy = m.read(context.output_grad(0), n, params.out.size());
    if (prev_delta.size() < n) prev_delta.resize(n);
    float *dx = m.write(prev_delta, n, params.in.size());
    float *dw = m.update(context.input_grad(1), 1, c);
    float *db = m.update(context.input_grad(2), 1, c);
    detail::check(tdh_avepool_bwd(&d, static_cast<int>(n), x, w, dy, dx, dw, db, 1));
    m.commit(prev_delta);
    m.commit(context.input_grad(1));
    m.commit(context.input_grad(2));
  }
};

// ---- loss functions (type tags; tiny_dnn/lossfunctions/loss_function.h) ----
// f() is the loss value of one sample, evaluated on the host as the reference does (it is only
// ever read by get_loss / gradient_check); the gradients df() run on the device (tdh_loss_grad)
struct mse {  // loss_function.h:18-36
  static const int kind = TDH_LOSS_MSE;
  static float_t f(const vec_t &y, const vec_t &t) {
    float_t d{0.0};
    for (size_t i = 0; i < y.size(); ++i) d += (y[i] - t[i]) * (y[i] - t[i]);
    return d / static_cast<float_t>(y.size());
  }
  static vec_t df(const vec_t &y, const vec_t &t) {
    vec_t d(t.size());
    const float_t factor = float_t(2) / static_cast<float_t>(t.size());
    for (size_t i = 0; i < y.size(); ++i) d[i] = factor * (y[i] - t[i]);
    return d;
  }
};
struct cross_entropy {  // loss_function.h:108-128
  static const int kind = TDH_LOSS_CE;
  static float_t f(const vec_t &y, const vec_t &t) {
    float_t d{0};
    for (size_t i = 0; i < y.size(); ++i)
      d += -t[i] * std::log(y[i]) - (float_t(1) - t[i]) * std::log(float_t(1) - y[i]);
    return d;
  }
  static vec_t df(const vec_t &y, const vec_t &t) {
    vec_t d(t.size());
    for (size_t i = 0; i < y.size(); ++i) d[i] = (y[i] - t[i]) / (y[i] * (float_t(1) - y[i]));
    return d;
  }
};
struct cross_entropy_multiclass {  // loss_function.h:131-150
  static const int kind = TDH_LOSS_CE_MULTICLASS;
  static float_t f(const vec_t &y, const vec_t &t) {
    float_t d{0.0};
    for (size_t i = 0; i < y.size(); ++i) d += -t[i] * std::log(y[i]);
    return d;
  }
  static vec_t df(const vec_t &y, const vec_t &t) {
    vec_t d(t.size());
    for (size_t i = 0; i < y.size(); ++i) d[i] = -t[i] / y[i];
    return d;
  }
};
// loss_function.h:158-218: the loss gradient of one sample / of a mini-batch, on the host as in
// the reference (the layer-by-layer chain below hands it to the last layer's output edge; the
// device-resident step of network<sequential> computes the same values in its own kernels)
template <typename E>
vec_t gradient(const vec_t &y, const vec_t &t) {
  return E::df(y, t);
}
template <typename E>
std::vector<vec_t> gradient(const std::vector<vec_t> &y, const std::vector<vec_t> &t) {
  std::vector<vec_t> grads(y.size());
  for (size_t i = 0; i < y.size(); ++i) grads[i] = gradient<E>(y[i], t[i]);
  return grads;
}
inline void apply_cost_if_defined(std::vector<vec_t> &sample_gradient, const std::vector<vec_t> &sample_cost) {
  if (sample_gradient.size() != sample_cost.size()) return;
  for (size_t channel = 0; channel < sample_gradient.size(); ++channel)
    if (sample_gradient[channel].size() == sample_cost[channel].size())
      for (size_t e = 0; e < sample_gradient[channel].size(); ++e) sample_gradient[channel][e] *= sample_cost[channel][e];
}
template <typename E>
std::vector<tensor_t> gradient(const std::vector<tensor_t> &y, const std::vector<tensor_t> &t,
                               const std::vector<tensor_t> &t_cost) {
  std::vector<tensor_t> gradients(y.size());
  for (size_t sample = 0; sample < y.size(); ++sample) {
    gradients[sample] = gradient<E>(y[sample], t[sample]);
    if (sample < t_cost.size()) apply_cost_if_defined(gradients[sample], t_cost[sample]);
  }
  return gradients;
}

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
    // a weight vector (and its gradient) that the operators have mirrored is updated where it
    // lies: resident callers never see it cross the bus
    mirror &m = mirror::get();
    tensor_t *Wt = m.owner_of(W), *Gt = m.owner_of(dW);
    const float *g = Gt ? m.read(*Gt, 1, n) : g_.upload(dW, n);
    float *w = Wt ? m.update(*Wt, 1, n) : w_.upload(W, n);
    check(tdh_opt_update(&o, n, g, 1.0f, w, st.s0.get(), st.s1.get()));
    if (Wt) m.commit(*Wt);
    else if (n) check(tdh_memcpy_d2h(W.data(), w, n * sizeof(float)));
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

namespace weight_init {
// tiny_dnn/util/weight_init.h:15-108: the same classes, formulas and draw order (one fresh
// std::uniform_real_distribution / std::normal_distribution per value from the process-wide
// std::mt19937, tiny_dnn/util/random.h:44-79), so a program built against the same C++ library
// starts from the reference's own initial weights
class function {
 public:
  virtual ~function() {}
  virtual void fill(vec_t *weight, size_t fan_in, size_t fan_out) = 0;
};
class scalable : public function {
 public:
  explicit scalable(float_t value) : scale_(value) {}
  void scale(float_t value) { scale_ = value; }

 protected:
  float_t scale_;
};
inline void uniform_rand(vec_t *w, float_t lo, float_t hi) {
  for (float_t &v : *w) {
    std::uniform_real_distribution<float_t> dst(lo, hi);
    v = dst(random_generator::get_instance()());
  }
}
inline void gaussian_rand(vec_t *w, float_t mean, float_t sigma) {
  for (float_t &v : *w) {
    std::normal_distribution<float_t> dst(mean, sigma);
    v = dst(random_generator::get_instance()());
  }
}
class xavier : public scalable {  // U(+-sqrt(scale / (fan_in + fan_out))), scale 6
 public:
  xavier() : scalable(float_t(6)) {}
  explicit xavier(float_t value) : scalable(value) {}
  void fill(vec_t *weight, size_t fan_in, size_t fan_out) override {
    const float_t weight_base = std::sqrt(scale_ / (fan_in + fan_out));
    uniform_rand(weight, -weight_base, weight_base);
  }
};
class lecun : public scalable {   // U(+-scale / sqrt(fan_in)), scale 1
 public:
  lecun() : scalable(float_t{1}) {}
  explicit lecun(float_t value) : scalable(value) {}
  void fill(vec_t *weight, size_t fan_in, size_t) override {
    const float_t weight_base = scale_ / std::sqrt(float_t(fan_in));
    uniform_rand(weight, -weight_base, weight_base);
  }
};
class gaussian : public scalable {  // N(0, sigma)
 public:
  gaussian() : scalable(float_t{1}) {}
  explicit gaussian(float_t sigma) : scalable(sigma) {}
  void fill(vec_t *weight, size_t, size_t) override { gaussian_rand(weight, float_t{0}, scale_); }
};
class constant : public scalable {
 public:
  constant() : scalable(float_t{0}) {}
  explicit constant(float_t value) : scalable(value) {}
  void fill(vec_t *weight, size_t, size_t) override { std::fill(weight->begin(), weight->end(), scale_); }
};
class he : public scalable {      // N(0, sqrt(scale / fan_in)), scale 2
 public:
  he() : scalable(float_t{2}) {}
  explicit he(float_t value) : scalable(value) {}
  void fill(vec_t *weight, size_t fan_in, size_t) override {
    gaussian_rand(weight, float_t{0}, std::sqrt(scale_ / fan_in));
  }
};
}  // namespace weight_init

// tiny_dnn/util/util.h:273-315
enum class vector_type : int32_t {
  data   = 0x0001000,  // input/output data, fed by other layer or input channel
  weight = 0x0002000,  // trainable parameters, updated for each back propagation
  bias   = 0x0002001,
  label  = 0x0004000,
  aux    = 0x0010000   // layer-specific storage
};
inline vector_type operator&(vector_type lhs, vector_type rhs) {
  return static_cast<vector_type>(static_cast<int32_t>(lhs) & static_cast<int32_t>(rhs));
}
inline bool is_trainable_weight(vector_type vtype) { return (vtype & vector_type::weight) == vector_type::weight; }
inline std::vector<vector_type> std_input_order(bool has_bias) {
  if (has_bias) return {vector_type::data, vector_type::weight, vector_type::bias};
  return {vector_type::data, vector_type::weight};
}

enum class net_phase { train, test };  // tiny_dnn/util/util.h:71

// ---- the computational graph: node, edge (tiny_dnn/node.h:40-136) ----
class node;
class layer;
class edge;
typedef std::shared_ptr<edge> edgeptr_t;

class node : public std::enable_shared_from_this<node> {
 public:
  node(size_t in_size, size_t out_size) : prev_(in_size), next_(out_size) {}
  virtual ~node() {}
  const std::vector<edgeptr_t> &prev() const { return prev_; }
  const std::vector<edgeptr_t> &next() const { return next_; }
  size_t prev_port(const edge &e) const {
    auto it = std::find_if(prev_.begin(), prev_.end(), [&](edgeptr_t ep) { return ep.get() == &e; });
    return static_cast<size_t>(std::distance(prev_.begin(), it));
  }
  size_t next_port(const edge &e) const {
    auto it = std::find_if(next_.begin(), next_.end(), [&](edgeptr_t ep) { return ep.get() == &e; });
    return static_cast<size_t>(std::distance(next_.begin(), it));
  }
  std::vector<node *> prev_nodes() const;
  std::vector<node *> next_nodes() const;

 protected:
  node() = delete;
  friend void connect(layer *head, layer *tail, size_t head_index, size_t tail_index);
  mutable std::vector<edgeptr_t> prev_;
  mutable std::vector<edgeptr_t> next_;
};

// An edge owns the data and the gradient tensor between two layers, as in the reference, and
// both are adopted by the device mirror for the edge's lifetime: the operators find them on the
// device, and the accessors below are where host code meets them.
class edge {
 public:
  edge(node *prev, const shape3d &shape, vector_type vtype)
    : shape_(shape), vtype_(vtype), data_({vec_t(shape.size())}), grad_({vec_t(shape.size())}), prev_(prev) {
    detail::mirror::get().adopt(data_);
    detail::mirror::get().adopt(grad_);
  }
  edge(const edge &) = delete;
  edge &operator=(const edge &) = delete;
  ~edge() {
    detail::mirror::get().release(data_);
    detail::mirror::get().release(grad_);
  }

  // node.h:89-103: dst = sum over the samples' gradients, in sample order
  void merge_grads(vec_t *dst) {
    detail::mirror::get().to_host(grad_);
    const vec_t &grad_head = grad_[0];
    const size_t sz = grad_head.size();
    dst->resize(sz);
    std::copy(grad_head.begin(), grad_head.end(), dst->begin());
    for (size_t sample = 1; sample < grad_.size(); ++sample)
      for (size_t i = 0; i < sz; ++i) (*dst)[i] += grad_[sample][i];
  }
  // node.h:105-111, on both sides without a transfer
  void clear_grads() {
    detail::mirror::get().clear(grad_);
    host_wrote_grad_ = false;
  }

  // Host access. The host copy is brought up to date first (a download only when the device
  // holds newer values); through the non-const forms the host may write, so the device image
  // counts as stale afterwards.
  tensor_t *get_data() {
    detail::mirror::get().to_host(data_);
    detail::mirror::get().host_modified(data_);
    return &data_;
  }
  const tensor_t *get_data() const {
    detail::mirror::get().to_host(const_cast<tensor_t &>(data_));
    return &data_;
  }
  tensor_t *get_gradient() {
    detail::mirror::get().to_host(grad_);
    detail::mirror::get().host_modified(grad_);
    host_wrote_grad_ = true;
    return &grad_;
  }
  const tensor_t *get_gradient() const {
    detail::mirror::get().to_host(const_cast<tensor_t &>(grad_));
    return &grad_;
  }

  // What layer::forward / backward / update_weight hand to the operators: the same tensors,
  // without a transfer and without a change of the valid bits (the operators set those).
  tensor_t *borrowed_data() { return &data_; }
  tensor_t *borrowed_gradient() { return &grad_; }
  // The operators add a weight gradient, already summed over the batch, into sample slot 0 on
  // the device. While no host code has had write access to the gradient since clear_grads, the
  // other slots are still zero and slot 0 on the device is what merge_grads would return.
  bool merged_gradient_on_device() const {
    return !host_wrote_grad_ && detail::mirror::get().device_is_newer(grad_);
  }

  const std::vector<node *> &next() const { return next_; }
  node *prev() { return prev_; }
  const node *prev() const { return prev_; }
  const shape3d &shape() const { return shape_; }
  vector_type vtype() const { return vtype_; }
  void add_next_node(node *next) { next_.push_back(next); }

 private:
  shape3d shape_;
  vector_type vtype_;
  tensor_t data_;
  tensor_t grad_;
  node *prev_;                // previous node, "producer" of this tensor
  std::vector<node *> next_;  // next nodes, "consumers" of this tensor
  bool host_wrote_grad_ = false;
};

inline std::vector<node *> node::prev_nodes() const {
  std::vector<node *> vecs;
  for (auto &e : prev_)
    if (e && e->prev()) vecs.insert(vecs.end(), e->prev());
  return vecs;
}
inline std::vector<node *> node::next_nodes() const {
  std::vector<node *> vecs;
  for (auto &e : next_)
    if (e) {
      auto n = e->next();
      vecs.insert(vecs.end(), n.begin(), n.end());
    }
  return vecs;
}

// ---- layers: constructor arguments as in tiny_dnn/layers/*.h. A layer works in two ways:
//  * layer by layer, as in the reference (tiny_dnn/layers/layer.h): forward() / backward()
//    marshal the tensors of the layer's edges into forward_propagation / back_propagation,
//    which run the layer's OpKernel::compute; update_weight hands the merged gradient and the
//    weights to optimizer::update. Every tensor of an edge stays on the device in between.
//  * described to network<sequential> (describe()), which turns the descriptions into one
//    device-resident tdh_net whose whole train step is fused and replayed as a graph.
struct layer_desc {
  tdh_layer l;
  std::vector<uint8_t> tbl;
};

class layer : public node {
 public:
  // layer.h:58-76
  layer(const std::vector<vector_type> &in_type, const std::vector<vector_type> &out_type)
    : node(in_type.size(), out_type.size()), initialized_(false), parallelize_(true),
      in_channels_(in_type.size()), out_channels_(out_type.size()), in_type_(in_type), out_type_(out_type),
      trainable_(true), weight_init_(std::make_shared<weight_init::xavier>()),
      bias_init_(std::make_shared<weight_init::constant>()) {}
  virtual ~layer() {}
  layer(const layer &) = default;
  layer &operator=(const layer &) = default;

  virtual layer_desc describe(const shape3d &prev_out) const = 0;
  virtual std::string layer_type() const = 0;
  // the name the reference registers for the class (tiny_dnn/util/serialization_layer_list.h),
  // which serialize_prolog writes in front of a layer's weights in a cereal archive
  virtual std::string archive_type_name() const = 0;
  // number of incoming connections of an output unit / outgoing ones of an input unit, which
  // the initialisers scale by (layer.h:298-306)
  virtual size_t fan_in_size() const { return 0; }
  virtual size_t fan_out_size() const { return 0; }
  virtual size_t fan_in_size(size_t) const { return fan_in_size(); }
  virtual size_t fan_out_size(size_t) const { return fan_out_size(); }
  // the (off, on) values label2vec turns class labels into when this is the last layer
  // (layer.h:276-278; activation layers give their scale(), activation_layer.h:121)
  virtual std::pair<float_t, float_t> out_value_range() const { return {float_t{0.0}, float_t{1.0}}; }
  // entries of the weight vector as the reference declares it, where that is more than this
  // library keeps (average pooling): init_weight draws that many values
  virtual size_t declared_weight_size(size_t kept) const { return kept; }
  // layer::weight_init / bias_init (layer.h:338-360)
  template <typename WeightInit>
  layer &weight_init(const WeightInit &f) {
    weight_init_ = std::make_shared<WeightInit>(f);
    return *this;
  }
  template <typename BiasInit>
  layer &bias_init(const BiasInit &f) {
    bias_init_ = std::make_shared<BiasInit>(f);
    return *this;
  }

  // layer.h:271-295
  virtual std::vector<shape3d> in_shape() const = 0;
  virtual std::vector<shape3d> out_shape() const = 0;
  virtual void set_in_shape(const shape3d &) {
    throw nn_error("Can't set shape. Shape inferring not applicable for this layer (yet).");
  }
  // layer.h:414-433
  virtual void forward_propagation(const std::vector<tensor_t *> &in_data, std::vector<tensor_t *> &out_data) = 0;
  virtual void back_propagation(const std::vector<tensor_t *> &in_data, const std::vector<tensor_t *> &out_data,
                                std::vector<tensor_t *> &out_grad, std::vector<tensor_t *> &in_grad) = 0;
  virtual void post_update() {}
  virtual void set_context(net_phase) {}

  void set_parallelize(bool parallelize) { parallelize_ = parallelize; }
  bool parallelize() const { return parallelize_; }
  core::backend_t engine() const { return core::backend_t::hip; }
  size_t in_channels() const { return in_channels_; }
  size_t out_channels() const { return out_channels_; }
  size_t in_data_size() const {
    size_t n = 0;
    const std::vector<shape3d> sh = in_shape();
    for (size_t i = 0; i < sh.size(); ++i)
      if (in_type_[i] == vector_type::data) n += sh[i].size();
    return n;
  }
  size_t out_data_size() const {
    size_t n = 0;
    const std::vector<shape3d> sh = out_shape();
    for (size_t i = 0; i < sh.size(); ++i)
      if (out_type_[i] == vector_type::data) n += sh[i].size();
    return n;
  }
  size_t in_size() const { return in_data_size(); }
  size_t out_size() const { return out_data_size(); }
  std::vector<vector_type> in_types() const { return in_type_; }
  std::vector<vector_type> out_types() const { return out_type_; }
  void set_trainable(bool trainable) { trainable_ = trainable; }
  bool trainable() const { return trainable_; }

  // layer.h:153-211. The vectors handed out are the edges' own: the const forms download what
  // the device holds newer, the non-const forms also count as a write by the host.
  std::vector<const vec_t *> weights() const {
    std::vector<const vec_t *> v;
    for (size_t i = 0; i < in_channels_; i++)
      if (is_trainable_weight(in_type_[i])) v.push_back(get_weight_data(i));
    return v;
  }
  std::vector<vec_t *> weights() {
    std::vector<vec_t *> v;
    for (size_t i = 0; i < in_channels_; i++)
      if (is_trainable_weight(in_type_[i])) v.push_back(get_weight_data(i));
    return v;
  }
  std::vector<tensor_t *> weights_grads() {
    std::vector<tensor_t *> v;
    for (size_t i = 0; i < in_channels_; i++)
      if (is_trainable_weight(in_type_[i])) v.push_back(ith_in_node(i)->get_gradient());
    return v;
  }
  std::vector<edgeptr_t> inputs() {
    std::vector<edgeptr_t> nodes(in_channels_);
    for (size_t i = 0; i < in_channels_; i++) nodes[i] = ith_in_node(i);
    return nodes;
  }
  std::vector<edgeptr_t> outputs() {
    std::vector<edgeptr_t> nodes(out_channels_);
    for (size_t i = 0; i < out_channels_; i++) nodes[i] = ith_out_node(i);
    return nodes;
  }

  // layer.h:213-251: the host writes the first layer's input and the last layer's output gradient
  void set_out_grads(const std::vector<const vec_t *> *grad, size_t cnt) {
    size_t n = 0;
    for (size_t i = 0; i < out_channels_; i++) {
      if (out_type_[i] != vector_type::data) continue;
      tensor_t &dst_grad = *ith_out_node(i)->get_gradient();
      if (n >= cnt) throw nn_error("set_out_grads: fewer gradient channels than data outputs");
      const auto &src_grad = grad[n++];
      dst_grad.resize(src_grad.size());
      for (size_t j = 0; j < src_grad.size(); ++j) dst_grad[j] = *src_grad[j];
    }
  }
  void set_in_data(const std::vector<const vec_t *> *data, size_t cnt) {
    size_t n = 0;
    for (size_t i = 0; i < in_channels_; i++) {
      if (in_type_[i] != vector_type::data) continue;
      tensor_t &dst_data = *ith_in_node(i)->get_data();
      if (n >= cnt) throw nn_error("set_in_data: fewer data channels than data inputs");
      const auto &src_data = data[n++];
      dst_data.resize(src_data.size());
      for (size_t j = 0; j < src_data.size(); ++j) dst_data[j] = *src_data[j];
    }
  }
  void output(std::vector<const tensor_t *> &out) const {
    out.clear();
    for (size_t i = 0; i < out_channels_; i++)
      if (out_type_[i] == vector_type::data)
        out.push_back(static_cast<const edge *>(next_[i].get())->get_data());
  }

  // layer.h:527-575: the tensors of the edges, as they are, go to the layer's operators
  void forward() {
    fwd_in_data_.resize(in_channels_);
    fwd_out_data_.resize(out_channels_);
    for (size_t i = 0; i < in_channels_; i++) fwd_in_data_[i] = ith_in_node(i)->borrowed_data();
    set_sample_count(fwd_in_data_[0]->size());
    for (size_t i = 0; i < out_channels_; i++) {
      fwd_out_data_[i] = ith_out_node(i)->borrowed_data();
      ith_out_node(i)->clear_grads();
    }
    forward_propagation(fwd_in_data_, fwd_out_data_);
  }
  void backward() {
    bwd_in_data_.resize(in_channels_);
    bwd_in_grad_.resize(in_channels_);
    bwd_out_data_.resize(out_channels_);
    bwd_out_grad_.resize(out_channels_);
    for (size_t i = 0; i < in_channels_; i++) {
      const auto &nd  = ith_in_node(i);
      bwd_in_data_[i] = nd->borrowed_data();
      bwd_in_grad_[i] = nd->borrowed_gradient();
    }
    for (size_t i = 0; i < out_channels_; i++) {
      const auto &nd   = ith_out_node(i);
      bwd_out_data_[i] = nd->borrowed_data();
      bwd_out_grad_[i] = nd->borrowed_gradient();
    }
    back_propagation(bwd_in_data_, bwd_out_data_, bwd_out_grad_, bwd_in_grad_);
  }

  // layer.h:584-655
  void setup(bool reset_weight) {
    if (in_shape().size() != in_channels_ || out_shape().size() != out_channels_)
      throw nn_error("Connection mismatch at setup layer");
    for (size_t i = 0; i < out_channels_; i++)
      if (!next_[i]) next_[i] = std::make_shared<edge>(this, out_shape()[i], out_type_[i]);
    if (reset_weight || !initialized_) init_weight();
  }
  void init_weight() {
    if (!trainable_) {
      initialized_ = true;
      return;
    }
    for (size_t i = 0; i < in_channels_; i++) {
      switch (in_type_[i]) {
        case vector_type::weight: weight_init_->fill(get_weight_data(i), fan_in_size(i), fan_out_size(i)); break;
        case vector_type::bias: bias_init_->fill(get_weight_data(i), fan_in_size(i), fan_out_size(i)); break;
        default: break;
      }
    }
    initialized_ = true;
  }
  void clear_grads() {
    for (size_t i = 0; i < in_type_.size(); i++) ith_in_node(i)->clear_grads();
  }
  // layer.h:663-682. The operators leave the gradient of a weight tensor summed over the batch
  // in sample slot 0 on the device; while the host has not written the gradient since the last
  // clear_grads, that slot IS the merged gradient (the other slots are zero) and it goes to the
  // optimizer where it lies. Otherwise the reference's merge runs on the host. rcp_batch_size is
  // 1 / (rows of the weight tensor) = 1, as in the reference.
  void update_weight(optimizer *o) {
    vec_t &diff = weights_diff_;
    for (size_t i = 0; i < in_type_.size(); i++) {
      if (!(trainable() && is_trainable_weight(in_type_[i]))) continue;
      edge &e       = *ith_in_node(i);
      vec_t &target = (*e.borrowed_data())[0];
      const bool parallelize = target.size() >= 512;
      if (e.merged_gradient_on_device()) {
        o->update((*e.borrowed_gradient())[0], target, parallelize);
      } else {
        e.merge_grads(&diff);
        const float_t rcp_batch_size = float_t(1.0) / float_t(e.borrowed_data()->size());
        for (size_t j = 0; j < diff.size(); ++j) diff[j] *= rcp_batch_size;
        o->update(diff, target, parallelize);
      }
    }
    clear_grads();
    post_update();
  }
  bool has_same_weights(const layer &rhs, float_t eps) const {
    auto w1 = weights();
    auto w2 = rhs.weights();
    if (w1.size() != w2.size()) return false;
    for (size_t i = 0; i < w1.size(); i++) {
      if (w1[i]->size() != w2[i]->size()) return false;
      for (size_t j = 0; j < w1[i]->size(); j++)
        if (std::abs(w1[i]->at(j) - w2[i]->at(j)) > eps) return false;
    }
    return true;
  }
  // layer.h:699-718: room for every sample of the batch; never shrinks. Only the outer vectors
  // grow: no values cross the bus here.
  virtual void set_sample_count(size_t sample_count) {
    auto resize = [sample_count](tensor_t *tensor) { tensor->resize(sample_count, (*tensor)[0]); };
    for (size_t i = 0; i < in_channels_; i++) {
      if (!is_trainable_weight(in_type_[i])) resize(ith_in_node(i)->borrowed_data());
      resize(ith_in_node(i)->borrowed_gradient());
    }
    for (size_t i = 0; i < out_channels_; i++) {
      if (!is_trainable_weight(out_type_[i])) resize(ith_out_node(i)->borrowed_data());
      resize(ith_out_node(i)->borrowed_gradient());
    }
  }

  std::shared_ptr<weight_init::function> weight_init_fn() const { return weight_init_; }
  std::shared_ptr<weight_init::function> bias_init_fn() const { return bias_init_; }

 protected:
  bool initialized_;
  bool parallelize_;
  size_t in_channels_, out_channels_;
  std::vector<vector_type> in_type_, out_type_;
  vec_t weights_diff_;

 private:
  friend void connect(layer *head, layer *tail, size_t head_index, size_t tail_index);
  bool trainable_;
  std::shared_ptr<weight_init::function> weight_init_, bias_init_;
  std::vector<tensor_t *> fwd_in_data_, fwd_out_data_, bwd_in_data_, bwd_in_grad_, bwd_out_data_, bwd_out_grad_;

  // layer.h:790-857
  edgeptr_t ith_in_node(size_t i) {
    if (!prev_[i]) prev_[i] = std::make_shared<edge>(nullptr, in_shape()[i], in_type_[i]);
    return prev()[i];
  }
  edgeptr_t ith_out_node(size_t i) {
    if (!next_[i]) next_[i] = std::make_shared<edge>(this, out_shape()[i], out_type_[i]);
    return next()[i];
  }
  vec_t *get_weight_data(size_t i) { return &(*(ith_in_node(i)->get_data()))[0]; }
  const vec_t *get_weight_data(size_t i) const {
    const edge *e = const_cast<layer *>(this)->ith_in_node(i).get();
    return &(*e->get_data())[0];
  }
};

// layer.h:859-884
inline void connect(layer *head, layer *tail, size_t head_index = 0, size_t tail_index = 0) {
  const shape3d out_shape = head->out_shape()[head_index];
  shape3d in_shape        = tail->in_shape()[tail_index];
  head->setup(false);
  if (in_shape.size() == 0) {  // shape inferring: activation layers take the shape in front of them
    tail->set_in_shape(out_shape);
    in_shape = out_shape;
  }
  if (out_shape.size() != in_shape.size())
    throw nn_error("layer dimension mismatch!\noutput size of Nth layer must be equal to input of (N+1)th layer\n" +
                   std::to_string(head->out_data_size()) + " != " + std::to_string(tail->in_data_size()) + " (" +
                   head->layer_type() + " -> " + tail->layer_type() + ")");
  if (!head->next_[head_index]) throw nn_error("output edge must not be null");
  tail->prev_[tail_index] = head->next_[head_index];
  tail->prev_[tail_index]->add_next_node(tail);
}
inline layer &operator<<(layer &lhs, layer &rhs) {
  connect(&lhs, &rhs);
  return rhs;
}

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
                      core::backend_t backend_type = core::default_engine())
    : layer(std_input_order(has_bias), {vector_type::data}) {
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
    init_backend();
  }
  // the operators keep a pointer to this object's params_: a copy gets operators of its own
  // (the reference rebuilds them in its move constructor, convolutional_layer.h:258-266)
  convolutional_layer(const convolutional_layer &o) : layer(o), params_(o.params_) { init_backend(); }
  convolutional_layer &operator=(const convolutional_layer &o) {
    layer::operator=(o);
    params_ = o.params_;
    init_backend();
    return *this;
  }
  std::string layer_type() const override { return "conv"; }
  std::string archive_type_name() const override { return "conv"; }
  // convolutional_layer.h:269-277
  size_t fan_in_size() const override { return params_.weight.width_ * params_.weight.height_ * params_.in.depth_; }
  size_t fan_out_size() const override {
    return (params_.weight.width_ / params_.w_stride) * (params_.weight.height_ / params_.h_stride) *
           params_.out.depth_;
  }
  // convolutional_layer.h:279-291
  std::vector<shape3d> in_shape() const override {
    if (params_.has_bias) return {params_.in, params_.weight, shape3d(1, 1, params_.out.depth_)};
    return {params_.in, params_.weight};
  }
  std::vector<shape3d> out_shape() const override { return {params_.out}; }
  // layer::forward_propagation / back_propagation (convolutional_layer.h:283-337) on the HIP
  // engine: the unpadded edge tensors go straight to the operators
  void forward_propagation(const std::vector<tensor_t *> &in_data, std::vector<tensor_t *> &out_data) override {
    core::OpKernelContext ctx;
    ctx.set_in_out(in_data, out_data);
    ctx.setEngine(core::backend_t::hip);
    kernel_fwd_->compute(ctx);
  }
  void back_propagation(const std::vector<tensor_t *> &in_data, const std::vector<tensor_t *> &out_data,
                        std::vector<tensor_t *> &out_grad, std::vector<tensor_t *> &in_grad) override {
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
  void init_backend() {  // convolutional_layer.h:508-531
    kernel_fwd_.reset(new Conv2dOp(core::OpKernelConstruction(nullptr, &params_)));
    kernel_back_.reset(new Conv2dGradOp(core::OpKernelConstruction(nullptr, &params_)));
  }
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
                        core::backend_t backend_type = core::default_engine())
    : layer(std_input_order(has_bias), {vector_type::data}) {
    detail::require_hip(backend_type);
    params_.in_size_ = in_dim; params_.out_size_ = out_dim; params_.has_bias_ = has_bias;
    init_backend();
  }
  fully_connected_layer(const fully_connected_layer &o) : layer(o), params_(o.params_) { init_backend(); }
  fully_connected_layer &operator=(const fully_connected_layer &o) {
    layer::operator=(o);
    params_ = o.params_;
    init_backend();
    return *this;
  }
  std::string layer_type() const override { return "fully-connected"; }
  std::string archive_type_name() const override { return "fully_connected"; }
  size_t fan_in_size() const override { return params_.in_size_; }     // fully_connected_layer.h:51-53
  size_t fan_out_size() const override { return params_.out_size_; }
  // fully_connected_layer.h:55-68
  std::vector<shape3d> in_shape() const override {
    if (params_.has_bias_)
      return {shape3d(params_.in_size_, 1, 1), shape3d(params_.in_size_, params_.out_size_, 1),
              shape3d(params_.out_size_, 1, 1)};
    return {shape3d(params_.in_size_, 1, 1), shape3d(params_.in_size_, params_.out_size_, 1)};
  }
  std::vector<shape3d> out_shape() const override { return {shape3d(params_.out_size_, 1, 1)}; }
  void forward_propagation(const std::vector<tensor_t *> &in_data, std::vector<tensor_t *> &out_data) override {
    core::OpKernelContext ctx;
    ctx.set_in_out(in_data, out_data);
    ctx.setEngine(core::backend_t::hip);
    kernel_fwd_->compute(ctx);
  }
  void back_propagation(const std::vector<tensor_t *> &in_data, const std::vector<tensor_t *> &out_data,
                        std::vector<tensor_t *> &out_grad, std::vector<tensor_t *> &in_grad) override {
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
  void init_backend() {  // fully_connected_layer.h:105-119
    kernel_fwd_.reset(new FullyConnectedOp(core::OpKernelConstruction(nullptr, &params_)));
    kernel_back_.reset(new FullyConnectedGradOp(core::OpKernelConstruction(nullptr, &params_)));
  }
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
                    core::backend_t backend_type = core::default_engine())
    : layer({vector_type::data}, {vector_type::data}) {
    detail::require_hip(backend_type);
    detail::set_pool_params(params_, in_width, in_height, in_channels, pooling_size_x,
                            pooling_size_y, stride_x, stride_y, ceil_mode, pad_type);
    init_backend();
  }
  max_pooling_layer(const max_pooling_layer &o) : layer(o), params_(o.params_) { init_backend(); }
  max_pooling_layer &operator=(const max_pooling_layer &o) {
    layer::operator=(o);
    params_ = o.params_;
    init_backend();
    return *this;
  }
  std::string layer_type() const override { return "max-pool"; }
  std::string archive_type_name() const override { return "maxpool"; }
  std::vector<shape3d> in_shape() const override { return {params_.in}; }
  std::vector<shape3d> out_shape() const override { return {params_.out}; }
  // maxpool_params::out2inmax of the last forward pass (downloads the device records if they
  // are the newer ones)
  const std::vector<std::vector<size_t>> &out2inmax() {
    detail::argmax_to_host(params_);
    return params_.out2inmax;
  }
  void forward_propagation(const std::vector<tensor_t *> &in_data, std::vector<tensor_t *> &out_data) override {
    core::OpKernelContext ctx;
    ctx.set_in_out(in_data, out_data);
    ctx.setEngine(core::backend_t::hip);
    kernel_fwd_->compute(ctx);
  }
  void back_propagation(const std::vector<tensor_t *> &in_data, const std::vector<tensor_t *> &out_data,
                        std::vector<tensor_t *> &out_grad, std::vector<tensor_t *> &in_grad) override {
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
  void init_backend() {  // max_pooling_layer.h:237-250
    kernel_fwd_.reset(new MaxPoolOp(core::OpKernelConstruction(nullptr, &params_)));
    kernel_back_.reset(new MaxPoolGradOp(core::OpKernelConstruction(nullptr, &params_)));
  }
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
                        padding pad_type = padding::valid)
    : layer(std_input_order(true), {vector_type::data}) {
    if ((in_width % pool_size_x) || (in_height % pool_size_y))
      throw nn_error("width/height not multiples of pooling size");
    detail::set_pool_params(params_, in_width, in_height, in_channels, pool_size_x, pool_size_y,
                            stride_x, stride_y, ceil_mode, pad_type);
    init_backend();
  }
  average_pooling_layer(const average_pooling_layer &o) : layer(o), params_(o.params_) { init_backend(); }
  average_pooling_layer &operator=(const average_pooling_layer &o) {
    layer::operator=(o);
    params_ = o.params_;
    init_backend();
    return *this;
  }
  std::string layer_type() const override { return "ave-pool"; }
  std::string archive_type_name() const override { return "avepool"; }
  // partial_connected_layer.h:46-48 with the connections of average_pooling_layer.h:270-304:
  // every output reads pool_x*pool_y inputs, every input feeds one output (windows that tile)
  size_t fan_in_size() const override { return params_.pool_size_x * params_.pool_size_y; }
  size_t fan_out_size() const override { return 1; }
  size_t declared_weight_size(size_t kept) const override {  // average_pooling_layer.h:222-226
    return kept * params_.pool_size_x * params_.pool_size_y;
  }
  // average_pooling_layer.h:223-227: the weight vector is declared with one entry per window
  // element and channel (only the first `channels` are ever read)
  std::vector<shape3d> in_shape() const override {
    return {params_.in, shape3d(params_.pool_size_x, params_.pool_size_y, params_.in.depth_),
            shape3d(1, 1, params_.out.depth_)};
  }
  std::vector<shape3d> out_shape() const override { return {params_.out}; }
  void forward_propagation(const std::vector<tensor_t *> &in_data, std::vector<tensor_t *> &out_data) override {
    core::OpKernelContext ctx;
    ctx.set_in_out(in_data, out_data);
    ctx.setEngine(core::backend_t::hip);
    kernel_fwd_->compute(ctx);
  }
  void back_propagation(const std::vector<tensor_t *> &in_data, const std::vector<tensor_t *> &out_data,
                        std::vector<tensor_t *> &out_grad, std::vector<tensor_t *> &in_grad) override {
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
  void init_backend() {
    kernel_fwd_.reset(new AvePoolOp(core::OpKernelConstruction(nullptr, &params_)));
    kernel_back_.reset(new AvePoolGradOp(core::OpKernelConstruction(nullptr, &params_)));
  }
  core::avepool_params params_;
  std::shared_ptr<core::OpKernel> kernel_fwd_, kernel_back_;
};

// activation layers (tiny_dnn/activations/*.h): shape is inherited from the previous layer;
// forward_activation / backward_activation keep the reference's signatures
// (activation_layer.h:93-112) on single samples
class activation_layer : public layer {
 public:
  std::string layer_type() const override { return type_; }
  std::string archive_type_name() const override {
    static const char *const names[] = {"tanh", "relu", "softmax", "sigmoid", "leaky_relu", "elu", "selu",
                                        "softplus", "softsign", "asinh", "tanh_scaled"};
    return names[kind_];
  }
  // *_layer::scale() of the reference's activations: tanh and asinh (-0.8, 0.8), softmax (0, 1),
  // all others (0.1, 0.9)
  std::pair<float_t, float_t> out_value_range() const override {
    if (kind_ == TDH_ACT_TANH || kind_ == TDH_ACT_ASINH) return {float_t(-0.8), float_t(0.8)};
    if (kind_ == TDH_ACT_SOFTMAX) return {float_t(0), float_t(1)};
    return {float_t(0.1), float_t(0.9)};
  }
  layer_desc describe(const shape3d &) const override {
    layer_desc r;
    std::memset(&r.l, 0, sizeof(r.l));
    r.l.kind     = TDH_L_ACT;
    r.l.act      = kind_;
    r.l.act_p[0] = p_[0];
    r.l.act_p[1] = p_[1];
    return r;
  }
  // activation_layer.h:66-72: the shape is that of the layer in front (connect() sets it)
  std::vector<shape3d> in_shape() const override { return {in_shape_}; }
  std::vector<shape3d> out_shape() const override { return {in_shape_}; }
  void set_in_shape(const shape3d &in_shape) override { in_shape_ = in_shape; }
  // activation_layer::forward_propagation / back_propagation (activation_layer.h:74-91) over
  // whole batches, through the device mirror like the operators
  void forward_propagation(const std::vector<tensor_t *> &in_data, std::vector<tensor_t *> &out_data) override {
    detail::ensure_init();
    detail::mirror &m = detail::mirror::get();
    const tensor_t &x = *in_data[0];
    tensor_t &y       = *out_data[0];
    const size_t n = x.size(), len = m.row_length(x);
    if (y.size() < n) y.resize(n);
    const float *xd = m.read(x, n, len);
    detail::check(tdh_act_fwd_p(kind_, p_, static_cast<int>(n), static_cast<int>(len), xd, m.write(y, n, len)));
    m.commit(y);
  }
  void back_propagation(const std::vector<tensor_t *> &in_data, const std::vector<tensor_t *> &out_data,
                        std::vector<tensor_t *> &out_grad, std::vector<tensor_t *> &in_grad) override {
    detail::ensure_init();
    detail::mirror &m = detail::mirror::get();
    const tensor_t &y = *out_data[0];
    tensor_t &dx      = *in_grad[0];
    const size_t n = y.size(), len = m.row_length(y);
    if (dx.size() < n) dx.resize(n);
    const float *xd = m.read(*in_data[0], n, len), *yd = m.read(y, n, len), *dyd = m.read(*out_grad[0], n, len);
    detail::check(tdh_act_bwd_p(kind_, p_, static_cast<int>(n), static_cast<int>(len), xd, yd, dyd,
                                m.write(dx, n, len)));
    m.commit(dx);
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
    : layer({vector_type::data}, {vector_type::data}), kind_(kind), type_(type) {
    p_[0] = p0;
    p_[1] = p1;
  }
  int kind_;
  const char *type_;
  float p_[2];
  shape3d in_shape_;

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

// The two layers below run on the device through their own operators when used the way the
// reference's tests use a single layer (forward_propagation / back_propagation on host
// tensors), and are layer kinds of the device-resident step of network<sequential>: there the
// running averages of batch normalization live on the device (weights(i, 2) / weights(i, 3))
// and fit draws every step's dropout masks on the host with the reference's generator.
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
    : layer({vector_type::data}, {vector_type::data}), channels_(in_channels), spatial_(in_spatial_size),
      phase_(phase), momentum_(momentum),
      eps_(epsilon), update_immidiately_(false), mean_(in_channels), variance_(in_channels),
      mean_current_(in_channels), variance_current_(in_channels), stddev_(in_channels),
      buf_(new detail::norm_buffers()) {}

  std::string layer_type() const override { return "batch-norm"; }
  std::string archive_type_name() const override { return "batchnorm"; }
  layer_desc describe(const shape3d &) const override {
    layer_desc r;
    std::memset(&r.l, 0, sizeof(r.l));
    r.l.kind        = TDH_L_BATCHNORM;
    r.l.bn_channels = static_cast<int32_t>(channels_);
    r.l.bn_spatial  = static_cast<int32_t>(spatial_);
    r.l.bn_eps      = eps_;
    r.l.bn_momentum = momentum_;
    return r;
  }
  std::vector<shape3d> in_shape() const override { return {shape3d(spatial_, 1, channels_)}; }
  std::vector<shape3d> out_shape() const override { return {shape3d(spatial_, 1, channels_)}; }

  // batch_normalization_layer.h:127-169
  void forward_propagation(const std::vector<tensor_t *> &in_data, std::vector<tensor_t *> &out_data) override {
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
                        std::vector<tensor_t *> &out_grad, std::vector<tensor_t *> &in_grad) override {
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

  void set_context(net_phase ctx) override { phase_ = ctx; }
  // batch_normalization_layer.h:171-177
  void post_update() override {
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
    : layer({vector_type::data}, {vector_type::data}), phase_(phase), dropout_rate_(dropout_rate),
      scale_(float_t(1) / (float_t(1) - dropout_rate)),
      in_size_(in_dim), mask_(1, std::vector<uint8_t>(in_dim)), buf_(new detail::norm_buffers()) {}

  std::string layer_type() const override { return "dropout"; }
  std::string archive_type_name() const override { return "dropout"; }
  layer_desc describe(const shape3d &) const override {
    layer_desc r;
    std::memset(&r.l, 0, sizeof(r.l));
    r.l.kind         = TDH_L_DROPOUT;
    r.l.dropout_rate = dropout_rate_;
    return r;
  }
  std::vector<shape3d> in_shape() const override { return {shape3d(in_size_, 1, 1)}; }
  std::vector<shape3d> out_shape() const override { return {shape3d(in_size_, 1, 1)}; }
  void set_dropout_rate(float_t rate) {
    dropout_rate_ = rate;
    scale_        = float_t(1) / (float_t(1) - dropout_rate_);
  }
  float_t dropout_rate() const { return dropout_rate_; }

  // dropout_layer.h:84-117: in the train phase every element of every sample draws its own
  // bernoulli(rate), sample after sample; the products run on the device
  void forward_propagation(const std::vector<tensor_t *> &in_data, std::vector<tensor_t *> &out_data) override {
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
                        std::vector<tensor_t *> &out_grad, std::vector<tensor_t *> &in_grad) override {
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

  void set_context(net_phase ctx) override { phase_ = ctx; }
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
    for (int b = 0; b < 2; ++b) {
      x_[b].resize(x_len * max_batch);
      t_[b].resize(t_len * max_batch);
    }
  }
  feeder(const feeder &) = delete;
  feeder &operator=(const feeder &) = delete;
  ~feeder() {
    if (f_) tdh_feeder_destroy(f_);
  }
  // Two batches may be on their way at once, and the feeder's thread reads a batch until it
  // is acquired: the flattened copies alternate between two buffers (the one written here
  // belonged to the batch staged two calls ago, which has been acquired by now).
  void stage(const std::vector<vec_t> &x, const std::vector<vec_t> &t, size_t first, size_t n) {
    std::vector<float> &xf = x_[turn_], &tf = t_[turn_];
    turn_ ^= 1;
    for (size_t s = 0; s < n; ++s) {
      if (x[first + s].size() < x_len_ || t[first + s].size() < t_len_)
        throw nn_error("fit: sample shorter than the network's input / output");
      std::memcpy(xf.data() + s * x_len_, x[first + s].data(), x_len_ * sizeof(float));
      std::memcpy(tf.data() + s * t_len_, t[first + s].data(), t_len_ * sizeof(float));
    }
    check(tdh_feeder_stage(f_, static_cast<int>(n), xf.data(), tf.data()));
  }
  tdh_feeder *get() const { return f_; }

 private:
  tdh_feeder *f_ = nullptr;
  size_t x_len_, t_len_;
  std::vector<float> x_[2], t_[2];
  int turn_ = 0;
};
}  // namespace detail

// tiny_dnn/network.h:32-38
enum class content_type { weights, model, weights_and_model };
enum class file_format { binary, portable_binary, json };

namespace detail {
// Weights-only cereal archives as network::save(filename, content_type::weights, binary /
// portable_binary) writes them (tiny_dnn/network.h:676-728,787-811, nodes::save_weights
// tiny_dnn/nodes.h:203-214): per layer the registered type name as a string (u64 length +
// bytes; serialize_prolog, tiny_dnn/util/serialization_helper.h:118-123), then every trainable
// vector as u64 element count + float32 values (serialization_functions.h:747-754). A
// portable_binary archive starts with one byte: 1 when what follows is little-endian, which is
// what cereal writes on such a host and what is written here.
struct archive_layer {
  std::string type;
  std::vector<vec_t> vectors;
};
inline void put_u64(std::ostream &os, uint64_t v) {
  unsigned char b[8];
  for (int i = 0; i < 8; ++i) b[i] = static_cast<unsigned char>(v >> (8 * i));
  os.write(reinterpret_cast<const char *>(b), 8);
}
inline void write_weight_archive(std::ostream &os, const std::vector<archive_layer> &layers, file_format format) {
  if (format != file_format::binary && format != file_format::portable_binary)
    throw nn_error("invalid serialization format");
  if (format == file_format::portable_binary) os.put(char(1));
  for (const archive_layer &l : layers) {
    put_u64(os, l.type.size());
    os.write(l.type.data(), static_cast<std::streamsize>(l.type.size()));
    for (const vec_t &v : l.vectors) {
      put_u64(os, v.size());
      for (float_t f : v) {  // little-endian float32, whatever the host
        uint32_t bits;
        std::memcpy(&bits, &f, 4);
        const unsigned char b[4] = {static_cast<unsigned char>(bits), static_cast<unsigned char>(bits >> 8),
                                    static_cast<unsigned char>(bits >> 16), static_cast<unsigned char>(bits >> 24)};
        os.write(reinterpret_cast<const char *>(b), 4);
      }
    }
  }
}
// vector_counts[i]: trainable vectors of layer i. Throws nn_error when the stream ends early.
inline std::vector<archive_layer> read_weight_archive(std::istream &is, const std::vector<size_t> &vector_counts,
                                                      file_format format) {
  if (format != file_format::binary && format != file_format::portable_binary)
    throw nn_error("invalid serialization format");
  bool little = true;
  if (format == file_format::portable_binary) {
    const int flag = is.get();
    if (flag == std::char_traits<char>::eof()) throw nn_error("archive is empty");
    little = flag != 0;
  }
  auto bytes = [&](unsigned char *dst, size_t n) {
    is.read(reinterpret_cast<char *>(dst), static_cast<std::streamsize>(n));
    if (static_cast<size_t>(is.gcount()) != n) throw nn_error("archive ends inside a layer record");
  };
  auto u64 = [&]() {
    unsigned char b[8];
    bytes(b, 8);
    uint64_t v = 0;
    for (int i = 0; i < 8; ++i) v |= static_cast<uint64_t>(b[i]) << (8 * (little ? i : 7 - i));
    return v;
  };
  std::vector<archive_layer> out;
  for (size_t count : vector_counts) {
    archive_layer l;
    const uint64_t name_len = u64();
    if (name_len > 4096) throw nn_error("archive: a layer name of " + std::to_string(name_len) + " bytes");
    l.type.resize(name_len);
    if (name_len) bytes(reinterpret_cast<unsigned char *>(&l.type[0]), name_len);
    for (size_t k = 0; k < count; ++k) {
      const uint64_t n = u64();
      if (n > (uint64_t(1) << 32)) throw nn_error("archive: a weight vector of " + std::to_string(n) + " values");
      vec_t v(n);
      std::vector<unsigned char> raw(4 * n);
      if (n) bytes(raw.data(), raw.size());
      for (uint64_t i = 0; i < n; ++i) {
        const unsigned char *b = raw.data() + 4 * i;
        const uint32_t bits = little ? (uint32_t(b[0]) | uint32_t(b[1]) << 8 | uint32_t(b[2]) << 16 | uint32_t(b[3]) << 24)
                                     : (uint32_t(b[3]) | uint32_t(b[2]) << 8 | uint32_t(b[1]) << 16 | uint32_t(b[0]) << 24);
        std::memcpy(&v[i], &bits, 4);
      }
      l.vectors.push_back(std::move(v));
    }
    out.push_back(std::move(l));
  }
  return out;
}
}  // namespace detail

// ---- nodes / sequential (tiny_dnn/nodes.h:60-303): the layer-by-layer chain ----
// rvalues and shared_ptrs are kept alive by the container, lvalues are referred to, as in the
// reference. forward() writes the batch into the first layer's input edge, runs every layer's
// forward() and reads the last layer's output edge; backward() writes the loss gradient into
// the last layer's output edge and runs every layer's backward() back to front. Everything in
// between stays on the device (see class edge).
class nodes {
 public:
  typedef std::vector<layer *>::iterator iterator;
  typedef std::vector<layer *>::const_iterator const_iterator;
  virtual ~nodes() {}
  virtual void backward(const std::vector<tensor_t> &first) = 0;
  virtual std::vector<tensor_t> forward(const std::vector<tensor_t> &first) = 0;
  virtual void update_weights(optimizer *opt) {
    for (auto l : nodes_) l->update_weight(opt);
  }
  virtual void setup(bool reset_weight) {
    for (auto l : nodes_) l->setup(reset_weight);
  }
  void clear_grads() {
    for (auto l : nodes_) l->clear_grads();
  }
  size_t size() const { return nodes_.size(); }
  iterator begin() { return nodes_.begin(); }
  iterator end() { return nodes_.end(); }
  const_iterator begin() const { return nodes_.begin(); }
  const_iterator end() const { return nodes_.end(); }
  layer *operator[](size_t index) { return nodes_[index]; }
  const layer *operator[](size_t index) const { return nodes_[index]; }
  size_t in_data_size() const { return nodes_.front()->in_data_size(); }
  size_t out_data_size() const { return nodes_.back()->out_data_size(); }
  template <typename T>
  T &at(size_t index) {
    T *v = dynamic_cast<T *>(nodes_[index]);
    if (v) return *v;
    throw nn_error("failed to cast");
  }
  virtual float_t target_value_min(int = 0) const { return nodes_.back()->out_value_range().first; }
  virtual float_t target_value_max(int = 0) const { return nodes_.back()->out_value_range().second; }
  void label2vec(const label_t *t, size_t num, std::vector<vec_t> &vec) const {
    const size_t outdim = out_data_size();
    vec.reserve(num);
    for (size_t i = 0; i < num; i++) {
      if (t[i] >= outdim) throw nn_error("label out of range");
      vec.emplace_back(outdim, target_value_min());
      vec.back()[t[i]] = target_value_max();
    }
  }

 protected:
  template <typename T>
  void push_back(T &&node) {
    push_back_impl(std::forward<T>(node), typename std::is_rvalue_reference<decltype(node)>::type());
  }
  template <typename T>
  void push_back(std::shared_ptr<T> node) {
    own_nodes_.push_back(node);
    nodes_.push_back(own_nodes_.back().get());
  }
  // [sample][channel][feature] -> [channel][sample][feature] (nodes.h:228-250)
  void reorder_for_layerwise_processing(const std::vector<tensor_t> &input,
                                        std::vector<std::vector<const vec_t *>> &output) {
    const size_t sample_count = input.size(), channel_count = input[0].size();
    output.resize(channel_count);
    for (size_t i = 0; i < channel_count; ++i) output[i].resize(sample_count);
    for (size_t sample = 0; sample < sample_count; ++sample) {
      if (input[sample].size() != channel_count) throw nn_error("samples with different channel counts");
      for (size_t channel = 0; channel < channel_count; ++channel) output[channel][sample] = &input[sample][channel];
    }
  }
  template <typename T>
  void push_back_impl(T &&node, std::true_type) {
    own_nodes_.push_back(std::make_shared<typename std::remove_reference<T>::type>(std::forward<T>(node)));
    nodes_.push_back(own_nodes_.back().get());
  }
  template <typename T>
  void push_back_impl(T &&node, std::false_type) {
    nodes_.push_back(&node);
  }
  std::vector<std::shared_ptr<layer>> own_nodes_;
  std::vector<layer *> nodes_;
};

class sequential : public nodes {
 public:
  void backward(const std::vector<tensor_t> &first) override {
    std::vector<std::vector<const vec_t *>> reordered_grad;
    reorder_for_layerwise_processing(first, reordered_grad);
    if (reordered_grad.size() != 1) throw nn_error("sequential::backward: one output channel expected");
    nodes_.back()->set_out_grads(&reordered_grad[0], 1);
    for (auto l = nodes_.rbegin(); l != nodes_.rend(); l++) (*l)->backward();
  }
  std::vector<tensor_t> forward(const std::vector<tensor_t> &first) override {
    std::vector<std::vector<const vec_t *>> reordered_data;
    reorder_for_layerwise_processing(first, reordered_data);
    if (reordered_data.size() != 1) throw nn_error("sequential::forward: one input channel expected");
    nodes_.front()->set_in_data(&reordered_data[0], 1);
    for (auto l : nodes_) l->forward();
    std::vector<const tensor_t *> out;
    nodes_.back()->output(out);
    // back to [sample][layer][feature] (nodes.h:346-359)
    const size_t sample_count = first.size();  // (the edge may hold more rows than this batch)
    std::vector<tensor_t> normalized_output(sample_count, tensor_t(1));
    for (size_t sample = 0; sample < sample_count; ++sample) normalized_output[sample][0] = (*out[0])[sample];
    return normalized_output;
  }
  template <typename T>
  void add(T &&layer) {
    push_back(std::forward<T>(layer));
    if (nodes_.size() != 1) connect(nodes_[nodes_.size() - 2], nodes_[nodes_.size() - 1], 0, 0);
    check_connectivity();
  }
  void check_connectivity() {
    for (size_t i = 0; i + 1 < nodes_.size(); i++)
      if (nodes_[i]->outputs()[0] != nodes_[i + 1]->inputs()[0]) throw nn_error("");
  }
};

enum grad_check_mode { GRAD_CHECK_ALL, GRAD_CHECK_RANDOM };  // tiny_dnn/util/util.h:68-69

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

  // How a step runs. fused (the default): the layers are described to one device-resident
  // tdh_net whose whole train step is fused and replayed as a HIP graph. layer_by_layer: the
  // reference's own loop (tiny_dnn/network.h:169-213, 840-926, nodes.h:276-303): every layer's
  // forward() / backward() marshals its edges' tensors into OpKernel::compute, the loss gradient
  // is computed on the host from the net's output, and layer::update_weight hands gradients and
  // weights to optimizer::update; the tensors stay on the device between the layers either way.
  // Each mode keeps its own copy of the weights: choose before weights are set or drawn.
  enum class execution { fused, layer_by_layer };
  void set_execution(execution mode) {
    if (mode != mode_ && initialized_) throw nn_error("set_execution: choose the mode before weights are set");
    mode_ = mode;
  }
  execution get_execution() const { return mode_; }
  // the chain of layer_by_layer execution (the layers of this network, connected by edges)
  sequential &chain() {
    if (chain_.size() != layers_.size()) {
      if (chain_.size()) throw nn_error("layers were added after the layer-by-layer chain was built");
      for (auto &l : layers_) chain_.add(*l);
    }
    return chain_;
  }
  size_t layer_size() const { return layers_.size(); }
  size_t depth() const { return layer_size(); }
  const layer *operator[](size_t index) const { return layers_[index].get(); }

  size_t in_data_size() {
    return mode_ == execution::layer_by_layer ? chain().in_data_size() : (build(1), tdh_net_in_size(net_));
  }
  size_t out_data_size() {
    return mode_ == execution::layer_by_layer ? chain().out_data_size() : (build(1), tdh_net_out_size(net_));
  }

  // trainable tensors of layer `index`: which = 0 weight, 1 bias
  vec_t weights(size_t index, int which) {
    if (mode_ == execution::layer_by_layer) {  // the edge's vector, at its declared length
      chain().setup(false);
      const layer &l = *layers_[index];
      const std::vector<const vec_t *> w = l.weights();
      return static_cast<size_t>(which) < w.size() ? *w[which] : vec_t();
    }
    build(max_batch_ ? max_batch_ : 1);
    vec_t v(tdh_net_param_size(net_, static_cast<int>(index), which));
    detail::check(tdh_net_get_param(net_, static_cast<int>(index), which, v.data()));
    return v;
  }
  void set_weights(size_t index, int which, const vec_t &v) {
    if (mode_ == execution::layer_by_layer) {
      chain().setup(false);
      const std::vector<vec_t *> w = layers_[index]->weights();
      if (static_cast<size_t>(which) >= w.size() || v.size() > w[which]->size()) throw nn_error("set_weights: size mismatch");
      std::copy(v.begin(), v.end(), w[which]->begin());  // (a used prefix of an average-pooling vector is enough)
      initialized_ = true;
      return;
    }
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
    return fit<Error>(opt, inputs, desired_outputs, batch_size, epoch, on_batch_enumerate,
                      on_epoch_enumerate, /*reset_weights=*/false);
  }
  // reset_weights: network::fit's argument of that name (tiny_dnn/network.h:368-386); weights
  // that have never been set or initialised are drawn by init_weight either way (:852-853,
  // layer::setup, tiny_dnn/layers/layer.h:584-614)
  template <typename Error, typename Optimizer, typename OnBatch, typename OnEpoch>
  bool fit(Optimizer &opt, const std::vector<vec_t> &inputs, const std::vector<vec_t> &desired_outputs,
           size_t batch_size, int epoch, OnBatch on_batch_enumerate, OnEpoch on_epoch_enumerate,
           bool reset_weights) {
    if (inputs.size() != desired_outputs.size() || inputs.empty() || batch_size == 0) return false;
    if (mode_ == execution::layer_by_layer)
      return fit_layer_by_layer<Error>(opt, inputs, desired_outputs, batch_size, epoch, on_batch_enumerate,
                                       on_epoch_enumerate, reset_weights);
    build(batch_size);
    if (reset_weights || !initialized_) init_weight();
    const size_t in_len = tdh_net_in_size(net_), out_len = tdh_net_out_size(net_);
    set_netphase(net_phase::train);  // network.h:852
    opt.reset();  // network.h:856; the device copy of the state vectors is cleared with it
    detail::check(tdh_net_reset_optimizer(net_));
    tdh_opt o = opt.descriptor();
    // batches travel two ahead: while a step runs, the batch after it is being uploaded and the
    // one after that flattened and copied to pinned memory
    detail::feeder feed(in_len, out_len, batch_size);
    const size_t per_epoch = (inputs.size() + batch_size - 1) / batch_size;
    const size_t total     = per_epoch * static_cast<size_t>(epoch);
    auto stage = [&](size_t k) {
      const size_t i = (k % per_epoch) * batch_size;
      const size_t n = std::min(batch_size, inputs.size() - i);
      feed.stage(inputs, desired_outputs, i, n);
    };
    if (total) stage(0);
    if (total > 1) stage(1);
    for (size_t k = 0; k < total; ++k) {
      const float *xd = nullptr, *td = nullptr;
      int n = 0;
      detail::check(tdh_feeder_acquire(feed.get(), &xd, &td, &n));
      if (k + 2 < total) stage(k + 2);  // the feeder's thread copies and uploads while this one launches
      draw_dropout_masks(static_cast<size_t>(n));
      detail::check(tdh_net_train_step(net_, &o, Error::kind, n, xd, td, 1));
      on_batch_enumerate();
      if ((k + 1) % per_epoch == 0) on_epoch_enumerate();
    }
    opt.absorb(o);
    set_netphase(net_phase::test);  // network.h:877
    return true;
  }

  // network::set_netphase (tiny_dnn/network.h:438-442)
  void set_netphase(net_phase phase) {
    if (mode_ == execution::layer_by_layer) {
      phase_ = phase;
      for (auto &l : layers_) l->set_context(phase);
      return;
    }
    build(max_batch_ ? max_batch_ : 1);
    phase_ = phase;
    detail::check(tdh_net_set_phase(net_, phase == net_phase::train));
  }

  // network::train (tiny_dnn/network.h:284-308): labels become one-hot targets whose off / on
  // values are the last layer's out_value_range (nodes::label2vec, tiny_dnn/nodes.h:180-189)
  template <typename Error, typename Optimizer>
  bool train(Optimizer &opt, const std::vector<vec_t> &inputs, const std::vector<label_t> &class_labels,
             size_t batch_size, int epoch) {
    if (inputs.size() != class_labels.size() || inputs.size() < batch_size) return false;
    if (mode_ != execution::layer_by_layer) build(batch_size);
    const size_t out_len = out_data_size();
    const std::pair<float_t, float_t> range = layers_.back()->out_value_range();
    std::vector<vec_t> t(class_labels.size(), vec_t(out_len, range.first));
    for (size_t i = 0; i < class_labels.size(); ++i) {
      if (class_labels[i] >= out_len) throw nn_error("label out of range");
      t[i][class_labels[i]] = range.second;
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
      for (int which = 0; which < 4; ++which) {  // 2, 3: a batch-norm layer's running averages
        const vec_t v = weights(i, which);       // (batch_normalization_layer.h:179-189)
        for (float_t w : v) os << w << " ";
        for (size_t k = v.size(); k < file_length(i, which); ++k) os << float_t(0) << " ";
      }
  }
  void load(std::istream &is) {
    build(max_batch_ ? max_batch_ : 1);
    for (size_t i = 0; i < layers_.size(); ++i)
      for (int which = 0; which < 4; ++which) {
        vec_t v(tdh_net_param_size(net_, static_cast<int>(i), which));
        for (float_t &w : v) is >> w;
        float_t skipped;
        for (size_t k = v.size(); k < file_length(i, which); ++k) is >> skipped;
        if (is.fail()) throw nn_error("load: the stream holds fewer weights than the network");
        if (!v.empty()) set_weights(i, which, v);
      }
    initialized_ = true;
  }
  // network::save / load (tiny_dnn/network.h:676-728) with the reference's arguments and
  // defaults. content_type::weights in binary or portable_binary is read and written, byte for
  // byte the reference's files; the model description (content_type::model and the default
  // weights_and_model) and json are not part of this library and raise nn_error.
  void save(const std::string &filename, content_type what = content_type::weights_and_model,
            file_format format = file_format::binary) {
    require_weights_archive(what, format);
    build(max_batch_ ? max_batch_ : 1);
    std::vector<detail::archive_layer> layers(layers_.size());
    for (size_t i = 0; i < layers_.size(); ++i) {
      layers[i].type = layers_[i]->archive_type_name();
      for (int which = 0; which < 2; ++which) {
        vec_t v = weights(i, which);
        if (v.empty()) continue;
        v.resize(file_length(i, which), float_t(0));
        layers[i].vectors.push_back(std::move(v));
      }
    }
    std::ofstream ofs(filename.c_str(), std::ios::binary | std::ios::out);
    if (ofs.fail() || ofs.bad()) throw nn_error("failed to open:" + filename);
    detail::write_weight_archive(ofs, layers, format);
  }
  void load(const std::string &filename, content_type what = content_type::weights_and_model,
            file_format format = file_format::binary) {
    require_weights_archive(what, format);
    std::ifstream ifs(filename.c_str(), std::ios::binary | std::ios::in);
    if (ifs.fail() || ifs.bad()) throw nn_error("failed to open:" + filename);
    build(max_batch_ ? max_batch_ : 1);
    std::vector<size_t> counts(layers_.size(), 0);
    for (size_t i = 0; i < layers_.size(); ++i)
      for (int which = 0; which < 2; ++which)
        if (tdh_net_param_size(net_, static_cast<int>(i), which)) ++counts[i];
    const std::vector<detail::archive_layer> layers = detail::read_weight_archive(ifs, counts, format);
    for (size_t i = 0; i < layers_.size(); ++i) {
      size_t k = 0;
      for (int which = 0; which < 2; ++which) {
        const size_t n = tdh_net_param_size(net_, static_cast<int>(i), which);
        if (!n) continue;
        const vec_t &v = layers[i].vectors[k++];
        if (v.size() != file_length(i, which))
          throw nn_error("load: layer " + std::to_string(i) + " of the archive holds " + std::to_string(v.size()) +
                         " values, the network's " + std::to_string(file_length(i, which)));
        set_weights(i, which, vec_t(v.begin(), v.begin() + n));
      }
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
      for (int which = 0; which < 4; ++which) {
        const size_t n = tdh_net_param_size(net_, static_cast<int>(i), which), len = file_length(i, which);
        if (idx + len > data.size()) throw nn_error("fast_load: the file holds fewer weights than the network");
        if (n) set_weights(i, which, vec_t(data.begin() + idx, data.begin() + idx + n));
        idx += len;
      }
    initialized_ = true;
  }

  // network::init_weight (tiny_dnn/network.h:165) -> layer::init_weight
  // (tiny_dnn/layers/layer.h:625-655): layers front to back, weight before bias, each filled
  // by the layer's weight_init / bias_init function with the layer's fan sizes
  void init_weight() {
    if (mode_ == execution::layer_by_layer) {
      chain().setup(true);
      initialized_ = true;
      return;
    }
    build(max_batch_ ? max_batch_ : 1);
    for (size_t i = 0; i < layers_.size(); ++i) {
      layer &l = *layers_[i];
      for (int which = 0; which < 2; ++which) {
        const size_t n = tdh_net_param_size(net_, static_cast<int>(i), which);
        if (!n) continue;
        vec_t v(which == 0 ? l.declared_weight_size(n) : n);
        (which == 0 ? l.weight_init_fn() : l.bias_init_fn())->fill(&v, l.fan_in_size(), l.fan_out_size());
        v.resize(n);
        detail::check(tdh_net_set_param(net_, static_cast<int>(i), which, v.data()));
      }
    }
    initialized_ = true;
  }

  // network::fprop (tiny_dnn/network.h:184-204): a forward pass of the given samples; the batch
  // stays on the device as the one bprop works on
  vec_t fprop(const vec_t &in) { return fprop(std::vector<vec_t>{in})[0]; }
  std::vector<vec_t> fprop(const std::vector<vec_t> &in) {
    if (in.empty()) return {};
    if (mode_ == execution::layer_by_layer) {
      if (!initialized_) init_weight();
      std::vector<tensor_t> batch(in.size());
      for (size_t s = 0; s < in.size(); ++s) batch[s] = tensor_t{in[s]};
      const std::vector<tensor_t> y = chain().forward(batch);
      std::vector<vec_t> out(y.size());
      for (size_t s = 0; s < y.size(); ++s) out[s] = y[s][0];
      last_batch_ = in.size();
      return out;
    }
    build(std::max(in.size(), max_batch_ ? max_batch_ : 1));
    if (!initialized_) init_weight();
    const size_t in_len = tdh_net_in_size(net_), out_len = tdh_net_out_size(net_);
    for (const vec_t &v : in)
      if (v.size() != in_len) throw nn_error("input dimension mismatch");
    last_batch_ = in.size();
    detail::check(tdh_net_forward(net_, static_cast<int>(in.size()), x_.upload(in, in.size(), in_len)));
    std::vector<float> flat(in.size() * out_len);
    detail::check(tdh_memcpy_d2h(flat.data(), tdh_net_layer_out(net_, static_cast<int>(layers_.size()) - 1),
                                 flat.size() * sizeof(float)));
    std::vector<vec_t> out(in.size());
    for (size_t s = 0; s < in.size(); ++s) out[s].assign(flat.begin() + s * out_len, flat.begin() + (s + 1) * out_len);
    return out;
  }
  std::vector<tensor_t> fprop(const std::vector<tensor_t> &in) {  // one channel, as calc_delta asserts
    std::vector<vec_t> flat_in;
    for (const tensor_t &t : in) flat_in.push_back(t.at(0));
    const std::vector<vec_t> y = fprop(flat_in);
    std::vector<tensor_t> out(y.size());
    for (size_t s = 0; s < y.size(); ++s) out[s] = tensor_t{y[s]};
    return out;
  }

  // network::bprop (tiny_dnn/network.h:169-182): the loss gradient for targets t and the
  // backward pass through every layer, on the batch of the last fprop; weight and bias
  // gradients are ADDED to what is there (cleared by update_weights / clear_grads). `out` is
  // what fprop returned: the device still holds it, so it is not sent back.
  template <typename E>
  void bprop(const std::vector<vec_t> &out, const std::vector<vec_t> &t) {
    if (mode_ == execution::layer_by_layer) {  // network.h:169-182
      if (!last_batch_ || out.size() != last_batch_ || t.size() != last_batch_)
        throw nn_error("bprop: call fprop on the same batch first");
      std::vector<tensor_t> delta(out.size());
      for (size_t s = 0; s < out.size(); ++s) delta[s] = tensor_t{gradient<E>(out[s], t[s])};
      chain().backward(delta);
      return;
    }
    if (!net_ || !last_batch_ || out.size() != last_batch_ || t.size() != last_batch_)
      throw nn_error("bprop: call fprop on the same batch first");
    const size_t out_len = tdh_net_out_size(net_);
    detail::check(tdh_net_train_step(net_, nullptr, E::kind, static_cast<int>(last_batch_), x_.get(),
                                     t_.upload(t, t.size(), out_len), /*do_update=*/0));
  }
  template <typename E>
  void bprop(const std::vector<tensor_t> &out, const std::vector<tensor_t> &t, const std::vector<tensor_t> &) {
    std::vector<vec_t> o, tt;
    for (const tensor_t &v : out) o.push_back(v.at(0));
    for (const tensor_t &v : t) tt.push_back(v.at(0));
    bprop<E>(o, tt);
  }

  // network::update_weights (tiny_dnn/network.h:209-213): every layer's update_weight, then
  // the gradients are clear
  template <typename Optimizer>
  void update_weights(Optimizer *opt) {
    if (mode_ == execution::layer_by_layer) {
      chain().update_weights(opt);
      return;
    }
    build(max_batch_ ? max_batch_ : 1);
    tdh_opt o = opt->descriptor();
    detail::check(tdh_net_update_weights(net_, &o));
    opt->absorb(o);
  }
  void clear_grads() {
    if (mode_ == execution::layer_by_layer) chain().clear_grads();
    else if (net_) detail::check(tdh_net_clear_grads(net_));
  }
  // batch-reduced gradient of layer `index` (which = 0 weight, 1 bias) since the last update
  vec_t weights_grads(size_t index, int which) {
    build(max_batch_ ? max_batch_ : 1);
    vec_t v(tdh_net_param_size(net_, static_cast<int>(index), which));
    if (!v.empty())
      detail::check(tdh_memcpy_d2h(v.data(), tdh_net_layer_grad(net_, static_cast<int>(index), which),
                                   v.size() * sizeof(float)));
    return v;
  }

  // network::train_once / train_onebatch (tiny_dnn/network.h:887-926): fprop, bprop and
  // update_weights of `size` samples as one mini-batch
  template <typename E, typename Optimizer>
  void train_once(Optimizer &opt, const vec_t *in, const vec_t *t, size_t size) {
    if (mode_ == execution::layer_by_layer) {  // network.h:887-926
      const std::vector<vec_t> xs(in, in + size), ts(t, t + size);
      bprop<E>(fprop(xs), ts);
      chain().update_weights(&opt);
      return;
    }
    build(std::max(size, max_batch_ ? max_batch_ : 1));
    if (!initialized_) init_weight();
    const size_t in_len = tdh_net_in_size(net_), out_len = tdh_net_out_size(net_);
    const std::vector<vec_t> xs(in, in + size), ts(t, t + size);
    tdh_opt o = opt.descriptor();
    last_batch_ = size;
    draw_dropout_masks(size);
    detail::check(tdh_net_train_step(net_, &o, E::kind, static_cast<int>(size), x_.upload(xs, size, in_len),
                                     t_.upload(ts, size, out_len), 1));
    opt.absorb(o);
  }

  // network::get_loss (tiny_dnn/network.h:486-497): sum of E::f over the samples
  template <typename E>
  float_t get_loss(const std::vector<vec_t> &in, const std::vector<vec_t> &t) {
    float_t sum_loss = float_t(0);
    const std::vector<vec_t> y = fprop(in);
    for (size_t i = 0; i < in.size(); ++i) sum_loss += E::f(y[i], t[i]);
    return sum_loss;
  }

  // network::gradient_check (tiny_dnn/network.h:541-590, calc_delta :939-989): for every
  // trainable vector, the loss's central difference in single weights (step sqrt(float
  // epsilon)) against the gradient the backward pass gives, all (GRAD_CHECK_ALL) or ten random
  // entries of each vector (GRAD_CHECK_RANDOM, drawn like the reference's uniform_idx).
  // Samples are one-channel tensors, labels become targets through label2vec.
  template <typename E>
  bool gradient_check(const std::vector<tensor_t> &in, const std::vector<std::vector<label_t>> &t,
                      float_t eps, grad_check_mode mode) {
    if (in.size() != t.size() || in.empty()) throw nn_error("gradient_check: bad sample set");
    std::vector<vec_t> x, v;
    build(std::max(in.size(), max_batch_ ? max_batch_ : 1));
    if (!initialized_) init_weight();
    const size_t out_len = tdh_net_out_size(net_);
    for (size_t s = 0; s < in.size(); ++s) {
      x.push_back(in[s].at(0));
      const std::pair<float_t, float_t> range = layers_.back()->out_value_range();
      vec_t target(out_len, range.first);
      if (t[s].at(0) >= out_len) throw nn_error("label out of range");
      target[t[s][0]] = range.second;
      v.push_back(target);
    }
    for (size_t i = 0; i < layers_.size(); ++i) {
      for (int which = 0; which < 2; ++which) {
        const size_t n = tdh_net_param_size(net_, static_cast<int>(i), which);
        if (!n) continue;
        if (mode == GRAD_CHECK_ALL) {
          for (size_t j = 0; j < n; ++j)
            if (!calc_delta<E>(x, v, i, which, j, eps)) return false;
        } else if (mode == GRAD_CHECK_RANDOM) {
          for (size_t k = 0; k < 10; ++k) {
            std::uniform_int_distribution<int> dst(0, static_cast<int>(n) - 1);
            if (!calc_delta<E>(x, v, i, which, static_cast<size_t>(dst(random_generator::get_instance()())), eps))
              return false;
          }
        } else {
          throw nn_error("unknown grad-check type");
        }
      }
    }
    return true;
  }
  // the two figures of the last calc_delta (for reports)
  float_t last_numeric_gradient() const { return last_numeric_; }
  float_t last_bprop_gradient() const { return last_bprop_; }

  // network::predict (tiny_dnn/network.h:226-230)
  vec_t predict(const vec_t &in) {
    if (mode_ == execution::layer_by_layer) return fprop(in);
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
  // network::fit on the layer chain (tiny_dnn/network.h:840-879): setup, train phase, optimizer
  // reset, epochs over mini-batches of train_once, test phase
  template <typename Error, typename Optimizer, typename OnBatch, typename OnEpoch>
  bool fit_layer_by_layer(Optimizer &opt, const std::vector<vec_t> &inputs, const std::vector<vec_t> &desired_outputs,
                          size_t batch_size, int epoch, OnBatch on_batch_enumerate, OnEpoch on_epoch_enumerate,
                          bool reset_weights) {
    if (reset_weights || !initialized_) init_weight();
    else chain().setup(false);
    set_netphase(net_phase::train);
    opt.reset();
    for (int iter = 0; iter < epoch; iter++) {
      for (size_t i = 0; i < inputs.size(); i += batch_size) {
        train_once<Error>(opt, &inputs[i], &desired_outputs[i], std::min(batch_size, inputs.size() - i));
        on_batch_enumerate();
      }
      on_epoch_enumerate();
    }
    set_netphase(net_phase::test);
    return true;
  }
  // dropout_layer::forward_propagation in the train phase (dropout_layer.h:99-102): every
  // element of every sample of every dropout layer, front to back, draws its own
  // bernoulli(rate) from the process-wide generator; the masks are handed to the device net
  void draw_dropout_masks(size_t n) {
    if (phase_ != net_phase::train) return;
    for (size_t i = 0; i < layers_.size(); ++i) {
      const dropout_layer *d = dynamic_cast<const dropout_layer *>(layers_[i].get());
      if (!d) continue;
      const size_t len = tdh_net_layer_out_size(net_, static_cast<int>(i));
      mask_.resize(n * len);
      for (size_t e = 0; e < n * len; ++e) mask_[e] = bernoulli(d->dropout_rate());
      detail::check(tdh_net_set_dropout_mask(net_, static_cast<int>(i), static_cast<int>(n), mask_.data()));
    }
  }
  template <typename E>
  bool calc_delta(const std::vector<vec_t> &x, const std::vector<vec_t> &v, size_t layer_index, int which,
                  size_t check_index, double eps) {
    static const float_t delta = std::sqrt(std::numeric_limits<float_t>::epsilon());
    clear_grads();
    vec_t w = weights(layer_index, which);
    const float_t prev_w = w[check_index];
    w[check_index] = prev_w + delta;
    set_weights(layer_index, which, w);
    float_t f_p = float_t(0);
    for (size_t i = 0; i < x.size(); ++i) f_p += get_loss<E>({x[i]}, {v[i]});
    w[check_index] = prev_w - delta;
    set_weights(layer_index, which, w);
    float_t f_m = float_t(0);
    for (size_t i = 0; i < x.size(); ++i) f_m += get_loss<E>({x[i]}, {v[i]});
    const float_t delta_by_numerical = (f_p - f_m) / (float_t(2) * delta);
    w[check_index] = prev_w;
    set_weights(layer_index, which, w);
    bprop<E>(fprop(x), v);
    const float_t delta_by_bprop = weights_grads(layer_index, which)[check_index];
    clear_grads();
    last_numeric_ = delta_by_numerical;
    last_bprop_   = delta_by_bprop;
    return std::abs(delta_by_bprop - delta_by_numerical) <= eps;
  }
  static void require_weights_archive(content_type what, file_format format) {
    if (what != content_type::weights)
      throw nn_error("save/load: only content_type::weights is built; the model description is not part of "
                     "this library");
    if (format == file_format::json) throw nn_error("save/load: json archives are not built");
    if (format != file_format::binary && format != file_format::portable_binary)
      throw nn_error("invalid serialization format");
  }
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
                                 TDH_NET_FUSE_ACT_GRAD | TDH_NET_GRAPH | TDH_NET_SAMPLE_STEP, &fresh));
    if (net_) {
      for (size_t i = 0; i < layers_.size(); ++i)
        for (int which = 0; which < 4; ++which) {
          vec_t v(tdh_net_param_size(net_, static_cast<int>(i), which));
          if (v.empty()) continue;
          detail::check(tdh_net_get_param(net_, static_cast<int>(i), which, v.data()));
          detail::check(tdh_net_set_param(fresh, static_cast<int>(i), which, v.data()));
        }
      tdh_net_destroy(net_);
    }
    detail::check(tdh_net_set_phase(fresh, phase_ == net_phase::train));
    net_       = fresh;
    max_batch_ = batch;
  }

  std::vector<std::unique_ptr<layer>> layers_;
  execution mode_ = execution::fused;
  sequential chain_;
  tdh_net *net_     = nullptr;
  size_t max_batch_ = 0;
  bool initialized_ = false;
  net_phase phase_ = net_phase::train;   // a new net is in the train phase (layer constructors' default)
  std::vector<uint8_t> mask_;
  size_t last_batch_ = 0;                // samples of the last fprop / train_once, held in x_
  float_t last_numeric_ = 0, last_bprop_ = 0;
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
