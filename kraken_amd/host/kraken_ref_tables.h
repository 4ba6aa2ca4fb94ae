// The drop-in itself: kraken::Table subclasses over the C ABI (include/kraken_hip.h), written
// against the REFERENCE's own headers (kraken/ps/table.h, ps/optim/optim.h,
// ps/initializer/initializer.h, t/tensor.h), which must be on the include path. This is the file a
// Kraken maintainer adds to the tree; kraken_gpu_tables.h is the same code over a minimal Tensor
// for builds that have no Kraken tree.
//
// Nothing here throws, whatever the device does: the reference's server threads catch nothing
// (common/exception.h:13-31 is only thrown by tensor misuse), so every failure is an ErrorCode.
#pragma once

#include <cstring>
#include <memory>
#include <mutex>
#include <string>
#include <unordered_map>
#include <vector>

#include "common/error_code.h"
#include "kraken_hip.h"
#include "ps/initializer/initializer.h"
#include "ps/optim/optim.h"
#include "ps/table.h"
#include "t/element_type.h"
#include "t/shape.h"
#include "t/storage.h"
#include "t/tensor.h"

namespace kraken {

// [integration:begin]
// The model's optimizer for GPU tables (created where Ps::CreateModel calls Optim::Create,
// ps/ps.cc:604-633): the reference's Adagrad / Adam / RMSprop / SGD keep their hyper-parameters
// private, so the same conf map is parsed into the C ABI's krk_optim (krk_optim_set follows
// ps/optim/optim.cc:23-101 key by key). A GPU table never calls Update: the update runs on the
// device, fused with the row access.
class GpuOptim : public Optim {
  krk_optim raw_;

 public:
  GpuOptim(OptimType optim_type, const krk_optim& raw) : Optim(optim_type), raw_(raw) {}
  int32_t Update(const Tensor&, float, Value*) const override { return ErrorCode::kInterfaceUnImplementError; }
  const krk_optim* raw() const { return &raw_; }

  static std::unique_ptr<Optim> Create(OptimType optim_type,
                                       const std::unordered_map<std::string, std::string>& optim_conf) {
    std::unique_ptr<Optim> optim;
    krk_optim raw;
    if (krk_optim_defaults((int32_t)optim_type, &raw) != KRK_SUCCESS) return optim;   // as Optim::Create: null
    for (const auto& kv : optim_conf) krk_optim_set(&raw, kv.first.c_str(), kv.second.c_str());
    optim.reset(new GpuOptim(optim_type, raw));
    return optim;
  }
};

// null when `optim` is one of the reference's CPU optimizers: the table then answers 6
inline const krk_optim* ToKrkOptim(Optim* optim) {
  const GpuOptim* g = dynamic_cast<const GpuOptim*>(optim);
  return g ? g->raw() : nullptr;
}

// Page-locked host blocks for replies and gradients. A reply's rows are views of one such block,
// which the GPU writes across PCIe in place (no device-side staging, no pageable copy: a pull of
// 8192 rows of 16 floats takes 27 us instead of 58); the block goes back to the pool when the last
// Tensor of the reply is gone. Blocks are powers of two from 64 KB. Page-locking and releasing
// memory takes milliseconds and waits for the device, so the request path should almost never do
// either: a request takes the smallest idle block that holds it (up to eight times its size, so
// that requests of varying size share blocks), and the pool keeps idle blocks up to kMaxIdleBytes
// in all and kMaxIdlePerSize of one size; beyond that a returned block is released.
class PinnedPool {
  static constexpr size_t kMinBlock = 64 * 1024;
  static constexpr size_t kMaxIdleBytes = (size_t)1 << 30;
  static constexpr int kMaxIdlePerSize = 8;
  std::mutex mu_;
  std::vector<std::pair<void*, size_t>> free_;
  size_t idle_bytes_ = 0;

 public:
  ~PinnedPool() {
    for (auto& b : free_) krk_host_free(b.first);
  }
  // nullptr when page-locked memory cannot be had: the caller falls back to ordinary memory
  void* Take(size_t bytes, size_t* size) {
    size_t want = kMinBlock;
    while (want < bytes) want <<= 1;
    {
      std::lock_guard<std::mutex> lk(mu_);
      size_t best = free_.size();
      for (size_t i = 0; i < free_.size(); ++i) {
        const size_t have = free_[i].second;
        if (have >= want && have <= 8 * want && (best == free_.size() || have < free_[best].second)) best = i;
      }
      if (best != free_.size()) {
        void* p = free_[best].first;
        *size = free_[best].second;
        idle_bytes_ -= *size;
        free_[best] = free_.back();
        free_.pop_back();
        return p;
      }
    }
    void* p = nullptr;
    if (krk_host_malloc(&p, want) != KRK_SUCCESS) return nullptr;
    *size = want;
    return p;
  }
  void Give(void* p, size_t size) {
    {
      std::lock_guard<std::mutex> lk(mu_);
      int same = 0;
      for (auto& b : free_) same += b.second == size;
      if (same < kMaxIdlePerSize && idle_bytes_ + size <= kMaxIdleBytes) {
        free_.emplace_back(p, size);
        idle_bytes_ += size;
        return;
      }
    }
    krk_host_free(p);
  }
};

class GpuSparseTable : public Table {
  // a reply's block and the Storage that presents it to Tensors, returned to the pool together
  struct Reply {
    std::shared_ptr<PinnedPool> pool;
    void* block = nullptr;
    size_t size = 0;
    std::shared_ptr<Storage> storage;
    ~Reply() {
      if (block) pool->Give(block, size);
    }
  };
  std::shared_ptr<PinnedPool> pool_ = std::make_shared<PinnedPool>();
  int64_t dimension_;
  ElementType element_type_;
  std::unique_ptr<Initializer> initializer_;   // kept for conf() / checkpoint metadata
  krk_sparse* h_ = nullptr;
  int32_t create_rc_ = ErrorCode::kSuccess;

 public:
  GpuSparseTable(uint64_t id, const std::string& name, int64_t dimension, ElementType element_type,
                 std::unique_ptr<Initializer>&& initializer)
      : Table(TableType::kSparse, id, name),
        dimension_(dimension),
        element_type_(element_type),
        initializer_(std::move(initializer)) {
    krk_init ki;
    create_rc_ = krk_init_defaults((int32_t)initializer_->type(), &ki);
    if (create_rc_ != KRK_SUCCESS) return;
    for (const auto& kv : initializer_->conf()) krk_init_set(&ki, kv.first.c_str(), kv.second.c_str());
    // the engine holds fp32 rows; another element type is refused at the first call
    create_rc_ = element_type_.Is<float>() ? krk_sparse_create(dimension, &ki, /*capacity_hint=*/0, &h_)
                                           : ErrorCode::kSparseTableUnCompatibleError;
  }
  ~GpuSparseTable() override { krk_sparse_destroy(h_); }

  int64_t dimension() const { return dimension_; }
  ElementType element_type() const { return element_type_; }
  Initializer* initializer() const { return initializer_.get(); }
  krk_sparse* handle() const { return h_; }   // for the users of SparseTable::mutable_vals()

  int32_t Pull(const std::vector<uint64_t>& sparse_ids, std::vector<Tensor>* vals) override {
    if (!h_) return create_rc_;
    // one contiguous [n, dimension] buffer; each returned Tensor is a row view of it
    // (Tensor::Dense(shape, storage, byte offset, etype), t/tensor.h:58-59), so the serializer
    // sees the same vector<Tensor> as before without an allocation and a copy per row
    const size_t row_bytes = (size_t)dimension_ * sizeof(float);
    const size_t bytes = sparse_ids.size() * row_bytes + sizeof(float);
    std::shared_ptr<Storage> storage;
    auto reply = std::make_shared<Reply>();
    reply->pool = pool_;
    reply->block = pool_->Take(bytes, &reply->size);
    if (reply->block) {
      reply->storage = Storage::From(reply->block, reply->size);   // t/storage.h:42: memory it does not own
      storage = std::shared_ptr<Storage>(reply, reply->storage.get());   // keeps the block until the last row is gone
    } else {
      storage = Storage::Create(bytes);
    }
    const int32_t rc = krk_sparse_pull(h_, sparse_ids.data(), (int64_t)sparse_ids.size(),
                                       static_cast<float*>(storage->ptr()), 0);
    if (rc != ErrorCode::kSuccess) return rc;
    vals->clear();
    vals->reserve(sparse_ids.size());
    const Shape row_shape(std::vector<int64_t>{dimension_});
    for (size_t i = 0; i < sparse_ids.size(); ++i)
      vals->emplace_back(Tensor::Dense(row_shape, storage, i * row_bytes, element_type_));
    return ErrorCode::kSuccess;
  }

  int32_t Push(Optim* optim, const std::vector<uint64_t>& sparse_ids, const std::vector<Tensor>& grads,
               float lr) override {
    if (!h_) return create_rc_;
    const krk_optim* o = ToKrkOptim(optim);
    if (!o) return ErrorCode::kUnSupportOptimTypeError;
    if (grads.size() != sparse_ids.size()) return ErrorCode::kGradientUnCompatibleError;
    // the rows are gathered into one page-locked block, which the GPU reads in place
    const size_t bytes = sparse_ids.size() * (size_t)dimension_ * sizeof(float) + sizeof(float);
    Reply staged;
    staged.pool = pool_;
    staged.block = pool_->Take(bytes, &staged.size);
    std::vector<float> pageable;
    float* flat = static_cast<float*>(staged.block);
    if (!flat) {
      pageable.resize(sparse_ids.size() * (size_t)dimension_ + 1);
      flat = pageable.data();
    }
    for (size_t i = 0; i < sparse_ids.size(); ++i) {
      // ps/optim/adagrad.cc:29-32 and its siblings: a dense gradient of the row's size and type
      if (!grads[i].IsDense() || grads[i].Size() != dimension_ || grads[i].element_type() != element_type_)
        return ErrorCode::kGradientUnCompatibleError;
      std::memcpy(flat + i * (size_t)dimension_, grads[i].Ptr(), (size_t)dimension_ * sizeof(float));
    }
    return krk_sparse_push(h_, o, sparse_ids.data(), (int64_t)sparse_ids.size(), flat, dimension_, lr, 0);
  }
};

class GpuDenseTable : public Table {
  Shape shape_;
  ElementType element_type_;
  krk_dense* h_ = nullptr;
  int32_t create_rc_ = ErrorCode::kSuccess;

 public:
  // ps/dense_table.cc:10-13: the table starts as the given value
  GpuDenseTable(uint64_t id, const std::string& name, const Tensor& val)
      : Table(TableType::kDense, id, name), shape_(val.shape()), element_type_(val.element_type()) {
    create_rc_ = element_type_.Is<float>() && val.IsDense()
                     ? krk_dense_create(val.Data<float>(), val.Size(), 0, &h_)
                     : ErrorCode::kDenseTableUnCompatibleError;
  }
  ~GpuDenseTable() override { krk_dense_destroy(h_); }
  krk_dense* handle() const { return h_; }

  int32_t Pull(Tensor* val) override {   // ps/dense_table.cc:31-37: a copy
    if (!h_) return create_rc_;
    Tensor out = Tensor::Dense(shape_, element_type_);
    const int32_t rc = krk_dense_pull(h_, out.Data<float>(), 0);
    if (rc == ErrorCode::kSuccess) *val = out;
    return rc;
  }

  int32_t Push(Optim* optim, const Tensor& grad, float lr) override {   // ps/dense_table.cc:39-43
    if (!h_) return create_rc_;
    const krk_optim* o = ToKrkOptim(optim);
    if (!o) return ErrorCode::kUnSupportOptimTypeError;
    if (grad.IsCoo()) {
      // densified on the device like CooTensorImpl::ToDense (t/coo_tensor_impl.cc:250-260)
      const Tensor& idx = grad.indices();
      const Tensor& v = grad.values();
      if (grad.Size() != shape_.Size() || !v.element_type().Is<float>() || !idx.element_type().Is<int64_t>())
        return ErrorCode::kGradientUnCompatibleError;
      return krk_dense_push_coo(h_, o, idx.Data<int64_t>(), v.Data<float>(), v.Size(), lr, 0);
    }
    if (grad.element_type() != element_type_) return ErrorCode::kGradientUnCompatibleError;
    return krk_dense_push(h_, o, grad.Data<float>(), grad.Size(), lr, 0);
  }
};
// [integration:end]

}  // namespace kraken
