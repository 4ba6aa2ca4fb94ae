// Host-side C++ mirror of Kraken's table interface on top of the C ABI (include/kraken_hip.h).
//
// Same class names, argument meaning and int32 error codes as kraken/ps/table.h,
// ps/sparse_table.h, ps/dense_table.h, ps/optim/optim.h and ps/initializer/initializer.h, so code
// and tests written against the reference's tables read the same here. `Tensor` is the small
// subset of kraken/t/tensor.h those interfaces use (dense fp32, or COO with int64 indices).
// Inside a Kraken tree the same adapters derive from the real kraken::Table and use the real
// kraken::Tensor instead.
#pragma once

#include <cstdint>
#include <cstring>
#include <memory>
#include <string>
#include <unordered_map>
#include <vector>

#include "kraken_hip.h"

namespace kraken_gpu {

// kraken/common/error_code.h:7-33
struct ErrorCode {
  static constexpr int32_t kSuccess = KRK_SUCCESS;
  static constexpr int32_t kUnSupportOptimTypeError = KRK_UNSUPPORTED_OPTIM;
  static constexpr int32_t kInterfaceUnImplementError = KRK_INTERFACE_UNIMPLEMENTED;
  static constexpr int32_t kGradientUnCompatibleError = KRK_GRADIENT_UNCOMPATIBLE;
  static constexpr int32_t kSparseIdNotExistError = KRK_SPARSE_ID_NOT_EXIST;
  static constexpr int32_t kUnSupportInitializerTypeError = KRK_UNSUPPORTED_INITIALIZER;
  static constexpr int32_t kTableNotExistError = 21;   // a combined request names a table outside the group
  static const char* Msg(int32_t code) { return krk_error_message(code); }
};

// kraken/common/info.h:40-72
enum class TableType : uint8_t { kDense = 0, kSparse = 1 };
enum class OptimType : uint8_t { kAdagrad = 0, kAdam = 1, kRMSprop = 2, kSGD = 3 };
enum class InitializerType : uint8_t {
  kConstant = 0, kUniform = 1, kNormal = 2, kXavierUniform = 3, kXavierNormal = 4
};
enum class StateType : uint32_t {
  kSteps = 0, kMomentumBuffer = 1, kStateSum = 2, kFirstMoment = 3, kSecondMoment = 4,
  kSecondMomentMax = 5, kSquareAverage = 6, kGAve = 7
};

// The part of kraken::Tensor the table interface touches: a ref-counted fp32 buffer with a flat
// size (copies alias, Clone copies; t/tensor.h:7-9), or a COO pair of int64 flat indices and
// fp32 values as ToCoo produces (t/tensor_impl.cc:521-560).
class Tensor {
 public:
  Tensor() = default;
  static Tensor Dense(int64_t size) {
    Tensor t;
    t.data_ = std::make_shared<std::vector<float>>((size_t)size);
    return t;
  }
  static Tensor From(const float* p, int64_t size) {
    Tensor t = Dense(size);
    if (size) std::memcpy(t.data_->data(), p, sizeof(float) * (size_t)size);
    return t;
  }
  static Tensor Coo(const std::vector<int64_t>& indices, const std::vector<float>& values,
                    int64_t dense_size) {
    Tensor t;
    t.coo_ = true;
    t.indices_ = std::make_shared<std::vector<int64_t>>(indices);
    t.data_ = std::make_shared<std::vector<float>>(values);
    t.dense_size_ = dense_size;
    return t;
  }
  bool IsCoo() const { return coo_; }
  bool IsDense() const { return !coo_; }
  bool IsEmpty() const { return Size() == 0; }
  int64_t Size() const { return coo_ ? dense_size_ : (data_ ? (int64_t)data_->size() : 0); }
  int64_t nnz() const { return coo_ ? (int64_t)indices_->size() : 0; }
  float* Data() const { return data_ ? data_->data() : nullptr; }
  const int64_t* indices() const { return indices_ ? indices_->data() : nullptr; }
  Tensor Clone() const {
    if (coo_) return Coo(*indices_, *data_, dense_size_);
    return From(Data(), Size());
  }
  float operator[](int64_t i) const { return (*data_)[(size_t)(i < 0 ? i + Size() : i)]; }

 private:
  std::shared_ptr<std::vector<float>> data_;
  std::shared_ptr<std::vector<int64_t>> indices_;
  bool coo_ = false;
  int64_t dense_size_ = 0;
};

// ps/optim/optim.h: a model-wide optimizer built from a string conf (ps/optim/optim.cc:18-105).
class Optim {
 public:
  static std::unique_ptr<Optim> Create(OptimType optim_type,
                                       const std::unordered_map<std::string, std::string>& optim_conf) {
    std::unique_ptr<Optim> optim;
    krk_optim raw;
    if (krk_optim_defaults((int32_t)optim_type, &raw) != KRK_SUCCESS) return optim;
    for (const auto& kv : optim_conf) krk_optim_set(&raw, kv.first.c_str(), kv.second.c_str());
    optim.reset(new Optim(raw));
    return optim;
  }
  OptimType optim_type() const { return (OptimType)raw_.type; }
  const krk_optim* raw() const { return &raw_; }

 private:
  explicit Optim(const krk_optim& raw) : raw_(raw) {}
  krk_optim raw_;
};

// ps/initializer/initializer.h (ps/initializer/initializer.cc:22-61).
class Initializer {
 public:
  static std::unique_ptr<Initializer> Create(
      InitializerType init_type, const std::unordered_map<std::string, std::string>& init_conf) {
    std::unique_ptr<Initializer> init;
    krk_init raw;
    if (krk_init_defaults((int32_t)init_type, &raw) != KRK_SUCCESS) return init;
    for (const auto& kv : init_conf) krk_init_set(&raw, kv.first.c_str(), kv.second.c_str());
    init.reset(new Initializer(raw));
    return init;
  }
  InitializerType type() const { return (InitializerType)raw_.type; }
  const krk_init* raw() const { return &raw_; }

 private:
  explicit Initializer(const krk_init& raw) : raw_(raw) {}
  krk_init raw_;
};

// ps/table.h:11-39 : the four virtuals, unimplemented by default (ps/table.cc:24-40).
class Table {
 public:
  virtual ~Table() = default;
  TableType type() const { return type_; }
  uint64_t id() const { return id_; }
  const std::string& name() const { return name_; }

  virtual int32_t Pull(Tensor* /*val*/) { return ErrorCode::kInterfaceUnImplementError; }
  virtual int32_t Push(Optim* /*optim*/, const Tensor& /*grad*/, float /*lr*/) {
    return ErrorCode::kInterfaceUnImplementError;
  }
  virtual int32_t Pull(const std::vector<uint64_t>& /*sparse_ids*/, std::vector<Tensor>* /*vals*/) {
    return ErrorCode::kInterfaceUnImplementError;
  }
  virtual int32_t Push(Optim* /*optim*/, const std::vector<uint64_t>& /*sparse_ids*/,
                       const std::vector<Tensor>& /*grads*/, float /*lr*/) {
    return ErrorCode::kInterfaceUnImplementError;
  }

 protected:
  Table(TableType type, uint64_t id, const std::string& name) : type_(type), id_(id), name_(name) {}
  TableType type_;
  uint64_t id_;
  std::string name_;
};

// ps/sparse_table.h with the rows in HBM. Pull returns copies (ps/sparse_table.cc:57,64);
// Push takes unique ids and one gradient tensor per id.
class SparseTable : public Table {
 public:
  SparseTable(uint64_t id, const std::string& name, int64_t dimension,
              std::unique_ptr<Initializer>&& initializer, int64_t capacity_hint = 0)
      : Table(TableType::kSparse, id, name), dimension_(dimension), initializer_(std::move(initializer)) {
    create_code_ = initializer_ ? krk_sparse_create(dimension, initializer_->raw(), capacity_hint, &h_)
                                : ErrorCode::kUnSupportInitializerTypeError;
  }
  ~SparseTable() override { krk_sparse_destroy(h_); }
  SparseTable(const SparseTable&) = delete;
  SparseTable& operator=(const SparseTable&) = delete;

  int32_t create_code() const { return create_code_; }   // 0, 13, or a device error
  int64_t dimension() const { return dimension_; }
  Initializer* initializer() const { return initializer_.get(); }
  krk_sparse* handle() const { return h_; }

  int32_t Pull(const std::vector<uint64_t>& sparse_ids, std::vector<Tensor>* vals) override {
    if (!h_) return create_code_;
    const int64_t n = (int64_t)sparse_ids.size();
    std::vector<float> flat((size_t)(n * dimension_));
    const int32_t rc = krk_sparse_pull(h_, sparse_ids.data(), n, flat.data(), 0);
    if (rc != ErrorCode::kSuccess) return rc;
    vals->resize((size_t)n);
    for (int64_t i = 0; i < n; ++i) (*vals)[(size_t)i] = Tensor::From(flat.data() + i * dimension_, dimension_);
    return ErrorCode::kSuccess;
  }

  int32_t Push(Optim* optim, const std::vector<uint64_t>& sparse_ids, const std::vector<Tensor>& grads,
               float lr) override {
    if (!h_) return create_code_;
    if (!optim) return ErrorCode::kUnSupportOptimTypeError;
    const int64_t n = (int64_t)sparse_ids.size();
    if ((int64_t)grads.size() != n) return ErrorCode::kGradientUnCompatibleError;
    std::vector<float> flat((size_t)(n * dimension_));
    for (int64_t i = 0; i < n; ++i) {
      // ps/optim/adagrad.cc:29-32 : every gradient must have the row's size
      if (grads[(size_t)i].IsCoo() || grads[(size_t)i].Size() != dimension_)
        return ErrorCode::kGradientUnCompatibleError;
      std::memcpy(flat.data() + i * dimension_, grads[(size_t)i].Data(), sizeof(float) * (size_t)dimension_);
    }
    return krk_sparse_push(h_, optim->raw(), sparse_ids.data(), n, flat.data(), dimension_, lr, 0);
  }

 private:
  int64_t dimension_;
  std::unique_ptr<Initializer> initializer_;
  krk_sparse* h_ = nullptr;
  int32_t create_code_ = 0;
};

// protocol/combine_push_sparse_table_prot.h:12-15
struct CombinePushSparseTableItem {
  std::vector<uint64_t> sparse_ids;
  std::vector<Tensor> grads;
};

// The sparse tables of equal dimension that combined requests address together. CombinePull /
// CombinePush have the signatures of Ps::CombinePullSparseTable / CombinePushSparseTable
// (ps/ps_op.cc:370-387, 456-469) without the router version; where the reference loops over the
// tables of the request, here one launch serves them all. Tables outside the request take part
// with zero ids. Destroy the group before its tables.
class SparseTableGroup {
 public:
  explicit SparseTableGroup(const std::vector<SparseTable*>& tables) : tables_(tables) {
    std::vector<krk_sparse*> hs;
    for (SparseTable* t : tables_) hs.push_back(t ? t->handle() : nullptr);
    create_code_ = krk_group_create(hs.data(), (int32_t)hs.size(), &h_);
    dimension_ = tables_.empty() || !tables_[0] ? 0 : tables_[0]->dimension();
  }
  ~SparseTableGroup() { krk_group_destroy(h_); }
  SparseTableGroup(const SparseTableGroup&) = delete;
  SparseTableGroup& operator=(const SparseTableGroup&) = delete;

  int32_t create_code() const { return create_code_; }
  krk_group* handle() const { return h_; }

  int32_t CombinePull(const std::unordered_map<uint64_t, std::vector<uint64_t>>& table_sparse_ids,
                      std::unordered_map<uint64_t, std::vector<Tensor>>* table_vals) {
    if (!h_) return create_code_;
    std::vector<uint64_t> ids;
    std::vector<int64_t> offsets(tables_.size() + 1, 0);
    size_t found = 0;
    for (size_t m = 0; m < tables_.size(); ++m) {
      auto it = table_sparse_ids.find(tables_[m]->id());
      if (it != table_sparse_ids.end()) {
        ids.insert(ids.end(), it->second.begin(), it->second.end());
        ++found;
      }
      offsets[m + 1] = (int64_t)ids.size();
    }
    if (found != table_sparse_ids.size()) return ErrorCode::kTableNotExistError;   // ps_op.cc:348-351
    std::vector<float> flat(ids.size() * (size_t)dimension_);
    const int32_t rc = krk_group_pull(h_, ids.data(), offsets.data(), flat.data(), 0);
    if (rc != ErrorCode::kSuccess) return rc;
    for (size_t m = 0; m < tables_.size(); ++m) {
      if (!table_sparse_ids.count(tables_[m]->id())) continue;
      std::vector<Tensor> vals;
      for (int64_t i = offsets[m]; i < offsets[m + 1]; ++i)
        vals.push_back(Tensor::From(flat.data() + i * dimension_, dimension_));
      table_vals->emplace(tables_[m]->id(), std::move(vals));
    }
    return ErrorCode::kSuccess;
  }

  // unique_ids = true: the request as Emitter::CombinePushSparseTable sends it (ids already
  // deduplicated per table). false: ids may repeat within a table and their gradients are summed
  // on the device (worker/emitter.cc:552-606 moved to the server).
  int32_t CombinePush(Optim* optim, const std::unordered_map<uint64_t, CombinePushSparseTableItem>& table_items,
                      float lr, bool unique_ids = true) {
    if (!h_) return create_code_;
    if (!optim) return ErrorCode::kUnSupportOptimTypeError;
    std::vector<uint64_t> ids;
    std::vector<float> flat;
    std::vector<int64_t> offsets(tables_.size() + 1, 0);
    size_t found = 0;
    for (size_t m = 0; m < tables_.size(); ++m) {
      auto it = table_items.find(tables_[m]->id());
      if (it != table_items.end()) {
        const CombinePushSparseTableItem& item = it->second;
        if (item.grads.size() != item.sparse_ids.size()) return ErrorCode::kGradientUnCompatibleError;
        for (size_t i = 0; i < item.sparse_ids.size(); ++i) {
          const Tensor& g = item.grads[i];
          if (g.IsCoo() || g.Size() != dimension_) return ErrorCode::kGradientUnCompatibleError;
          ids.push_back(item.sparse_ids[i]);
          flat.insert(flat.end(), g.Data(), g.Data() + dimension_);
        }
        ++found;
      }
      offsets[m + 1] = (int64_t)ids.size();
    }
    if (found != table_items.size()) return ErrorCode::kTableNotExistError;
    return unique_ids ? krk_group_push(h_, optim->raw(), ids.data(), offsets.data(), flat.data(), dimension_, lr, 0)
                      : krk_group_push_raw(h_, optim->raw(), ids.data(), offsets.data(), flat.data(), dimension_,
                                           lr, 0);
  }

 private:
  std::vector<SparseTable*> tables_;
  int64_t dimension_ = 0;
  krk_group* h_ = nullptr;
  int32_t create_code_ = 0;
};

// ps/dense_table.h with the parameter vector in HBM; a COO gradient is densified on the device.
class DenseTable : public Table {
 public:
  DenseTable(uint64_t id, const std::string& name, const Tensor& val)
      : Table(TableType::kDense, id, name), size_(val.Size()) {
    create_code_ = krk_dense_create(val.Data(), val.Size(), 0, &h_);
  }
  // Adopts a table the library built (krk_dense_load_file).
  DenseTable(uint64_t id, const std::string& name, krk_dense* adopted)
      : Table(TableType::kDense, id, name), size_(0), h_(adopted) {
    if (krk_dense_size(h_, &size_) != KRK_SUCCESS) create_code_ = KRK_E_ARGUMENT;
  }
  ~DenseTable() override { krk_dense_destroy(h_); }
  DenseTable(const DenseTable&) = delete;
  DenseTable& operator=(const DenseTable&) = delete;

  int32_t create_code() const { return create_code_; }
  krk_dense* handle() const { return h_; }

  int32_t Pull(Tensor* val) override {
    if (!h_) return create_code_;
    Tensor out = Tensor::Dense(size_);
    const int32_t rc = krk_dense_pull(h_, out.Data(), 0);
    if (rc == ErrorCode::kSuccess) *val = out;
    return rc;
  }

  int32_t Push(Optim* optim, const Tensor& grad, float lr) override {
    if (!h_) return create_code_;
    if (!optim) return ErrorCode::kUnSupportOptimTypeError;
    if (grad.IsCoo()) {
      if (grad.nnz() > 0 && grad.Size() != size_) return ErrorCode::kGradientUnCompatibleError;
      return krk_dense_push_coo(h_, optim->raw(), grad.indices(), grad.Data(), grad.nnz(), lr, 0);
    }
    return krk_dense_push(h_, optim->raw(), grad.Data(), grad.Size(), lr, 0);
  }

 private:
  int64_t size_;
  krk_dense* h_ = nullptr;
  int32_t create_code_ = 0;
};

}  // namespace kraken_gpu
