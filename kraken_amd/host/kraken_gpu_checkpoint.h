// kraken/checkpoint/checkpoint.h's table functions for the GPU tables of kraken_gpu_tables.h:
// same names and argument meaning, bool results like the reference. The byte layout lives in
// the shared library (krk_*_save_file / krk_*_load_file, include/kraken_hip.h).
//
//   SaveSparseTable / LoadSparseTable   checkpoint/checkpoint.cc:465-509, 586-649  (*.sparse)
//   SaveDenseTable  / LoadDenseTable    checkpoint/checkpoint.cc:444-463, 535-557  (*.dense)
#ifndef KRAKEN_GPU_CHECKPOINT_H_
#define KRAKEN_GPU_CHECKPOINT_H_

#include <functional>

#include "kraken_gpu_tables.h"

namespace kraken_gpu {
namespace io {

inline bool SaveSparseTable(const std::string& path, SparseTable* table) {
  return table->handle() &&
         krk_sparse_save_file(table->handle(), path.c_str(), table->id(), table->name().c_str()) == KRK_SUCCESS;
}

// `keep` stands for node_id == router.Hit(utils::Hash(table_id, sparse_id)) (checkpoint.cc:640);
// an empty function keeps every row.
inline bool LoadSparseTable(const std::string& path, SparseTable* table,
                            const std::function<bool(uint64_t)>& keep = nullptr) {
  if (!table->handle()) return false;
  auto thunk = [](uint64_t id, void* ctx) -> int32_t {
    return (*static_cast<const std::function<bool(uint64_t)>*>(ctx))(id) ? 1 : 0;
  };
  return krk_sparse_load_file(table->handle(), path.c_str(), table->id(), table->name().c_str(),
                              keep ? +thunk : nullptr, const_cast<std::function<bool(uint64_t)>*>(&keep),
                              nullptr) == KRK_SUCCESS;
}

// The tensor is recorded with `shape` (default: one dimension).
inline bool SaveDenseTable(const std::string& path, DenseTable* table, const std::vector<int64_t>& shape = {}) {
  return table->handle() && krk_dense_save_file(table->handle(), path.c_str(), table->id(), table->name().c_str(),
                                                shape.data(), (int32_t)shape.size()) == KRK_SUCCESS;
}

inline std::unique_ptr<DenseTable> LoadDenseTable(const std::string& path) {
  krk_dense* h = nullptr;
  uint64_t id = 0;
  char name[1024];
  if (krk_dense_load_file(path.c_str(), &h, &id, name, sizeof(name), nullptr, nullptr) != KRK_SUCCESS)
    return nullptr;
  return std::unique_ptr<DenseTable>(new DenseTable(id, name, h));
}

}  // namespace io
}  // namespace kraken_gpu

#endif  // KRAKEN_GPU_CHECKPOINT_H_
