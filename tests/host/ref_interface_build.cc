// Compiles kraken_amd/host/kraken_ref_tables.h against the reference's OWN headers (kraken/ps/table.h,
// ps/optim/optim.h, ps/initializer/initializer.h, t/tensor.h, included in place from the reference
// tree) and links the reference's own tensor, table and initializer sources with
// libkraken_hip.so: `override` on all four virtuals, the row views of Tensor::Dense(shape,
// storage, offset, etype) and the optimizer mapping are checked by the reference's compiler
// contract, not by a look-alike. Run without arguments it drives the tables through the
// reference's interface as emitter_test.cc does; with --no-gpu it checks that a machine without
// a usable GPU gets error codes and no exception.
#include <cmath>
#include <cstdio>
#include <cstring>
#include <memory>
#include <string>
#include <vector>

#include "kraken_ref_tables.h"

using namespace kraken;

static int failures = 0;
#define CHECK(cond)                                                        \
  do {                                                                     \
    if (!(cond)) {                                                         \
      std::printf("FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond);        \
      ++failures;                                                          \
    }                                                                      \
  } while (0)

int main(int argc, char** argv) {
  const bool no_gpu = argc > 1 && std::strcmp(argv[1], "--no-gpu") == 0;
  const int64_t dim = 16;
  std::unique_ptr<Optim> sgd = GpuOptim::Create(OptimType::kSGD, {});
  std::unique_ptr<Optim> adagrad = GpuOptim::Create(OptimType::kAdagrad, {{"eps", "1e-6"}, {"weight_decay", "0.5"}});
  CHECK(sgd && adagrad && adagrad->optim_type() == OptimType::kAdagrad);
  CHECK(ToKrkOptim(adagrad.get())->has_weight_decay == 1 && ToKrkOptim(adagrad.get())->eps == 1e-6f);
  CHECK(!GpuOptim::Create((OptimType)9, {}));                       // Optim::Create returns null for an unknown type
  // an optimizer that is not a GpuOptim, as the reference's own Adagrad / Adam / RMSprop / SGD are
  // (their Update needs t/math.cc, which needs Eigen, so they are not constructed here)
  struct HostOptim : Optim {
    HostOptim() : Optim(OptimType::kSGD) {}
    int32_t Update(const Tensor&, float, Value*) const override { return ErrorCode::kSuccess; }
  };
  std::unique_ptr<Optim> cpu_optim(new HostOptim());
  std::unique_ptr<Table> sparse;
  std::unique_ptr<Table> dense;
  try {
    sparse.reset(new GpuSparseTable(3, "emb", dim, ElementType::From<float>(),
                                    Initializer::Create(InitializerType::kConstant, {{"value", "0.25"}})));
    Tensor init = Tensor::Dense(std::vector<int64_t>{4, 8}, ElementType::From<float>());
    for (int64_t i = 0; i < init.Size(); ++i) init.Data<float>()[i] = (float)i;
    dense.reset(new GpuDenseTable(4, "w", init));
  } catch (...) {
    std::printf("FAILED: a constructor threw\n");
    return 1;
  }
  CHECK(sparse->type() == TableType::kSparse && sparse->id() == 3 && sparse->name() == "emb");
  const std::vector<uint64_t> ids = {7, 9, 7, ~0ull};
  std::vector<Tensor> rows;
  int32_t rc = 0;
  try {
    rc = sparse->Pull(ids, &rows);
  } catch (...) {
    std::printf("FAILED: Pull threw\n");
    return 1;
  }
  if (no_gpu) {
    // no usable device: every call reports the device failure as a code, nothing throws
    CHECK(rc == KRK_E_DEVICE);
    std::vector<Tensor> grads(ids.size(), Tensor::Dense(std::vector<int64_t>{dim}, ElementType::From<float>()));
    CHECK(sparse->Push(sgd.get(), ids, grads, 0.1f) == KRK_E_DEVICE);
    Tensor out;
    CHECK(dense->Pull(&out) == KRK_E_DEVICE);
    CHECK(dense->Push(sgd.get(), Tensor::Dense(std::vector<int64_t>{32}, ElementType::From<float>()), 0.1f) ==
          KRK_E_DEVICE);
    // the interface's own defaults still answer for the other half of each table
    CHECK(sparse->Pull(&out) == ErrorCode::kInterfaceUnImplementError);
    CHECK(dense->Pull(ids, &rows) == ErrorCode::kInterfaceUnImplementError);
    std::printf(failures ? "ref_interface_build: %d failures\n" : "ref_interface_build --no-gpu ok\n", failures);
    return failures ? 1 : 0;
  }
  // kraken/test/worker/emitter_test.cc:65-87: Constant init, rows as [n] tensors of the row width
  CHECK(rc == ErrorCode::kSuccess && rows.size() == ids.size());
  for (const Tensor& r : rows) {
    CHECK(r.Size() == dim && r.element_type() == ElementType::From<float>());
    for (int64_t j = 0; j < dim; ++j) CHECK(r.Data<float>()[j] == 0.25f);
  }
  // emitter_test.cc:89-123: after == before - lr * grad for unique ids
  const std::vector<uint64_t> uniq = {7, 9, ~0ull};
  std::vector<Tensor> grads;
  for (size_t i = 0; i < uniq.size(); ++i) {
    Tensor g = Tensor::Dense(std::vector<int64_t>{dim}, ElementType::From<float>());
    for (int64_t j = 0; j < dim; ++j) g.Data<float>()[j] = 0.5f * (float)(i + 1);
    grads.push_back(g);
  }
  CHECK(sparse->Push(cpu_optim.get(), uniq, grads, 0.1f) == ErrorCode::kUnSupportOptimTypeError);
  CHECK(sparse->Push(sgd.get(), uniq, grads, 0.1f) == ErrorCode::kSuccess);
  CHECK(sparse->Pull(uniq, &rows) == ErrorCode::kSuccess);
  for (size_t i = 0; i < uniq.size(); ++i)
    for (int64_t j = 0; j < dim; ++j) CHECK(std::fabs(rows[i].Data<float>()[j] - (0.25f - 0.1f * 0.5f * (float)(i + 1))) < 1e-7f);
  // a reply's rows are views of one page-locked block that belongs to the reply: a later reply
  // does not overwrite them, and they outlive the request vector they came back in
  {
    std::vector<Tensor> first, second;
    CHECK(sparse->Pull(uniq, &first) == ErrorCode::kSuccess);
    const Tensor kept = first[1];
    first.clear();
    CHECK(sparse->Pull({uniq[0]}, &second) == ErrorCode::kSuccess);
    for (int64_t j = 0; j < dim; ++j) CHECK(std::fabs(kept.Data<float>()[j] - (0.25f - 0.1f * 0.5f * 2.0f)) < 1e-7f);
    for (int64_t j = 0; j < dim; ++j) CHECK(std::fabs(second[0].Data<float>()[j] - (0.25f - 0.1f * 0.5f)) < 1e-7f);
    // a large reply takes a block of its own size
    std::vector<uint64_t> many(70000);
    for (size_t i = 0; i < many.size(); ++i) many[i] = 1000000 + i;
    std::vector<Tensor> big;
    CHECK(sparse->Pull(many, &big) == ErrorCode::kSuccess && big.size() == many.size());
    CHECK(big.back().Data<float>()[dim - 1] == 0.25f && big.front().Data<float>()[0] == 0.25f);
  }
  CHECK(sparse->Push(sgd.get(), {12345}, {grads[0]}, 0.1f) == ErrorCode::kSparseIdNotExistError);
  std::vector<Tensor> narrow = {Tensor::Dense(std::vector<int64_t>{dim - 1}, ElementType::From<float>())};
  CHECK(sparse->Push(sgd.get(), {7}, narrow, 0.1f) == ErrorCode::kGradientUnCompatibleError);
  // emitter_test.cc:36-63: dense round trip and SGD
  Tensor out;
  CHECK(dense->Pull(&out) == ErrorCode::kSuccess && out.Size() == 32 && out.shape()[0] == 4 && out.shape()[1] == 8);
  for (int64_t i = 0; i < 32; ++i) CHECK(out.Data<float>()[i] == (float)i);
  Tensor g = Tensor::Dense(std::vector<int64_t>{4, 8}, ElementType::From<float>());
  for (int64_t i = 0; i < 32; ++i) g.Data<float>()[i] = 2.0f;
  CHECK(dense->Push(sgd.get(), g, 0.5f) == ErrorCode::kSuccess);
  CHECK(dense->Pull(&out) == ErrorCode::kSuccess);
  for (int64_t i = 0; i < 32; ++i) CHECK(out.Data<float>()[i] == (float)i - 1.0f);
  std::printf(failures ? "ref_interface_build: %d failures\n" : "ref_interface_build ok\n", failures);
  return failures ? 1 : 0;
}
