// Host-side test of the C++ table adapters, shaped like the reference's own
// kraken/test/worker/emitter_test.cc:36-158 with the RPC layer removed: dense pull round trip,
// dense SGD, sparse insert with a Constant initializer, sparse SGD, and the error codes a server
// thread can see (ps/sparse_table.cc:96-98, ps/optim/adagrad.cc:29-32, ps/table.cc:24-40).
// Exits 0 when every check holds; prints the first failure otherwise.
//   table_interface_test            -> needs a GPU
//   table_interface_test --no-gpu   -> checks that construction fails loudly without one
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>

#include "kraken_gpu_checkpoint.h"
#include "kraken_gpu_tables.h"

using namespace kraken_gpu;

static int failures = 0;
#define EXPECT(cond)                                                        \
  do {                                                                      \
    if (!(cond)) {                                                          \
      std::printf("FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond);         \
      ++failures;                                                           \
    }                                                                       \
  } while (0)

static Tensor RandomTensor(int64_t n, std::mt19937& rng) {
  std::uniform_real_distribution<float> d(-1.0f, 1.0f);
  Tensor t = Tensor::Dense(n);
  for (int64_t i = 0; i < n; ++i) t.Data()[i] = d(rng);
  return t;
}

// gtest's EXPECT_FLOAT_EQ: within 4 ULP.
static bool FloatEq(float a, float b) {
  if (a == b) return true;
  int32_t ia, ib;
  std::memcpy(&ia, &a, 4);
  std::memcpy(&ib, &b, 4);
  if ((ia < 0) != (ib < 0)) return false;
  return std::abs(ia - ib) <= 4;
}

static int no_gpu_mode() {
  auto init = Initializer::Create(InitializerType::kConstant, {{"value", "1"}});
  SparseTable st(2, "SparseTable0", 100, std::move(init));
  EXPECT(st.create_code() == KRK_E_DEVICE);
  std::vector<Tensor> vals;
  EXPECT(st.Pull({0, 1}, &vals) == KRK_E_DEVICE);
  DenseTable dt(0, "DenseTable0", Tensor::Dense(16));
  EXPECT(dt.create_code() == KRK_E_DEVICE);
  Tensor out;
  EXPECT(dt.Pull(&out) == KRK_E_DEVICE);
  std::printf("%s\n", failures ? "FAILED" : "no-gpu ok");
  return failures ? 1 : 0;
}

int main(int argc, char** argv) {
  if (argc > 1 && std::strcmp(argv[1], "--no-gpu") == 0) return no_gpu_mode();
  std::mt19937 rng(7);
  auto sgd = Optim::Create(OptimType::kSGD, {});
  EXPECT(sgd && sgd->optim_type() == OptimType::kSGD);
  EXPECT(!Optim::Create((OptimType)9, {}));
  EXPECT(!Initializer::Create((InitializerType)9, {}));

  // emitter_test.cc:36-49 : register, pull back bit-exact
  Tensor d0 = RandomTensor(100, rng), g0 = RandomTensor(100, rng);
  DenseTable dense(0, "DensTable0", d0);
  EXPECT(dense.create_code() == 0);
  Tensor r0;
  EXPECT(dense.Pull(&r0) == 0);
  for (int i = 0; i < 100; ++i) EXPECT(r0[i] == d0[i]);
  // :51-63 : r0 == d0 - lr * g0
  float lr = 0.4375f;
  EXPECT(dense.Push(sgd.get(), g0, lr) == 0);
  EXPECT(dense.Pull(&r0) == 0);
  for (int i = 0; i < 100; ++i) EXPECT(FloatEq(r0[i], d0[i] - lr * g0[i]));
  EXPECT(dense.Push(sgd.get(), RandomTensor(7, rng), lr) == ErrorCode::kGradientUnCompatibleError);
  // a COO gradient is densified: only the listed elements move under plain SGD
  Tensor before = r0.Clone();
  EXPECT(dense.Push(sgd.get(), Tensor::Coo({3, 50}, {1.0f, -2.0f}, 100), 0.5f) == 0);
  EXPECT(dense.Pull(&r0) == 0);
  for (int i = 0; i < 100; ++i) {
    const float want = i == 3 ? before[i] - 0.5f : i == 50 ? before[i] + 1.0f : before[i];
    EXPECT(FloatEq(r0[i], want));
  }
  // the default Table refuses the sparse calls (ps/table.cc:32-40)
  std::vector<Tensor> none;
  EXPECT(static_cast<Table&>(dense).Pull({1}, &none) == ErrorCode::kInterfaceUnImplementError);

  // :65-72 : sparse insert-on-pull with a Constant initializer
  const float v0 = 321.5f;
  SparseTable sparse(2, "SparseTable0", 100,
                     Initializer::Create(InitializerType::kConstant, {{"value", std::to_string(v0)}}));
  EXPECT(sparse.create_code() == 0 && sparse.dimension() == 100);
  std::vector<Tensor> vals;
  EXPECT(sparse.Pull({0, 1}, &vals) == 0);
  EXPECT(vals.size() == 2 && vals[0].Size() == 100);
  for (int r = 0; r < 2; ++r)
    for (int i = 0; i < 100; ++i) EXPECT(vals[r][i] == v0);
  // :89-110 : real == v0 - lr * grad
  std::vector<Tensor> grads = {RandomTensor(100, rng), RandomTensor(100, rng)};
  lr = 0.625f;
  EXPECT(sparse.Push(sgd.get(), {0, 1}, grads, lr) == 0);
  EXPECT(sparse.Pull({0, 1}, &vals) == 0);
  for (int r = 0; r < 2; ++r)
    for (int i = 0; i < 100; ++i) EXPECT(FloatEq(vals[r][i], v0 - lr * grads[r][i]));
  // pulled tensors are copies: changing one does not change the table (sparse_table.cc:57)
  vals[0].Data()[0] = 1e9f;
  std::vector<Tensor> again;
  EXPECT(sparse.Pull({0}, &again) == 0);
  EXPECT(FloatEq(again[0][0], v0 - lr * grads[0][0]));
  // ps/sparse_table.cc:96-98 and ps/optim/*.cc size check
  EXPECT(sparse.Push(sgd.get(), {0, 99}, grads, lr) == ErrorCode::kSparseIdNotExistError);
  std::vector<Tensor> narrow = {RandomTensor(50, rng), RandomTensor(50, rng)};
  EXPECT(sparse.Push(sgd.get(), {0, 1}, narrow, lr) == ErrorCode::kGradientUnCompatibleError);
  EXPECT(std::strcmp(ErrorCode::Msg(12), "SparseId not exist") == 0);
  EXPECT(static_cast<Table&>(sparse).Pull(&r0) == ErrorCode::kInterfaceUnImplementError);

  // Adagrad twice on one row: state persists between pushes (adagrad.cc:34-45)
  auto adagrad = Optim::Create(OptimType::kAdagrad, {{"eps", "1e-10"}});
  SparseTable s2(3, "SparseTable1", 4, Initializer::Create(InitializerType::kConstant, {{"value", "1"}}));
  EXPECT(s2.Pull({5}, &vals) == 0);
  std::vector<Tensor> g = {Tensor::Dense(4)};
  for (int i = 0; i < 4; ++i) g[0].Data()[i] = 0.5f * (i + 1);
  EXPECT(s2.Push(adagrad.get(), {5}, g, 0.1f) == 0);
  EXPECT(s2.Push(adagrad.get(), {5}, g, 0.1f) == 0);
  EXPECT(s2.Pull({5}, &vals) == 0);
  for (int i = 0; i < 4; ++i) {
    const float gi = 0.5f * (i + 1);
    float sum = gi * gi, w = 1.0f;
    w -= 0.1f * (gi / (std::sqrt(sum) + 1e-10f));
    sum += gi * gi;
    w -= 0.1f * (gi / (std::sqrt(sum) + 1e-10f));
    EXPECT(FloatEq(vals[0][i], w));
  }
  // emitter_test.cc:75-87, 112-158 : two tables, combined pull and combined push with SGD
  {
    const float c0 = 7.5f, c1 = -3.25f;
    SparseTable t0(10, "Combine0", 100, Initializer::Create(InitializerType::kConstant, {{"value", std::to_string(c0)}}));
    SparseTable t1(11, "Combine1", 100, Initializer::Create(InitializerType::kConstant, {{"value", std::to_string(c1)}}));
    SparseTableGroup grp({&t0, &t1});
    EXPECT(grp.create_code() == 0);
    std::unordered_map<uint64_t, std::vector<Tensor>> got;
    EXPECT(grp.CombinePull({{10, {0, 1}}, {11, {0, 1}}}, &got) == 0);
    EXPECT(got.size() == 2 && got[10].size() == 2 && got[11].size() == 2);
    for (int r = 0; r < 2; ++r)
      for (int i = 0; i < 100; ++i) EXPECT(got[10][r][i] == c0 && got[11][r][i] == c1);
    std::unordered_map<uint64_t, CombinePushSparseTableItem> items;
    items[10] = {{0, 1}, {RandomTensor(100, rng), RandomTensor(100, rng)}};
    items[11] = {{1}, {RandomTensor(100, rng)}};
    lr = 0.625f;
    EXPECT(grp.CombinePush(sgd.get(), items, lr) == 0);
    got.clear();
    EXPECT(grp.CombinePull({{11, {1, 0}}, {10, {1, 0}}}, &got) == 0);
    for (int i = 0; i < 100; ++i) {
      EXPECT(FloatEq(got[10][0][i], c0 - lr * items[10].grads[1][i]));
      EXPECT(FloatEq(got[10][1][i], c0 - lr * items[10].grads[0][i]));
      EXPECT(FloatEq(got[11][0][i], c1 - lr * items[11].grads[0][i]));
      EXPECT(got[11][1][i] == c1);
    }
    // repeated ids: their gradients are summed before the single update (emitter.cc:584-604)
    std::unordered_map<uint64_t, CombinePushSparseTableItem> rep;
    Tensor ga = Tensor::Dense(100), gb = Tensor::Dense(100);
    for (int i = 0; i < 100; ++i) {
      ga.Data()[i] = 0.25f * (i % 7);
      gb.Data()[i] = -0.5f * (i % 3);
    }
    rep[11] = {{0, 0, 0}, {ga, gb, ga}};
    EXPECT(grp.CombinePush(sgd.get(), rep, 0.5f, /*unique_ids=*/false) == 0);
    std::vector<Tensor> one;
    EXPECT(t1.Pull({0}, &one) == 0);                            // a member's own call sees the group's write
    for (int i = 0; i < 100; ++i) EXPECT(one[0][i] == c1 - 0.5f * (2 * ga[i] + gb[i]));
    // errors: a table outside the group, an id the table has never seen, a narrow gradient
    EXPECT(grp.CombinePull({{12, {0}}}, &got) == ErrorCode::kTableNotExistError);
    std::unordered_map<uint64_t, CombinePushSparseTableItem> bad;
    bad[10] = {{77}, {RandomTensor(100, rng)}};
    EXPECT(grp.CombinePush(sgd.get(), bad, lr) == ErrorCode::kSparseIdNotExistError);
    bad[10] = {{0}, {RandomTensor(50, rng)}};
    EXPECT(grp.CombinePush(sgd.get(), bad, lr) == ErrorCode::kGradientUnCompatibleError);
  }

  // checkpoint/checkpoint.cc:444-509, 535-649 : through *.sparse / *.dense files and on
  const char* tmp = std::getenv("TMPDIR");
  const std::string dir = tmp ? tmp : "/tmp";
  const std::string sparse_path = dir + "/krk_host_test.sparse", dense_path = dir + "/krk_host_test.dense";
  EXPECT(io::SaveSparseTable(sparse_path, &s2));
  SparseTable s3(3, "SparseTable1", 4, Initializer::Create(InitializerType::kConstant, {{"value", "1"}}));
  EXPECT(io::LoadSparseTable(sparse_path, &s3, [](uint64_t id) { return id == 5; }));
  SparseTable other(4, "SparseTable1", 4, Initializer::Create(InitializerType::kConstant, {{"value", "1"}}));
  EXPECT(!io::LoadSparseTable(sparse_path, &other));          // another table id: refused (:611-616)
  EXPECT(s2.Push(adagrad.get(), {5}, g, 0.1f) == 0);
  EXPECT(s3.Push(adagrad.get(), {5}, g, 0.1f) == 0);          // carries on with the saved state_sum
  std::vector<Tensor> a, b;
  EXPECT(s2.Pull({5}, &a) == 0 && s3.Pull({5}, &b) == 0);
  for (int i = 0; i < 4; ++i) EXPECT(a[0][i] == b[0][i]);
  EXPECT(io::SaveDenseTable(dense_path, &dense, {10, 10}));
  std::unique_ptr<DenseTable> dense2 = io::LoadDenseTable(dense_path);
  EXPECT(dense2 && dense2->id() == 0 && dense2->name() == "DensTable0");
  Tensor x, y;
  EXPECT(dense2 && dense.Pull(&x) == 0 && dense2->Pull(&y) == 0 && x.Size() == y.Size());
  for (int i = 0; i < 100 && dense2; ++i) EXPECT(x[i] == y[i]);
  EXPECT(!io::LoadDenseTable(sparse_path));                    // a sparse file is no dense table
  std::remove(sparse_path.c_str());
  std::remove(dense_path.c_str());
  std::printf("%s\n", failures ? "FAILED" : "table interface ok");
  return failures ? 1 : 0;
}
