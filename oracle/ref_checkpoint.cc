// Test infrastructure only. Writes table files with the reference's OWN serializer
// (kraken/common/serialize.h, checkpoint/file_writer.cc, t/tensor*.cc compiled where they lie),
// and reads files back with its own deserializer, so that the byte layout of *.sparse / *.dense
// files is pinned by the code that defines it.
//
// checkpoint/checkpoint.cc itself cannot be compiled here (it includes configor, which is not in
// this image), so the order of the fields is restated below, statement for statement, from
// Checkpoint::SaveDenseTable (checkpoint.cc:445-462) and Checkpoint::SaveSparseTable
// (checkpoint.cc:464-509), LoadDenseTable (:535-584) and LoadSparseTable (:586-649); every
// `serialize << x` / `deserialize >> x` executes the reference's operator for that type.
// The tensor sources reference t/math.cc, which needs Eigen (absent); those symbols stay
// unresolved in this binary and are never called (constructing, filling and serializing a
// tensor does not go through t/math.cc).
//
//   ref_checkpoint write-sparse <path> <dim> <rows> <states: comma list of StateType numbers or -> <steps 0|1>
//   ref_checkpoint write-dense  <path> <size>
//   ref_checkpoint dump-sparse  <path>      -> text, one row per line
//   ref_checkpoint dump-dense   <path>
//   ref_checkpoint write-rows   <path> <n> <dim>   -> std::vector<Tensor> as an RPC body carries it
//   ref_checkpoint dump-rows    <path>
//
// Row r of a written table: id = splitmix64(r); val[j] = pattern(id, 0, j); state s:
// pattern(id, s + 1, j); steps = 1 + id % 7. pattern is exact in fp32 (multiples of 1/64).
#include <cinttypes>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <memory>
#include <mutex>
#include <string>
#include <vector>

#include "checkpoint/file_reader.h"
#include "checkpoint/file_writer.h"
#include "common/deserialize.h"
#include "common/info.h"
#include "common/parallel_skip_list.h"
#include "common/serialize.h"
#include "ps/initializer/initializer.h"
#include "t/tensor.h"

using namespace kraken;

static uint64_t splitmix64(uint64_t x) {
  uint64_t z = x + 0x9E3779B97F4A7C15ull;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

static float pattern(uint64_t id, int which, int64_t j) {
  const uint64_t h = splitmix64(id * 31 + (uint64_t)which * 1000003 + (uint64_t)j);
  return (float)((int64_t)(h % 2049) - 1024) / 64.0f;
}

static Tensor filled(uint64_t id, int which, int64_t dim) {
  Tensor t = Tensor::Dense({dim}, ElementType::From<float>());
  float* p = t.Data<float>();
  for (int64_t j = 0; j < dim; ++j) p[j] = pattern(id, which, j);
  return t;
}

static int write_sparse(const char* path, int64_t dim, int64_t rows, const char* states, int with_steps) {
  std::vector<uint32_t> st;
  if (strcmp(states, "-") != 0) {
    std::string s(states);
    size_t pos = 0;
    while (pos < s.size()) {
      size_t c = s.find(',', pos);
      if (c == std::string::npos) c = s.size();
      st.push_back((uint32_t)atoi(s.substr(pos, c - pos).c_str()));
      pos = c + 1;
    }
  }
  // SparseTable's member (ps/sparse_table.h:29) with the container's default of 8 slots
  ParallelSkipList<uint64_t, Value> vals;
  for (int64_t r = 0; r < rows; ++r) {
    const uint64_t id = splitmix64((uint64_t)r);
    Value v;
    v.val = filled(id, 0, dim);
    for (uint32_t s : st) v.states.emplace((StateType)s, filled(id, (int)s + 1, dim));
    if (with_steps) v.states_i.emplace(StateType::kSteps, (int64_t)(1 + id % 7));
    const size_t slot = vals.HitSlot(id);
    auto h = vals.UniqueSkipListHandler(slot);
    h.skip_list.Insert(id, v);
  }

  io::FileWriter writer(path);
  if (!writer.IsOpen()) return 2;
  Serialize serialize(&writer);
  // checkpoint.cc:473-480
  const TableType type = TableType::kSparse;
  const uint64_t table_id = 7;
  const std::string name = "emb";
  const ElementType etype = ElementType::From<float>();
  // the initializer and its conf strings are the reference's own (ps/initializer/initializer.cc:22-61,
  // normal_initializer.cc:12-14), as SparseTable::initializer() hands them to the writer
  const std::unique_ptr<Initializer> init =
      Initializer::Create(InitializerType::kNormal, {{"mean", "0.0"}, {"stddev", "0.01"}});
  if (!init) return 4;
  const InitializerType init_type = init->type();
  const std::unordered_map<std::string, std::string> conf = init->conf();
  if (!(serialize << type) || !(serialize << table_id) || !(serialize << name) || !(serialize << dim) ||
      !(serialize << etype) || !(serialize << init_type) || !(serialize << conf))
    return 3;
  // checkpoint.cc:484-505
  uint64_t slot_count = vals.slot_count();
  if (!(serialize << slot_count)) return 3;
  for (uint64_t slot = 0; slot < slot_count; ++slot) {
    auto h = vals.SharedSkipListHandler(slot);
    uint64_t skip_list_size = h.skip_list.Size();
    if (!(serialize << skip_list_size)) return 3;
    for (auto it = h.skip_list.Begin(); it.Valid(); it.Next()) {
      if (!(serialize << it.key()) || !(serialize << it.value())) return 3;
    }
  }
  return 0;
}

static int write_dense(const char* path, int64_t size) {
  io::FileWriter writer(path);
  if (!writer.IsOpen()) return 2;
  Serialize serialize(&writer);
  Value v;
  v.val = Tensor::Dense({size / 4, 4}, ElementType::From<float>());
  float* p = v.val.Data<float>();
  for (int64_t j = 0; j < size; ++j) p[j] = pattern(99, 0, j);
  v.states.emplace(StateType::kFirstMoment, filled(99, 4, size).Reshape({size / 4, 4}));
  v.states.emplace(StateType::kSecondMoment, filled(99, 5, size).Reshape({size / 4, 4}));
  v.states_i.emplace(StateType::kSteps, 12);
  // checkpoint.cc:454-459
  const TableType type = TableType::kDense;
  const uint64_t table_id = 3;
  const std::string name = "dense0";
  if (!(serialize << type) || !(serialize << table_id) || !(serialize << name) || !(serialize << v)) return 3;
  return 0;
}

static void print_tensor(const Tensor& t) {
  printf("[");
  const auto& dims = t.shape().dims();
  for (size_t i = 0; i < dims.size(); ++i) printf("%s%" PRId64, i ? "x" : "", dims[i]);
  printf("]");
  const float* p = t.Data<float>();
  for (int64_t j = 0; j < t.Size(); ++j) printf(" %.9g", p[j]);
}

static void print_value(const Value& v) {
  printf("val ");
  print_tensor(v.val);
  for (uint32_t s = 0; s < 8; ++s) {
    auto it = v.states.find((StateType)s);
    if (it == v.states.end()) continue;
    printf(" | state %u ", s);
    print_tensor(it->second);
  }
  for (uint32_t s = 0; s < 8; ++s) {
    auto it = v.states_i.find((StateType)s);
    if (it == v.states_i.end()) continue;
    printf(" | int %u %" PRId64, s, it->second);
  }
  printf("\n");
}

static int dump_sparse(const char* path) {
  io::FileReader reader(path);
  if (!reader.IsOpen()) return 2;
  Deserialize deserialize(&reader);
  // checkpoint.cc:596-619
  TableType type;
  uint64_t table_id;
  std::string name;
  int64_t dim;
  ElementType etype;
  InitializerType init_type;
  std::unordered_map<std::string, std::string> conf;
  if (!(deserialize >> type) || !(deserialize >> table_id) || !(deserialize >> name) || !(deserialize >> dim) ||
      !(deserialize >> etype) || !(deserialize >> init_type) || !(deserialize >> conf))
    return 3;
  printf("type %u id %" PRIu64 " name %s dim %" PRId64 " dtype %u init %u conf", (unsigned)type, table_id,
         name.c_str(), dim, (unsigned)etype.dtype, (unsigned)init_type);
  std::vector<std::string> keys;
  for (auto& kv : conf) keys.push_back(kv.first);
  std::sort(keys.begin(), keys.end());
  for (auto& k : keys) printf(" %s=%s", k.c_str(), conf[k].c_str());
  printf("\n");
  // checkpoint.cc:621-645
  uint64_t slot_count;
  if (!(deserialize >> slot_count)) return 3;
  printf("slots %" PRIu64 "\n", slot_count);
  for (uint64_t slot = 0; slot < slot_count; ++slot) {
    uint64_t size;
    if (!(deserialize >> size)) return 3;
    printf("slot %" PRIu64 " rows %" PRIu64 "\n", slot, size);
    for (uint64_t i = 0; i < size; ++i) {
      uint64_t id;
      Value v;
      if (!(deserialize >> id) || !(deserialize >> v)) return 3;
      printf("id %" PRIu64 " ", id);
      print_value(v);
    }
  }
  return 0;
}

static int dump_dense(const char* path) {
  io::FileReader reader(path);
  if (!reader.IsOpen()) return 2;
  Deserialize deserialize(&reader);
  // checkpoint.cc:545-556
  TableType type;
  uint64_t table_id;
  std::string name;
  Value v;
  if (!(deserialize >> type) || !(deserialize >> table_id) || !(deserialize >> name) || !(deserialize >> v))
    return 3;
  printf("type %u id %" PRIu64 " name %s\n", (unsigned)type, table_id, name.c_str());
  print_value(v);
  return 0;
}

// The body of a PullSparseTableResponse / the grads member of a PushSparseTableRequest
// (protocol/pull_sparse_table_prot.h:29-41, push_sparse_table_prot.h:11-30): row r is
// pattern(splitmix64(r), 0, j).
static int write_rows(const char* path, int64_t n, int64_t dim) {
  std::vector<Tensor> vals;
  for (int64_t r = 0; r < n; ++r) vals.emplace_back(filled(splitmix64((uint64_t)r), 0, dim));
  io::FileWriter writer(path);
  if (!writer.IsOpen()) return 2;
  Serialize serialize(&writer);
  return (serialize << vals) ? 0 : 3;
}

static int dump_rows(const char* path) {
  io::FileReader reader(path);
  if (!reader.IsOpen()) return 2;
  Deserialize deserialize(&reader);
  std::vector<Tensor> vals;
  if (!(deserialize >> vals)) return 3;
  printf("rows %zu\n", vals.size());
  for (const Tensor& t : vals) {
    print_tensor(t);
    printf("\n");
  }
  return 0;
}

int main(int argc, char** argv) {
  if (argc >= 7 && !strcmp(argv[1], "write-sparse"))
    return write_sparse(argv[2], atoll(argv[3]), atoll(argv[4]), argv[5], atoi(argv[6]));
  if (argc >= 4 && !strcmp(argv[1], "write-dense")) return write_dense(argv[2], atoll(argv[3]));
  if (argc >= 3 && !strcmp(argv[1], "dump-sparse")) return dump_sparse(argv[2]);
  if (argc >= 3 && !strcmp(argv[1], "dump-dense")) return dump_dense(argv[2]);
  if (argc >= 5 && !strcmp(argv[1], "write-rows")) return write_rows(argv[2], atoll(argv[3]), atoll(argv[4]));
  if (argc >= 3 && !strcmp(argv[1], "dump-rows")) return dump_rows(argv[2]);
  fprintf(stderr, "usage: see the head of oracle/ref_checkpoint.cc\n");
  return 1;
}
