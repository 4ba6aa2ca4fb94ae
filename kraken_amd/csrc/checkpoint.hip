// Table files in the layout of the reference's checkpoint (checkpoint/checkpoint.cc), written from
// and read into the GPU tables. Host code only: it reaches the device through the same entry
// points any other caller uses.
//
//   krk_sparse_save_file / krk_sparse_load_file   checkpoint/checkpoint.cc:465-509, 586-649  (*.sparse)
//   krk_dense_save_file  / krk_dense_load_file    checkpoint/checkpoint.cc:444-463, 535-557  (*.dense)
//
// Byte layout (common/serialize.h; every integer little-endian, no padding):
//   string          u64 length, bytes                                    serialize.h:86-94
//   map<str,str>    u64 count, then key string, value string             serialize.h:226-240
//   Shape           u64 rank, i64 dims[rank]                             serialize.h:146-148, 62-72
//   Tensor (dense)  u8 layout (0), Shape, u8 dtype (11 = fp32), data     serialize.h:156-176
//   Value           Tensor val,                                          serialize.h:296-298
//                   u64 count + {u32 StateType, Tensor} per state,       serialize.h:242-256
//                   u64 count + {u32 StateType, i64} per counter         serialize.h:258-272
//   *.sparse        u8 TableType (1), u64 id, string name, i64 dimension, u8 dtype,
//                   u8 InitializerType, map<str,str> initializer conf, u64 slot count (8),
//                   per slot: u64 rows, then {u64 id, Value} in ascending id order; an id lives
//                   in slot id % 8 (common/parallel_skip_list.h:12-21, 100-102)
//   *.dense         u8 TableType (0), u64 id, string name, Value
//
// Which states a row carries. The reference creates a state tensor the first time an optimizer
// touches the row, and the counter kSteps only under Adam (ps/optim/adam.cc:60). Here a table has
// a state column for all rows once any row needed it, so the writer emits a state for a row when
// the column exists and, if the table keeps per-row step counters, only when the row's counter
// is above zero; kSteps itself is written for tables that hold Adam's first moment. Reading is
// the inverse; a row that arrives with states but without kSteps gets the counter 1, which is
// what "this row has been updated before" means to SGD's momentum (ps/optim/sgd.cc:46-47).
#include <algorithm>
#include <fstream>
#include <string>
#include <unordered_map>
#include <vector>

#include "sparse_internal.h"

namespace krk {

constexpr uint8_t kTableDense = 0, kTableSparse = 1;   // common/info.h:40-43
constexpr uint8_t kLayoutStride = 0;                   // t/layout.h:11-14
constexpr uint8_t kDTypeFloat32 = 11;                  // t/element_type.h:23-37
constexpr uint64_t kSlotCount = 8;                     // common/parallel_skip_list.h:12-21

class FileWriter {   // checkpoint/file_writer.cc: a truncating binary stream
 public:
  explicit FileWriter(const char* path) : fs_(path, std::ios::out | std::ios::trunc | std::ios::binary) {}
  bool is_open() const { return fs_.is_open(); }
  bool bytes(const void* p, size_t n) { return (bool)fs_.write(static_cast<const char*>(p), (std::streamsize)n); }
  template <typename T>
  bool pod(T v) { return bytes(&v, sizeof(v)); }
  bool str(const std::string& s) { return pod<uint64_t>(s.size()) && bytes(s.data(), s.size()); }
  bool tensor(const float* p, const int64_t* shape, uint64_t rank, int64_t count) {
    if (!pod<uint8_t>(kLayoutStride) || !pod<uint64_t>(rank)) return false;
    for (uint64_t i = 0; i < rank; ++i)
      if (!pod<int64_t>(shape[i])) return false;
    return pod<uint8_t>(kDTypeFloat32) && bytes(p, sizeof(float) * (size_t)count);
  }
  bool row(const float* p, int64_t dim) { return tensor(p, &dim, 1, dim); }
  bool close() {
    fs_.flush();
    const bool ok = (bool)fs_;
    fs_.close();
    return ok;
  }

 private:
  std::ofstream fs_;
};

class FileReader {
 public:
  explicit FileReader(const char* path) : fs_(path, std::ios::in | std::ios::binary) {
    if (fs_.is_open()) {
      fs_.seekg(0, std::ios::end);
      size_ = (uint64_t)std::max<std::streamoff>(0, fs_.tellg());
      fs_.seekg(0, std::ios::beg);
    }
  }
  bool is_open() const { return fs_.is_open(); }
  bool bytes(void* p, size_t n) {
    if (!fs_.read(static_cast<char*>(p), (std::streamsize)n)) return false;
    at_ += n;
    return true;
  }
  // What is left of the file: no field may claim more than that, so a corrupt length can
  // neither overflow nor make this process allocate more than the file could fill.
  uint64_t left() const { return size_ - at_; }
  template <typename T>
  bool pod(T* v) { return bytes(v, sizeof(T)); }
  bool str(std::string* s) {
    uint64_t n;
    if (!pod(&n) || n > left()) return false;
    s->resize((size_t)n);
    return n == 0 || bytes(&(*s)[0], (size_t)n);
  }
  // a dense fp32 tensor of any rank, flattened; shape (may be null) receives the dims
  bool tensor(std::vector<float>* out, std::vector<int64_t>* shape) {
    uint8_t layout, dtype;
    uint64_t rank;
    if (!pod(&layout) || layout != kLayoutStride || !pod(&rank) || rank > 16) return false;
    uint64_t size = 1;
    if (shape) shape->clear();
    for (uint64_t i = 0; i < rank; ++i) {
      int64_t d;
      if (!pod(&d) || d < 0) return false;
      if (d != 0 && size > left() / (uint64_t)d) return false;   // more elements than bytes left
      size *= (uint64_t)d;
      if (shape) shape->push_back(d);
    }
    if (!pod(&dtype) || dtype != kDTypeFloat32 || size > left() / sizeof(float)) return false;
    out->resize((size_t)size);
    return size == 0 || bytes(out->data(), sizeof(float) * (size_t)size);
  }

 private:
  std::ifstream fs_;
  uint64_t size_ = 0;
  uint64_t at_ = 0;
};

// The conf map Initializer::conf() returns (ps/initializer/*_initializer.cc:11-13), values
// formatted with std::to_string as there.
static std::vector<std::pair<std::string, std::string>> initializer_conf(const krk_init& raw) {
  switch (raw.type) {
    case KRK_INIT_CONSTANT: return {{"value", std::to_string(raw.a)}};
    case KRK_INIT_UNIFORM: return {{"lower", std::to_string(raw.a)}, {"upper", std::to_string(raw.b)}};
    case KRK_INIT_NORMAL: return {{"mean", std::to_string(raw.a)}, {"stddev", std::to_string(raw.b)}};
    default: return {{"gain", std::to_string(raw.a)}};
  }
}

static int32_t io_fail(const char* what, const char* path) {
  set_error("%s: %s", what, path ? path : "(null)");
  return KRK_E_IO;
}

constexpr int64_t kChunkRows = 1 << 20;   // rows fetched from / sent to the table at a time

}  // namespace krk

using namespace krk;

extern "C" {

int32_t krk_sparse_save_file(krk_sparse* t, const char* path, uint64_t table_id, const char* name) {
  if (!t || !path || !name) return KRK_E_ARGUMENT;
  int64_t dim = 0, rows = 0;
  uint32_t mask = 0;
  KRK_TRY(krk_sparse_dim(t, &dim));
  KRK_TRY(krk_sparse_size(t, &rows));
  KRK_TRY(krk_sparse_states(t, &mask));
  FileWriter w(path);
  if (!w.is_open()) return io_fail("cannot open for writing", path);
  const auto conf = initializer_conf(t->init);
  bool ok = w.pod<uint8_t>(kTableSparse) && w.pod<uint64_t>(table_id) && w.str(name) && w.pod<int64_t>(dim) &&
            w.pod<uint8_t>(kDTypeFloat32) && w.pod<uint8_t>((uint8_t)t->init.type) && w.pod<uint64_t>(conf.size());
  for (const auto& kv : conf) ok = ok && w.str(kv.first) && w.str(kv.second);
  ok = ok && w.pod<uint64_t>(kSlotCount);
  if (!ok) return io_fail("write failed", path);

  std::vector<uint64_t> ids((size_t)rows);
  int64_t got = 0;
  if (rows) KRK_TRY(krk_sparse_export(t, ids.data(), nullptr, 1, nullptr, nullptr, rows, &got, 0));
  // slot-major, ascending inside a slot: the order ParallelSkipList is walked in
  std::sort(ids.begin(), ids.end(), [](uint64_t a, uint64_t b) {
    const uint64_t sa = a % kSlotCount, sb = b % kSlotCount;
    return sa != sb ? sa < sb : a < b;
  });
  uint64_t per_slot[kSlotCount] = {};
  for (uint64_t id : ids) per_slot[id % kSlotCount]++;

  std::vector<int> states;
  for (int st = 1; st < KRK_ST_COUNT; ++st)
    if (mask & (1u << st)) states.push_back(st);
  std::vector<char> row_has(states.size());
  const bool adam = (mask & (1u << KRK_ST_FIRST_MOMENT)) != 0;
  std::vector<float> vals;
  std::vector<std::vector<float>> st_vals(states.size());
  std::vector<int64_t> steps;
  std::vector<uint8_t> found;

  int64_t at = 0;
  for (uint64_t slot = 0; slot < kSlotCount; ++slot) {
    if (!w.pod<uint64_t>(per_slot[slot])) return io_fail("write failed", path);
    int64_t left = (int64_t)per_slot[slot];
    while (left > 0) {
      const int64_t n = std::min(left, kChunkRows);
      vals.resize((size_t)(n * dim));
      steps.resize((size_t)n);
      found.resize((size_t)n);
      KRK_TRY(krk_sparse_fetch(t, ids.data() + at, n, found.data(), vals.data(), 1, nullptr, nullptr, 0));
      KRK_TRY(sparse_fetch_words(t, ids.data() + at, n, steps.data()));
      for (size_t s = 0; s < states.size(); ++s) {
        st_vals[s].resize((size_t)(n * dim));
        KRK_TRY(krk_sparse_fetch(t, ids.data() + at, n, nullptr, nullptr, states[s], st_vals[s].data(), nullptr, 0));
      }
      for (int64_t i = 0; i < n && ok; ++i) {
        if (!found[(size_t)i]) {
          set_error("the table changed while it was being written: %s", path);
          return KRK_E_IO;
        }
        // The reference holds a state for a row once an update has created it. Here a column
        // exists for every row, so a row's state is written when it holds anything but zeros
        // (an absent state and a zero state update alike), and Adam's two moments whenever the
        // row has been counted. The counter alone does not say that a row was updated: only
        // Adam and SGD with momentum advance it.
        const bool has_momentum = ((uint64_t)steps[(size_t)i] & kHasMomentumBit) != 0;
        steps[(size_t)i] = (int64_t)((uint64_t)steps[(size_t)i] & ~kHasMomentumBit);
        const bool counter = adam && steps[(size_t)i] > 0;
        size_t emit = 0;
        for (size_t s = 0; s < states.size(); ++s) {
          const float* v = st_vals[s].data() + i * dim;
          // a row that SGD with momentum has updated holds a buffer even when it is all zeros:
          // its next update continues the buffer instead of seeding it (ps/optim/sgd.cc:46-52)
          bool any = (counter && (states[s] == KRK_ST_FIRST_MOMENT || states[s] == KRK_ST_SECOND_MOMENT)) ||
                     (has_momentum && states[s] == KRK_ST_MOMENTUM_BUFFER);
          for (int64_t j = 0; j < dim && !any; ++j) any = v[j] != 0.0f;
          row_has[s] = any;
          emit += any ? 1 : 0;
        }
        ok = w.pod<uint64_t>(ids[(size_t)(at + i)]) && w.row(vals.data() + i * dim, dim) && w.pod<uint64_t>(emit);
        for (size_t s = 0; s < states.size() && ok; ++s)
          if (row_has[s]) ok = w.pod<uint32_t>((uint32_t)states[s]) && w.row(st_vals[s].data() + i * dim, dim);
        ok = ok && w.pod<uint64_t>(counter ? 1 : 0);
        if (counter) ok = ok && w.pod<uint32_t>(KRK_ST_STEPS) && w.pod<int64_t>(steps[(size_t)i]);
      }
      if (!ok) return io_fail("write failed", path);
      at += n;
      left -= n;
    }
  }
  return w.close() ? KRK_SUCCESS : io_fail("write failed", path);
}

static int32_t sparse_load_file(krk_sparse* t, const char* path, uint64_t table_id, const char* name,
                                krk_keep_fn keep, void* keep_ctx, int64_t* rows_loaded);

int32_t krk_sparse_load_file(krk_sparse* t, const char* path, uint64_t table_id, const char* name,
                             krk_keep_fn keep, void* keep_ctx, int64_t* rows_loaded) {
  // nothing may throw across the C boundary: a file this process cannot hold is a file error
  try {
    return sparse_load_file(t, path, table_id, name, keep, keep_ctx, rows_loaded);
  } catch (const std::exception& e) {
    set_error("loading %s failed: %s", path ? path : "(null)", e.what());
    return KRK_E_IO;
  } catch (...) {
    return io_fail("loading failed", path);
  }
}

static int32_t sparse_load_file(krk_sparse* t, const char* path, uint64_t table_id, const char* name,
                                krk_keep_fn keep, void* keep_ctx, int64_t* rows_loaded) {
  if (!t || !path || !name) return KRK_E_ARGUMENT;
  if (rows_loaded) *rows_loaded = 0;
  int64_t dim = 0;
  KRK_TRY(krk_sparse_dim(t, &dim));
  FileReader r(path);
  if (!r.is_open()) return io_fail("cannot open for reading", path);
  uint8_t type, dtype, init_type;
  uint64_t file_id, n_conf, slot_count;
  std::string file_name, k, v;
  int64_t file_dim;
  bool ok = r.pod(&type) && r.pod(&file_id) && r.str(&file_name) && r.pod(&file_dim) && r.pod(&dtype) &&
            r.pod(&init_type) && r.pod(&n_conf) && n_conf < 1024;
  for (uint64_t i = 0; ok && i < n_conf; ++i) ok = r.str(&k) && r.str(&v);
  ok = ok && r.pod(&slot_count);
  if (!ok) return io_fail("truncated or malformed table file", path);
  // checkpoint/checkpoint.cc:611-616 : the file must describe this very table
  if (type != kTableSparse || file_id != table_id || file_name != name || file_dim != dim ||
      dtype != kDTypeFloat32 || init_type != (uint8_t)t->init.type) {
    set_error("%s holds another table (type %d id %llu name '%s' dimension %lld initializer %d)", path, (int)type,
              (unsigned long long)file_id, file_name.c_str(), (long long)file_dim, (int)init_type);
    return KRK_E_ARGUMENT;
  }

  std::vector<uint64_t> ids;
  std::vector<float> vals, tensor;
  std::vector<float> st_vals[KRK_ST_COUNT];
  std::vector<int64_t> steps;
  std::vector<size_t> with_momentum;   // rows of the chunk whose Value holds a momentum buffer
  uint32_t chunk_states = 0;
  int64_t loaded = 0;
  auto flush = [&]() -> int32_t {
    int64_t n = (int64_t)ids.size();
    if (n == 0) return KRK_SUCCESS;
    loaded += n;
    // checkpoint/checkpoint.cc:640 inserts whole Values with SkipList::Insert, which leaves an id
    // that is already present untouched (common/skip_list.h:240-242): weights, states and
    // counter alike. So only the ids the table does not hold yet are handed on.
    std::vector<int32_t> where((size_t)n);
    KRK_TRY(krk_sparse_lookup(t, ids.data(), n, where.data(), 0));
    size_t keep_n = 0;
    std::vector<size_t> new_index((size_t)n, (size_t)-1);
    for (size_t i = 0; i < (size_t)n; ++i) {
      if (where[i] >= 0) continue;
      new_index[i] = keep_n;
      if (keep_n != i) {
        ids[keep_n] = ids[i];
        steps[keep_n] = steps[i];
        std::copy(vals.begin() + i * dim, vals.begin() + (i + 1) * dim, vals.begin() + keep_n * dim);
        for (int st = 1; st < KRK_ST_COUNT; ++st)
          if (chunk_states & (1u << st))
            std::copy(st_vals[st].begin() + i * dim, st_vals[st].begin() + (i + 1) * dim,
                      st_vals[st].begin() + keep_n * dim);
      }
      ++keep_n;
    }
    if (keep_n != (size_t)n) {
      std::vector<size_t> moved;
      for (size_t row : with_momentum)
        if (new_index[row] != (size_t)-1) moved.push_back(new_index[row]);
      with_momentum.swap(moved);
      n = (int64_t)keep_n;
      ids.resize(keep_n);
      steps.resize(keep_n);
      vals.resize(keep_n * (size_t)dim);
      for (int st = 1; st < KRK_ST_COUNT; ++st)
        if (chunk_states & (1u << st)) st_vals[st].resize(keep_n * (size_t)dim);
    }
    if (n > 0) KRK_TRY(krk_sparse_import(t, ids.data(), n, vals.data(), 0));
    for (int st = 1; st < KRK_ST_COUNT && n > 0; ++st) {
      if (!(chunk_states & (1u << st))) continue;
      st_vals[st].resize((size_t)(n * dim), 0.0f);
      if (st == KRK_ST_MOMENTUM_BUFFER) {
        // receiving a momentum buffer marks a row as having one (SGD's first-update test), so
        // only the rows that carry it in the file are handed over; the others keep their zeros
        std::vector<uint64_t> m_ids;
        std::vector<float> m_vals;
        for (size_t row : with_momentum) {
          m_ids.push_back(ids[row]);
          m_vals.insert(m_vals.end(), st_vals[st].begin() + row * dim, st_vals[st].begin() + (row + 1) * dim);
        }
        KRK_TRY(krk_sparse_import_state(t, m_ids.data(), (int64_t)m_ids.size(), st, m_vals.data(), nullptr, 0));
      } else {
        KRK_TRY(krk_sparse_import_state(t, ids.data(), n, st, st_vals[st].data(), nullptr, 0));
      }
      st_vals[st].clear();
    }
    with_momentum.clear();
    bool any_steps = false;
    for (int64_t s : steps) any_steps = any_steps || s != 0;
    if (any_steps && n > 0) KRK_TRY(krk_sparse_import_state(t, ids.data(), n, 1, nullptr, steps.data(), 0));
    for (int st = 1; st < KRK_ST_COUNT; ++st) st_vals[st].clear();
    ids.clear();
    vals.clear();
    steps.clear();
    chunk_states = 0;
    return KRK_SUCCESS;
  };

  for (uint64_t slot = 0; slot < slot_count; ++slot) {
    uint64_t size;
    if (!r.pod(&size)) return io_fail("truncated table file", path);
    for (uint64_t i = 0; i < size; ++i) {
      uint64_t id, n_states, n_counters;
      if (!r.pod(&id) || !r.tensor(&tensor, nullptr) || (int64_t)tensor.size() != dim)
        return io_fail("truncated or malformed table file", path);
      // checkpoint/checkpoint.cc:640 : node_id == router.Hit(utils::Hash(table_id, sparse_id))
      const bool take = !keep || keep(id, keep_ctx) != 0;
      const size_t row = ids.size();
      if (take) {
        ids.push_back(id);
        vals.insert(vals.end(), tensor.begin(), tensor.end());
        steps.push_back(0);
      }
      if (!r.pod(&n_states) || n_states > 64) return io_fail("truncated or malformed table file", path);
      for (uint64_t s = 0; s < n_states; ++s) {
        uint32_t st;
        if (!r.pod(&st) || !r.tensor(&tensor, nullptr) || (int64_t)tensor.size() != dim)
          return io_fail("truncated or malformed table file", path);
        if (!take || st < 1 || st >= KRK_ST_COUNT) continue;
        chunk_states |= 1u << st;
        st_vals[st].resize(row * (size_t)dim, 0.0f);   // rows read before this state first appeared
        st_vals[st].insert(st_vals[st].end(), tensor.begin(), tensor.end());
        if (st == KRK_ST_MOMENTUM_BUFFER) with_momentum.push_back(row);
      }
      if (!r.pod(&n_counters) || n_counters > 64) return io_fail("truncated or malformed table file", path);
      for (uint64_t s = 0; s < n_counters; ++s) {
        uint32_t st;
        int64_t c;
        if (!r.pod(&st) || !r.pod(&c)) return io_fail("truncated table file", path);
        if (take && st == KRK_ST_STEPS) steps[row] = c;
      }
      if (take) {
        for (int st = 1; st < KRK_ST_COUNT; ++st)   // rows without a state the chunk has seen: zeros
          if (chunk_states & (1u << st)) st_vals[st].resize(ids.size() * (size_t)dim, 0.0f);
        if ((int64_t)ids.size() >= kChunkRows) KRK_TRY(flush());
      }
    }
  }
  KRK_TRY(flush());
  if (rows_loaded) *rows_loaded = loaded;
  return KRK_SUCCESS;
}

int32_t krk_dense_save_file(krk_dense* t, const char* path, uint64_t table_id, const char* name,
                            const int64_t* shape, int32_t rank) {
  if (!t || !path || !name || rank < 0 || rank > 16 || (rank > 0 && !shape)) return KRK_E_ARGUMENT;
  int64_t n = 0, steps = 0;
  uint32_t mask = 0;
  KRK_TRY(krk_dense_size(t, &n));
  KRK_TRY(krk_dense_states(t, &mask));
  KRK_TRY(krk_dense_steps(t, &steps));
  int64_t flat[1] = {n};
  if (rank == 0) {
    shape = flat;
    rank = 1;
  }
  int64_t count = 1;
  for (int32_t i = 0; i < rank; ++i) count *= shape[i];
  if (count != n) {
    set_error("shape does not hold the table's %lld elements", (long long)n);
    return KRK_E_ARGUMENT;
  }
  std::vector<float> buf((size_t)n);
  KRK_TRY(krk_dense_pull(t, buf.data(), 0));
  FileWriter w(path);
  if (!w.is_open()) return io_fail("cannot open for writing", path);
  uint64_t n_states = 0;
  for (int st = 1; st < KRK_ST_COUNT; ++st) n_states += (mask >> st) & 1u;
  bool ok = w.pod<uint8_t>(kTableDense) && w.pod<uint64_t>(table_id) && w.str(name) &&
            w.tensor(buf.data(), shape, (uint64_t)rank, n) && w.pod<uint64_t>(n_states);
  for (int st = 1; st < KRK_ST_COUNT && ok; ++st) {
    if (!(mask & (1u << st))) continue;
    KRK_TRY(krk_dense_state(t, st, buf.data(), 0));
    ok = w.pod<uint32_t>((uint32_t)st) && w.tensor(buf.data(), shape, (uint64_t)rank, n);
  }
  const bool counter = steps > 0 && (mask & (1u << KRK_ST_FIRST_MOMENT));
  ok = ok && w.pod<uint64_t>(counter ? 1 : 0);
  if (counter) ok = ok && w.pod<uint32_t>(KRK_ST_STEPS) && w.pod<int64_t>(steps);
  return ok && w.close() ? KRK_SUCCESS : io_fail("write failed", path);
}

static int32_t dense_load_file(const char* path, krk_dense** out, uint64_t* table_id, char* name, size_t name_cap,
                               int64_t* shape, int32_t* rank);

int32_t krk_dense_load_file(const char* path, krk_dense** out, uint64_t* table_id, char* name, size_t name_cap,
                            int64_t* shape, int32_t* rank) {
  try {
    return dense_load_file(path, out, table_id, name, name_cap, shape, rank);
  } catch (const std::exception& e) {
    set_error("loading %s failed: %s", path ? path : "(null)", e.what());
    return KRK_E_IO;
  } catch (...) {
    return io_fail("loading failed", path);
  }
}

static int32_t dense_load_file(const char* path, krk_dense** out, uint64_t* table_id, char* name, size_t name_cap,
                               int64_t* shape, int32_t* rank) {
  if (!path || !out) return KRK_E_ARGUMENT;
  *out = nullptr;
  FileReader r(path);
  if (!r.is_open()) return io_fail("cannot open for reading", path);
  uint8_t type;
  uint64_t file_id, n_states, n_counters;
  std::string file_name;
  std::vector<float> val, tensor;
  std::vector<int64_t> dims;
  if (!r.pod(&type) || !r.pod(&file_id) || !r.str(&file_name) || !r.tensor(&val, &dims))
    return io_fail("truncated or malformed table file", path);
  if (type != kTableDense) {
    set_error("%s does not hold a dense table", path);
    return KRK_E_ARGUMENT;
  }
  if (table_id) *table_id = file_id;
  if (name && name_cap) {
    const size_t n = std::min(name_cap - 1, file_name.size());
    memcpy(name, file_name.data(), n);
    name[n] = 0;
  }
  if (rank) {
    const int32_t cap = *rank;
    *rank = (int32_t)dims.size();
    if (shape)
      for (int32_t i = 0; i < cap && i < (int32_t)dims.size(); ++i) shape[i] = dims[(size_t)i];
  }
  krk_dense* t = nullptr;
  KRK_TRY(krk_dense_create(val.data(), (int64_t)val.size(), 0, &t));
  auto fail = [&](int32_t code) {
    krk_dense_destroy(t);
    return code;
  };
  if (!r.pod(&n_states) || n_states > 64) return fail(io_fail("truncated or malformed table file", path));
  for (uint64_t s = 0; s < n_states; ++s) {
    uint32_t st;
    if (!r.pod(&st) || !r.tensor(&tensor, nullptr) || tensor.size() != val.size())
      return fail(io_fail("truncated or malformed table file", path));
    if (st < 1 || st >= KRK_ST_COUNT) continue;
    const int32_t rc = krk_dense_import_state(t, (int32_t)st, tensor.data(), -1, 0);
    if (rc != KRK_SUCCESS) return fail(rc);
  }
  if (!r.pod(&n_counters) || n_counters > 64) return fail(io_fail("truncated or malformed table file", path));
  for (uint64_t s = 0; s < n_counters; ++s) {
    uint32_t st;
    int64_t c;
    if (!r.pod(&st) || !r.pod(&c)) return fail(io_fail("truncated table file", path));
    if (st == KRK_ST_STEPS) {
      const int32_t rc = krk_dense_import_state(t, 1, nullptr, c, 0);
      if (rc != KRK_SUCCESS) return fail(rc);
    }
  }
  *out = t;
  return KRK_SUCCESS;
}

}  // extern "C"
