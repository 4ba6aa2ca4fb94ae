/*
 * kraken_hip.h -- C ABI of the MI355X table engine behind Kraken's parameter-server tables.
 *
 * Every entry point returns one of Kraken's ErrorCode values
 * (kraken/common/error_code.h:7-33; 0 = success) or a negative KRK_E_* for
 * conditions the reference cannot have (device failures). Nothing throws
 * across this boundary; krk_last_error_string() describes the last failure on
 * the calling thread. Reference citations are relative to the reference
 * tree's kraken/ directory.
 *
 * Pointer arguments are host pointers unless KRK_DEVICE_PTRS is set in
 * `flags`, in which case every data pointer of that call (ids, rows,
 * gradients, outputs) is a device pointer on the table's GPU. Calls are
 * blocking unless KRK_ASYNC is also set (device pointers only): the work is
 * then only enqueued on the table's stream and a failure is reported by the
 * next blocking call or by the object's *_sync() function.
 *
 * Stream capture: do not record these calls into a HIP graph. Every launch that may insert
 * rows carries a launch number chosen on the host, and a replayed launch would present an old
 * number, under which rows created since would be taken for rows still being created.
 *
 * Threading: any number of host threads may call into one table; calls on one
 * table are serialised (the reference takes a unique lock per slot for Pull
 * and Push alike, ps/sparse_table.cc:48,88, and a unique lock for a dense
 * Push, ps/dense_table.cc:40).
 */
#ifndef KRAKEN_HIP_H_
#define KRAKEN_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define KRK_VERSION 1

/* flags */
#define KRK_DEVICE_PTRS 0x1u
#define KRK_ASYNC 0x2u
/* A worker pulls the rows of a batch's ids and, after its backward pass, pushes gradients for
 * the same ids (worker/emitter.cc:131-182 then :510-531; :552-612 for combined requests). The
 * two flags below let the second call reuse what the first one found. Both need
 * KRK_DEVICE_PTRS and are ignored by every other call.
 * KRK_NOTE_ROWS on krk_sparse_pull / krk_group_pull: the table (group) also keeps the row
 * number of every position of this request (4 bytes a position, in memory of its own) until
 * its next pull with the flag; single-table requests of 2^18 ids and more are not noted.
 * KRK_IDS_AS_PULLED on krk_sparse_push / krk_sparse_push_raw / krk_group_push /
 * krk_group_push_raw: the caller states that `ids` is the buffer of that pull (same pointer,
 * same counts) with its contents unchanged. The call then skips its own look-up of the ids
 * (push_raw: for requests of at most 8192 ids a table, where the look-up is a launch of its
 * own). It looks the ids up as usual when the pointer or the counts differ from what was
 * noted, when nothing was noted, or when rows have moved since (krk_sparse_erase, a table that
 * grew or gained optimizer columns). Results are the same either way; ids whose contents did
 * change give the updates of the old ids' rows. */
#define KRK_NOTE_ROWS 0x4u
#define KRK_IDS_AS_PULLED 0x8u

/* kraken/common/error_code.h:7-33 */
#define KRK_SUCCESS 0
#define KRK_UNSUPPORTED_OPTIM 6
#define KRK_INTERFACE_UNIMPLEMENTED 10
#define KRK_GRADIENT_UNCOMPATIBLE 11
#define KRK_SPARSE_ID_NOT_EXIST 12
#define KRK_UNSUPPORTED_INITIALIZER 13
/* no reference counterpart */
#define KRK_E_DEVICE (-2)       /* a HIP call failed, or no usable GPU            */
#define KRK_E_ARGUMENT (-3)     /* null handle, negative size, bad flag           */
#define KRK_E_CAPACITY (-4)     /* output buffer too small / table cannot grow    */
#define KRK_E_IO (-5)           /* a table file could not be opened, read or written */

/* kraken/common/info.h:46-72 */
enum { KRK_ADAGRAD = 0, KRK_ADAM = 1, KRK_RMSPROP = 2, KRK_SGD = 3 };
enum {
  KRK_INIT_CONSTANT = 0,
  KRK_INIT_UNIFORM = 1,
  KRK_INIT_NORMAL = 2,
  KRK_INIT_XAVIER_UNIFORM = 3,
  KRK_INIT_XAVIER_NORMAL = 4
};
enum {
  KRK_ST_STEPS = 0,
  KRK_ST_MOMENTUM_BUFFER = 1,
  KRK_ST_STATE_SUM = 2,
  KRK_ST_FIRST_MOMENT = 3,
  KRK_ST_SECOND_MOMENT = 4,
  KRK_ST_SECOND_MOMENT_MAX = 5,
  KRK_ST_SQUARE_AVERAGE = 6,
  KRK_ST_G_AVE = 7,
  KRK_ST_COUNT = 8
};

/* Flattened Optim::Create (ps/optim/optim.cc:18-105): the has_* flags are what
 * the presence of a conf key sets there. initial_accumulator has no reference
 * counterpart (Adagrad's state_sum always starts at zero, ps/optim/adagrad.cc:34-36);
 * it is added to the stored sum when the denominator is formed and must be 0
 * for reference behaviour. */
typedef struct krk_optim {
  int32_t type;
  int32_t has_weight_decay;
  float weight_decay;
  int32_t has_momentum;
  float momentum;
  int32_t has_dampening;
  float dampening;
  int32_t nesterov;
  float beta1;
  float beta2;
  float eps;
  int32_t amsgrad;
  float alpha;
  int32_t centered;
  float initial_accumulator;
} krk_optim;

/* Fills the defaults of ps/optim/optim.cc:23-101 for `type`. */
int32_t krk_optim_defaults(int32_t type, krk_optim* o);
/* Applies one "key=value" conf entry the way Optim::Create + utils::ParseConf
 * (common/utils.h:50-92) do; unknown keys are ignored, unparsable floats leave
 * the default, as in the reference. */
int32_t krk_optim_set(krk_optim* o, const char* key, const char* value);

/* Flattened Initializer::Create (ps/initializer/initializer.cc:22-61).
 * a,b = value,- | lower,upper | mean,stddev | gain,- | gain,- .
 * Random initialisers are counter based: a row's values depend only on
 * (seed, id, element), never on arrival order. The reference seeds from
 * std::random_device per call (t/math.cc:455-464), so only the distribution
 * can match. */
typedef struct krk_init {
  int32_t type;
  float a;
  float b;
  uint64_t seed;
} krk_init;
int32_t krk_init_defaults(int32_t type, krk_init* i);
int32_t krk_init_set(krk_init* i, const char* key, const char* value);

/* ---- runtime ------------------------------------------------------------- */
/* Selects the GPU used by objects created afterwards on this thread's process
 * (default 0). Fails with KRK_E_DEVICE when no gfx950 device is usable. */
int32_t krk_runtime_init(int32_t device);
const char* krk_last_error_string(void);
const char* krk_error_message(int32_t code);   /* ErrorCode::Msg, common/error_code.h:35-93 */
/* Harness helpers: device buffers and timing without any other GPU library. */
int32_t krk_malloc(void** dptr, size_t bytes);
int32_t krk_free(void* dptr);
/* Page-locked host memory. Host-pointer calls copy to and from the caller's buffers; when those
 * are pageable the copies are staged through the runtime's bounce buffers (about 5 GB/s towards
 * the host), when they come from here the GPU's copy engines reach them directly. A server
 * that receives requests and builds replies in buffers of its own should take them from here. */
int32_t krk_host_malloc(void** hptr, size_t bytes);
int32_t krk_host_free(void* hptr);
int32_t krk_memcpy_h2d(void* dst, const void* src, size_t bytes);
int32_t krk_memcpy_d2h(void* dst, const void* src, size_t bytes);
int32_t krk_memset(void* dptr, int value, size_t bytes);
int32_t krk_device_synchronize(void);
int32_t krk_mem_info(size_t* free_bytes, size_t* total_bytes);
/* A plain device-to-device streaming copy kernel on the null stream (not synchronised): the
 * measured bandwidth ceiling, and the known-size kernel byte counters are calibrated against.
 * Pointers and size must be multiples of 16. */
int32_t krk_stream_copy(void* dst, const void* src, size_t bytes);
/* The measured ceilings the table kernels are compared with (no reference counterpart; null
 * stream, not synchronised; time them with events on the null stream).
 * krk_hbm_probe: one streaming pass over `bytes` bytes: kind 0 reads src, 1 fills dst, 2 copies
 * src to dst; unroll = independent 16-byte accesses in flight per lane (1, 2, 4, 8);
 * nontemporal != 0 gives them the streaming hint; blocks = workgroups of 256 lanes. dst is
 * needed by every kind (the read-only kind never writes it). Pointers and size multiples of 16.
 * krk_hbm_probe_lines: n random, independent 128-byte lines inside base[0, region_bytes) (the
 * largest power-of-two number of lines that fits), eight lanes a line, read only (rmw == 0) or
 * read, changed and written back (rmw != 0): what a table kernel does per row, without the
 * index. salt picks the lines. base must be 128-byte aligned. */
int32_t krk_hbm_probe(int32_t kind, int32_t unroll, int32_t nontemporal, int32_t blocks, void* dst,
                      const void* src, size_t bytes);
int32_t krk_hbm_probe_lines(int32_t rmw, void* base, size_t region_bytes, int64_t n, uint64_t salt);

/* ---- sparse table --------------------------------------------------------- */
typedef struct krk_sparse krk_sparse;

/* SparseTable ctor (ps/sparse_table.cc:7-16) + Initializer::Create.
 * capacity_hint = expected number of rows (0 = small default); the table grows
 * on demand. Element type is fp32 (t/element_type.h code 11). */
int32_t krk_sparse_create(int64_t dim, const krk_init* init, int64_t capacity_hint,
                          krk_sparse** out);
int32_t krk_sparse_destroy(krk_sparse* t);
int32_t krk_sparse_dim(krk_sparse* t, int64_t* dim);
int32_t krk_sparse_size(krk_sparse* t, int64_t* rows);
/* Makes room for `rows` rows up front so that later pulls never reallocate. */
int32_t krk_sparse_reserve(krk_sparse* t, int64_t rows);
/* Waits for enqueued work and returns the first deferred error (then clears it). */
int32_t krk_sparse_sync(krk_sparse* t);
/* Makes the table enqueue its work on the caller's HIP stream (a hipStream_t) instead of its
 * own, so that KRK_ASYNC calls are ordered with the caller's other work on that stream: a
 * training framework passes the stream its tensors are produced and consumed on. NULL is a
 * stream like any other: HIP's default (null) stream, which is what a framework's "current
 * stream" handle is until the user switches streams. KRK_OWN_STREAM returns to the stream
 * created with the table (which does not wait for the null stream, nor the null stream for it).
 * Work already enqueued is waited for first. The stream must outlive its use by the table;
 * tables that belong to a group cannot switch. No reference counterpart. */
#define KRK_OWN_STREAM ((void*)(intptr_t)-1)
int32_t krk_sparse_set_stream(krk_sparse* t, void* stream);

/* SparseTable::Pull (ps/sparse_table.cc:33-75): out[i,:] = row of ids[i];
 * a missing id is inserted with the table's initializer and returned. ids may
 * repeat. out is [n, dim] contiguous. */
int32_t krk_sparse_pull(krk_sparse* t, const uint64_t* ids, int64_t n, float* out,
                        uint32_t flags);
/* SparseTable::Push (ps/sparse_table.cc:77-108) + Optim::Update on each row.
 * ids must be unique (the worker guarantees it, worker/emitter.cc:516-531).
 * grad_dim != dim returns 11 and changes nothing. A missing id returns 12;
 * rows whose ids exist are still updated (the reference stops at the first
 * missing id in an unspecified visiting order). */
int32_t krk_sparse_push(krk_sparse* t, const krk_optim* o, const uint64_t* ids, int64_t n,
                        const float* grads, int64_t grad_dim, float lr, uint32_t flags);
/* The worker-side half fused in front of Push: Emitter::PushSparseTable's
 * dedup + duplicate-gradient sum (worker/emitter.cc:510-531) followed by
 * SparseTable::Push, without materialising the unique list. ids may repeat;
 * grads is [n, grad_dim]. */
int32_t krk_sparse_push_raw(krk_sparse* t, const krk_optim* o, const uint64_t* ids, int64_t n,
                            const float* grads, int64_t grad_dim, float lr, uint32_t flags);

/* ---- multi-hot fields: Pull / Push fused with the worker's jagged pooling ---
 * A field holds `bags` bags; bag i owns ids[offsets[i] .. offsets[i+1]), offsets is
 * [bags + 1], starts at 0 and ends at n (checked when the pointers are host pointers;
 * device offsets are clamped to [0, n] and ids outside every bag are ignored).
 * weights is NULL or [n]: the per-id factors of JaggedTensor.weights()
 * (pytorch/jagged_embedding.py:41-45). */
#define KRK_POOL_SUM 0
#define KRK_POOL_MEAN 1
/* SparseTable::Pull (ps/sparse_table.cc:33-75, ids inserted when absent) followed by
 * jagged::SumForward / MeanForward (pytorch/py/jagged_ops.cc:14-56, 206-236) in one pass:
 * out[i] = row(first id) (* weight), then the bag's other rows added in position order; mean
 * multiplies by (float)(1.0 / float(len)); an empty bag yields patch_value. out is
 * [bags, dim]. The n pulled rows are never written out. Rows wider than 256 floats (64 when
 * dim is not a multiple of 4) return 10. */
int32_t krk_sparse_pull_pooled(krk_sparse* t, const uint64_t* ids, int64_t n, const int64_t* offsets,
                               int64_t bags, const float* weights, int32_t mode, float patch_value,
                               float* out, uint32_t flags);
/* The backward of the above fused with krk_sparse_push_raw: position p of bag i carries the
 * gradient bag_grads[i] (sum) or bag_grads[i] * (float)(1.0 / float(len)) (mean,
 * pytorch/py/jagged_ops.cc:303-334), times weights[p] when given; gradients of equal ids are
 * summed and each row is updated once, as in krk_sparse_push_raw. The [n, dim] per-position
 * gradient is never materialised. For the sum this is the transpose of the forward, which is
 * what pytorch/py/jagged_ops.cc:148-160 is meant to be (as written it fills only the first row
 * of each bag). bag_grads is [bags, grad_dim]. */
int32_t krk_sparse_push_pooled(krk_sparse* t, const krk_optim* o, const uint64_t* ids, int64_t n,
                               const int64_t* offsets, int64_t bags, const float* weights, int32_t mode,
                               const float* bag_grads, int64_t grad_dim, float lr, uint32_t flags);
/* The reply and the gradients of a sparse request in the reference's wire layout, so that a
 * server can hand its send and receive buffers over as they are: std::vector<Tensor> as
 * Serialize writes it (common/serialize.h:156-176, 214-228) = u64 count, then per row 18 header
 * bytes {u8 layout 0, u64 rank 1, i64 dim, u8 dtype 11} and dim floats. This is the body of a
 * PullSparseTableResponse (protocol/pull_sparse_table_prot.h:29-41) and the `grads` member of a
 * PushSparseTableRequest (protocol/push_sparse_table_prot.h:11-30). Host buffers, 8-byte
 * aligned, blocking; page-locked buffers are read and written in place.
 *   krk_wire_rows_bytes   size of such a block for n rows
 *   krk_sparse_pull_wire  krk_sparse_pull whose reply is that block (reply holds
 *                         krk_wire_rows_bytes(n, dim) bytes)
 *   krk_sparse_push_wire  krk_sparse_push whose gradients are that block; a count other than n, a
 *                         header that is not a dense fp32 vector of the table's width or a short
 *                         buffer returns 11 before any row is touched (the reference fails at
 *                         the offending row, after updating those before it). */
int64_t krk_wire_rows_bytes(int64_t n, int64_t dim);
int32_t krk_sparse_pull_wire(krk_sparse* t, const uint64_t* ids, int64_t n, void* reply);
int32_t krk_sparse_push_wire(krk_sparse* t, const krk_optim* o, const uint64_t* ids, int64_t n,
                             const void* grads_wire, int64_t wire_bytes, float lr);
/* id -> row lookup alone (ParallelSkipList::HitSlot + SkipList::Find,
 * common/parallel_skip_list.h:100-102, common/skip_list.h:315-324):
 * rows[i] = dense row index of ids[i], or -1 when absent. Row indices are
 * assigned in insertion order and have no reference analogue; hit/miss does. */
int32_t krk_sparse_lookup(krk_sparse* t, const uint64_t* ids, int64_t n, int32_t* rows,
                          uint32_t flags);
/* Bulk insert of explicit rows (SkipList::Insert semantics: an id that is
 * already present keeps its row, common/skip_list.h:237-243). vals is [n, dim]. */
int32_t krk_sparse_import(krk_sparse* t, const uint64_t* ids, int64_t n, const float* vals,
                          uint32_t flags);
/* Dump for the users of SparseTable::mutable_vals() (checkpoint/checkpoint.cc:465-509):
 * rows in insertion order. Any of ids/vals/state/steps may be NULL. state_type
 * selects which optimizer state fills `state` (zeros when it was never
 * created); steps is Adam's per-row counter. capacity = rows the buffers hold. */
int32_t krk_sparse_export(krk_sparse* t, uint64_t* ids, float* vals, int32_t state_type,
                          float* state, int64_t* steps, int64_t capacity, int64_t* rows,
                          uint32_t flags);
/* Ps::TryFetchSparseValues (ps/ps.cc:914-935) and the transfer-out walk (ps/ps.cc:289-321):
 * the Values of the ids that exist; nothing is inserted. found[i] = 1 where ids[i] is present;
 * vals / state are [n, dim] (zero rows for absent ids), steps is [n]. Any output may be NULL.
 * Blocking. */
int32_t krk_sparse_fetch(krk_sparse* t, const uint64_t* ids, int64_t n, uint8_t* found, float* vals,
                         int32_t state_type, float* state, int64_t* steps, uint32_t flags);
/* Which parts of a Value the table's rows carry besides the weights (common/info.h:74-92):
 * bit st is set when optimizer state st exists, bit 0 when rows keep a step counter. What a
 * checkpoint writer has to walk (checkpoint/checkpoint.cc:465-509). */
int32_t krk_sparse_states(krk_sparse* t, uint32_t* mask);
/* The rest of a Value for rows brought in with krk_sparse_import (transfer-in ps/ps.cc:789-792,
 * checkpoint load checkpoint/checkpoint.cc:620-645): one optimizer state [n, dim] and / or the
 * per-row step counters [n]. Either may be NULL. An id that is not in the table returns 12 and
 * leaves the other rows written. The counter is Adam's (StateType::kSteps, ps/optim/adam.cc:60).
 * A row that is handed a momentum buffer (state_type 1) is from then on a row that has one: SGD
 * with momentum seeds the buffer from the gradient only on rows that have none
 * (ps/optim/sgd.cc:46-52), so a loader hands momentum buffers over for exactly the rows whose
 * Value holds one. */
int32_t krk_sparse_import_state(krk_sparse* t, const uint64_t* ids, int64_t n, int32_t state_type,
                                const float* state, const int64_t* steps, uint32_t flags);
/* The clean-up after a cluster change (ps/ps.cc:92-109: SkipList::Remove on every row routed
 * elsewhere). The caller names the rows that go: krk_sparse_select_routed picks them by the
 * reference's routing rule on the device, or the host decides from krk_sparse_export's ids.
 * Ids that are not present are ignored; *erased (may be NULL) receives how many rows went. Rows stay densely numbered, so the row numbers
 * krk_sparse_lookup reports change. Costs a pass over the whole index; blocking. */
int32_t krk_sparse_erase(krk_sparse* t, const uint64_t* ids, int64_t n, int64_t* erased,
                         uint32_t flags);
/* The ids of the rows that Router::Hit(utils::Hash(table_id, sparse_id)) (common/router.cc:262-277,
 * common/utils.h:30-48) gives to node_id (owned != 0: the transfer-out walk, ps/ps.cc:289-321,
 * with the target's id) or to any other node (owned == 0: the clean-up, ps/ps.cc:92-109, with
 * this server's id), in row order (krk_sparse_export's), decided on the device from the table's
 * own keys. The ring is Router::vnodes() as two HOST arrays whatever the flags say: hash_v in
 * ascending order and the node id of each virtual node; an empty ring owns nothing. ids holds
 * `capacity` entries; *count receives how many were selected; KRK_E_CAPACITY (nothing written,
 * *count = the room needed) when capacity is too small. Feed the ids to krk_sparse_fetch /
 * krk_sparse_erase. Blocking. */
int32_t krk_sparse_select_routed(krk_sparse* t, uint64_t table_id, const uint64_t* ring_hash,
                                 const uint64_t* ring_node, int64_t ring_n, uint64_t node_id,
                                 int32_t owned, uint64_t* ids, int64_t capacity, int64_t* count,
                                 uint32_t flags);

/* The worker's routing of a request (Emitter::PullSparseTableImpl, worker/emitter.cc:139-149; push
 * :516-531; combined :221-233, 595-606): every id goes to the server that
 * Router::Hit(utils::Hash(table_id, sparse_id)) names (common/router.cc:262-277,
 * common/utils.h:30-48), and each server's request lists its ids in the order the worker met them.
 * Call it on the unique ids krk_dedup returns, as the reference routes after its dedup, so that a
 * hot id is routed once. The ring is Router::vnodes() as two HOST arrays whatever the flags say
 * (hash_v ascending, node id of each virtual node; at most 256 distinct nodes).
 *   node_ids[k], counts[k]  (host, node_capacity entries) the ring's nodes in ascending id order
 *                           and how many of the ids each owns; *n_nodes = how many nodes
 *   owner[p]                (may be NULL) the node id that owns ids[p]
 *   perm[n]                 the positions grouped by owner in node_ids order, position order kept
 *                           inside a group (a stable partition): node k's request is ids[perm[j]]
 *                           for j in [counts[0] + .. + counts[k-1], .. + counts[k])
 * Blocking. KRK_E_CAPACITY when node_capacity is too small (*n_nodes = the room needed). */
int32_t krk_route_ids(uint64_t table_id, const uint64_t* ring_hash, const uint64_t* ring_node, int64_t ring_n,
                      const uint64_t* ids, int64_t n, uint64_t* owner, int64_t* perm, uint64_t* node_ids,
                      int64_t* counts, int64_t node_capacity, int64_t* n_nodes, uint32_t flags);

/* ---- table files ------------------------------------------------------------- */
/* Checkpoint::SaveSparseTable (checkpoint/checkpoint.cc:465-509): the table as a *.sparse file in
 * the reference's byte layout (common/serialize.h), rows grouped by id % 8 and ascending inside
 * a group, each a Value (weights, the optimizer states the row carries, Adam's step counter).
 * table_id and name are the ones the reference's Table holds (ps/table.h:13-19). */
int32_t krk_sparse_save_file(krk_sparse* t, const char* path, uint64_t table_id, const char* name);
/* Checkpoint::LoadSparseTable (checkpoint/checkpoint.cc:586-649): inserts the file's rows. The
 * file must describe this table (type, id, name, dimension, element type, initializer type),
 * otherwise KRK_E_ARGUMENT. keep (may be NULL = every row) stands for the routing test
 * node_id == router.Hit(utils::Hash(table_id, sparse_id)) of line 640: a row is taken when it
 * returns non-zero. *rows_loaded (may be NULL) receives the rows taken. */
typedef int32_t (*krk_keep_fn)(uint64_t sparse_id, void* ctx);
int32_t krk_sparse_load_file(krk_sparse* t, const char* path, uint64_t table_id, const char* name,
                             krk_keep_fn keep, void* keep_ctx, int64_t* rows_loaded);

/* ---- groups of sparse tables: one combined request, one launch -------------- */
typedef struct krk_group krk_group;
/* The tables of a model that are pulled and pushed together
 * (CombinePullSparseTableRequest / CombinePushSparseTableRequest,
 * protocol/combine_pull_sparse_table_prot.h:13-33, combine_push_sparse_table_prot.h:12-33).
 * Members (1..32) must have equal dimension and belong to no other group. While the group
 * exists its members run on the group's stream, so single-table calls on a member stay
 * ordered with the group's calls. Destroy the group before its tables. */
int32_t krk_group_create(krk_sparse** tables, int32_t n, krk_group** out);
int32_t krk_group_destroy(krk_group* g);
int32_t krk_group_sync(krk_group* g);
/* Ps::CombinePullSparseTable (ps/ps_op.cc:370-387): the reference loops over the tables of the
 * request; here all of them are served by one launch. ids is the concatenation of every
 * table's ids in member order, offsets[n+1] (host memory, offsets[0] = 0) delimits them, out is
 * [offsets[n], dim]. Per table the semantics are krk_sparse_pull's. */
int32_t krk_group_pull(krk_group* g, const uint64_t* ids, const int64_t* offsets, float* out,
                       uint32_t flags);
/* Ps::CombinePushSparseTable (ps/ps_op.cc:456-469) with one optimizer for the whole model
 * (Ps::CreateModel, ps/ps.cc:604-633). ids unique within each table; grads is
 * [offsets[n], grad_dim]. Per table the semantics are krk_sparse_push's; the reference
 * returns at the first failing table, here every table is processed and the first error code
 * in member order is returned. */
int32_t krk_group_push(krk_group* g, const krk_optim* o, const uint64_t* ids, const int64_t* offsets,
                       const float* grads, int64_t grad_dim, float lr, uint32_t flags);
/* Emitter::CombinePushSparseTable's dedup + duplicate-gradient sum over (table, id) pairs
 * (worker/emitter.cc:552-606) fused with krk_group_push: ids may repeat within a table, the
 * gradients of equal ids are summed in position order and the optimizer runs once per distinct
 * row. One sort and one segmented reduction serve all members. The members' row capacities and
 * the member count must fit a 32-bit sort key together (KRK_E_CAPACITY otherwise: 32 tables of
 * up to 2^26 rows each, fewer tables for larger ones), at most 2^28 ids per call. Errors as
 * krk_group_push. */
int32_t krk_group_push_raw(krk_group* g, const krk_optim* o, const uint64_t* ids, const int64_t* offsets,
                           const float* grads, int64_t grad_dim, float lr, uint32_t flags);
/* krk_sparse_set_stream for a group and all its members. */
int32_t krk_group_set_stream(krk_group* g, void* stream);

/* Emitter::PullSparseTableImpl's dedup (worker/emitter.cc:131-149): unique ids
 * in first-occurrence order, inv[p] = index of ids[p] in uids. uids and inv
 * hold n entries; *n_unique receives U. */
int32_t krk_dedup(const uint64_t* ids, int64_t n, uint64_t* uids, int64_t* inv,
                  int64_t* n_unique, uint32_t flags);

/* krk_dedup for callers that cannot allocate device memory (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc). No counterpart in the reference. Every pointer
 * is a device pointer, n_unique included (one int64, written on the device); the launches are
 * enqueued on `stream` (a hipStream_t, NULL = the null stream) and the call returns without
 * waiting. The work space (request-local index, per-position arrays, scan sums) is a fixed array
 * of about 11.5 MB inside the library image, held by each GPU the library runs on until the
 * process ends; more than KRK_DEDUP_NOALLOC_MAX ids return KRK_E_CAPACITY. The array is shared by
 * all calls on a GPU: calls that overlap there (two streams, two threads) race. Results are
 * those of krk_dedup. inv may be NULL. */
#define KRK_DEDUP_NOALLOC_MAX (1 << 18)
int32_t krk_dedup_noalloc(const uint64_t* ids, int64_t n, uint64_t* uids, int64_t* inv,
                          int64_t* n_unique, void* stream);

/* Emitter::PushSparseTable's dedup + sum as a call of its own (worker/emitter.cc:510-531), for a
 * worker whose server is elsewhere: uids as krk_dedup, sums[u, :] = the gradient rows of unique
 * id u added in position order starting from a copy of the first. grads is [n, dim]; sums needs
 * room for n rows, *n_unique of them are written. inv may be NULL. Blocking. */
int32_t krk_dedup_sum(const uint64_t* ids, int64_t n, const float* grads, int64_t dim, uint64_t* uids,
                      int64_t* inv, float* sums, int64_t* n_unique, uint32_t flags);
/* The re-expansion after a pull of unique ids (worker/emitter.cc:162-182): out[p, :] =
 * rows[inv[p], :]. rows is [n_rows, dim], out [n, dim]. An index outside rows returns
 * KRK_E_ARGUMENT (those output rows are zero). Blocking. */
int32_t krk_expand_rows(const float* rows, int64_t n_rows, const int64_t* inv, int64_t n, int64_t dim,
                        float* out, uint32_t flags);

/* ---- dense table ---------------------------------------------------------- */
typedef struct krk_dense krk_dense;
/* DenseTable ctor (ps/dense_table.cc:10-13): the table starts as a copy of val[n]. */
int32_t krk_dense_create(const float* val, int64_t n, uint32_t flags, krk_dense** out);
int32_t krk_dense_destroy(krk_dense* t);
int32_t krk_dense_sync(krk_dense* t);
int32_t krk_dense_pull(krk_dense* t, float* out, uint32_t flags);      /* ps/dense_table.cc:31-37 */
/* DenseTable::Push (ps/dense_table.cc:39-43); n != table size returns 11. A device gradient
 * must be 16-byte aligned (KRK_E_ARGUMENT otherwise), as every device row buffer of the sparse
 * calls must. */
int32_t krk_dense_push(krk_dense* t, const krk_optim* o, const float* grad, int64_t n, float lr,
                       uint32_t flags);
/* COO gradient (values + int64 flat indices, as ToCoo emits them): densified
 * like CooTensorImpl::ToDense (t/coo_tensor_impl.cc:250-260, repeated indices
 * add up) and applied; nnz == 0 returns success without touching any state
 * (ps/optim/adam.cc:25-29). */
int32_t krk_dense_push_coo(krk_dense* t, const krk_optim* o, const int64_t* idx, const float* val,
                           int64_t nnz, float lr, uint32_t flags);
/* Optimizer state for parity dumps; zeros when never created. */
int32_t krk_dense_state(krk_dense* t, int32_t state_type, float* out, uint32_t flags);
int32_t krk_dense_steps(krk_dense* t, int64_t* steps);
int32_t krk_dense_size(krk_dense* t, int64_t* n);
/* Same bit mask as krk_sparse_states for the dense table's one Value. */
int32_t krk_dense_states(krk_dense* t, uint32_t* mask);
/* Restores one optimizer state [n] (may be NULL) and / or Adam's step counter (steps < 0
 * leaves it) of a table built from a saved Value (checkpoint/checkpoint.cc:535-557). */
int32_t krk_dense_import_state(krk_dense* t, int32_t state_type, const float* state, int64_t steps,
                               uint32_t flags);
/* Several dense tables served by one launch. Ps::CombinePullDenseTable (ps/ps_op.cc:177-252) pulls
 * every dense parameter of a model in one request, which the worker issues after every step
 * (pytorch/optimizer.py:151-173): pull writes the members' values one after the other, in member
 * order, into out[sum of sizes]. push applies Optim::Update to every member with its part of
 * grads[n] laid out the same way (the loop of Ps::PushDenseTable calls, ps/ps_op.cc:254-300, that a
 * step's gradient hooks make): n != the sum of the members' sizes returns 11; every member's Adam
 * counter advances by one. While a table is a member its own calls run on the group's stream,
 * ordered with the group's; destroy the group before its tables. */
typedef struct krk_dense_group krk_dense_group;
int32_t krk_dense_group_create(krk_dense** tables, int32_t n, krk_dense_group** out);
int32_t krk_dense_group_destroy(krk_dense_group* g);
int32_t krk_dense_group_sync(krk_dense_group* g);
int32_t krk_dense_group_size(krk_dense_group* g, int64_t* total);
int32_t krk_dense_group_pull(krk_dense_group* g, float* out, uint32_t flags);
int32_t krk_dense_group_push(krk_dense_group* g, const krk_optim* o, const float* grads, int64_t n, float lr,
                             uint32_t flags);
/* Checkpoint::SaveDenseTable / LoadDenseTable (checkpoint/checkpoint.cc:444-463, 535-557): a
 * *.dense file holds the table's type, id, name and Value. shape/rank give the tensor shape to
 * record (rank 0 = one dimension of n elements). Loading creates the table; *rank holds the
 * capacity of `shape` on entry and the file's rank on return; name receives at most
 * name_cap - 1 characters. table_id, name, shape and rank may be NULL. */
int32_t krk_dense_save_file(krk_dense* t, const char* path, uint64_t table_id, const char* name,
                            const int64_t* shape, int32_t rank);
int32_t krk_dense_load_file(const char* path, krk_dense** out, uint64_t* table_id, char* name,
                            size_t name_cap, int64_t* shape, int32_t* rank);

/* ---- threshold ("DCT") gradient codec -------------------------------------- */
typedef struct krk_dct krk_dct;
/* DCTEmitter::DenseBag (worker/dct_emitter.cc:12-14): zero residual, tau 0, step 0. */
int32_t krk_dct_create(int64_t n, krk_dct** out);
int32_t krk_dct_destroy(krk_dct* s);
/* DenseBag::MaybeToCoo (worker/dct_emitter.cc:16-43). idx/val hold `capacity`
 * entries; *nnz receives the count, or -1 when n < 256 (the gradient is to be
 * sent dense and no state changes). tau is the true k-th largest |grad + e|;
 * the reference's chunked TopK can skip the last n mod t_num elements
 * (t/math.cc:573-586). Returns KRK_E_CAPACITY (state unchanged) when
 * capacity < nnz. */
int32_t krk_dct_compress(krk_dct* s, const float* grad, uint64_t life_span, float eta,
                         int64_t* idx, float* val, int64_t capacity, int64_t* nnz,
                         uint32_t flags);
int32_t krk_dct_tau(krk_dct* s, float* tau);
int32_t krk_dct_step(krk_dct* s, uint64_t* step);
int32_t krk_dct_residual(krk_dct* s, float* out, uint32_t flags);
/* CooTensorImpl::ToDense for a 1-D shape (t/math.cc:1006-1046): dense[n] is
 * zeroed, then dense[idx[j]] += val[j]; entries whose index lies outside [0, n) are skipped.
 * From 2^22 elements on, strictly ascending indices (what ToCoo produces) are written in one
 * pass over the output; such a call waits for its launches even with KRK_ASYNC, because the
 * work space of this object-less entry point is shared between callers. */
int32_t krk_coo_to_dense(const int64_t* idx, const float* val, int64_t nnz, float* dense,
                         int64_t n, uint32_t flags);

/* ---- blockwise DCT-II (no reference counterpart) --------------------------- */
/* The reference's "DCT" emitter is the threshold codec above and contains no cosine transform
 * (worker/dct_emitter.cc:16-43); these two calls exist because this build's target names a
 * blockwise DCT. x holds n floats, n a multiple of the block length 256. forward writes, for
 * each block, the first `keep` coefficients of its orthonormal DCT-II (scipy.fft.dct(type=2,
 * norm="ortho")) to coeff[n / 256, keep]; inverse rebuilds n floats from them (DCT-III with
 * the missing coefficients taken as zero). keep is 64, 128, 192 or 256; 256 round-trips
 * exactly up to fp32 rounding, 64 is the emitter's default retention 1 - eta = 0.25. */
int32_t krk_dct2_forward(const float* x, float* coeff, int64_t n, int32_t keep, uint32_t flags);
int32_t krk_dct2_inverse(const float* coeff, float* x, int64_t n, int32_t keep, uint32_t flags);

/* ---- timing (HIP events on an object's own stream) ------------------------ */
typedef struct krk_event krk_event;
int32_t krk_event_create(krk_event** e);
int32_t krk_event_destroy(krk_event* e);
/* object = a krk_sparse*, krk_group*, krk_dense* or krk_dct*: the event is recorded on that
 * object's stream, behind the work already enqueued there. NULL = the null stream, where the
 * calls that own no object (krk_dedup, krk_dct2_*, krk_coo_to_dense, krk_stream_copy) run. */
int32_t krk_event_record(krk_event* e, void* object);
/* Work enqueued on object's stream after this call starts only once e (recorded before, on any
 * stream) has happened: how a span measured on one object's stream is made to include work that
 * ran on another's, without the host waiting for either. */
int32_t krk_event_wait(krk_event* e, void* object);
int32_t krk_event_elapsed_ms(krk_event* start, krk_event* stop, float* ms);

#ifdef __cplusplus
}
#endif
#endif /* KRAKEN_HIP_H_ */
