/*
 * tensornet_amd.h -- C ABI of the MI355X (gfx950) implementation of TensorNet's
 * sparse parameter-server hot path: the per-batch pull / push a single worker's
 * SparseTable serves, and the DenseTable flat-array optimizer update.
 *
 * Every entry point mirrors one interface of the reference (cited as
 * path:line relative to the reference tree) and follows these conventions:
 *   - returns an int status (TN_OK == 0); never aborts, never throws.
 *     tn_last_error() gives the message of the calling thread's last failure.
 *     Conditions the reference turns into a fatal CHECK come back as codes.
 *   - "device" pointers are plain HIP device addresses owned by the caller;
 *     "host" pointers are ordinary host memory.  The library never frees or
 *     keeps caller memory, and never copies table rows to the host.
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream).
 *     All work of a call is enqueued on that stream.  Calls on one table are
 *     serialised by a per-table host mutex; use one stream per table.
 *   - signs are uint64 carried in int64 tensors, exactly as in
 *     core/kernels/sparse_table_ops.cc:119,124.
 */
#ifndef TENSORNET_AMD_H_
#define TENSORNET_AMD_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ----------------------------------------------------------------- status */
enum {
    TN_OK = 0,
    TN_ERR_INVALID_ARGUMENT = 1, /* errors::InvalidArgument in the ops        */
    TN_ERR_BAD_HANDLE = 2,       /* CHECK core/ps/table/sparse_table.cc:147   */
    TN_ERR_DIM_MISMATCH = 3,     /* CHECK_EQ core/kernels/sparse_table_ops.cc:204,340 */
    TN_ERR_VAR_CAPACITY = 4,     /* CHECK_LT core/kernels/sparse_table_ops.cc:136 */
    TN_ERR_UNKNOWN_KEY = 5,      /* CHECK core/ps/optimizer/optimizer_kernel.h:315 */
    TN_ERR_TABLE_FULL = 6,       /* HBM table has no free slot left           */
    TN_ERR_HIP = 7,              /* a HIP runtime call failed                 */
    TN_ERR_ALREADY_INIT = 8,     /* CHECK core/ps/table/dense_table.cc:39     */
    TN_ERR_NOT_INIT = 9,
    TN_ERR_OUT_OF_MEMORY = 10,
    TN_ERR_UNSUPPORTED = 11
};

/* Message of the last failing call made by the calling thread ("" if none). */
const char* tn_last_error(void);

/* Library version string. */
const char* tn_version(void);

/* ------------------------------------------------------------- optimizers */
/*
 * Hyper-parameter blocks.  Field names, types (all float in the reference's
 * structs, doubles coming from Python are narrowed) and defaults follow
 * core/ps/optimizer/optimizer.h:36-144 with the Python-side defaults of
 * core/main/py_wrapper.cc:94-104 (AdaGrad), :121-127 (Adam), :149-156 (Ftrl).
 * tn_*_params_default() fills in those defaults.
 */
typedef struct tn_adagrad_params {
    float learning_rate;     /* 0.01 */
    float show_decay_rate;   /* 0.98 */
    float show_threshold;    /* 0.0  */
    float initial_g2sum;     /* 0    */
    float initial_scale;     /* 1    */
    float epsilon;           /* 1e-8 */
    float grad_decay_rate;   /* 1.0  */
    float mom_decay_rate;    /* 1.0  */
    int32_t no_show_days;    /* 1000 */
    int32_t elimination_logic; /* 0 or 1 */
} tn_adagrad_params;

typedef struct tn_adam_params {
    float learning_rate;   /* 0.01 */
    float show_decay_rate; /* 0.98 */
    float beta1;           /* 0.9  */
    float beta2;           /* 0.999 */
    float epsilon;         /* 1e-8 */
    float initial_scale;   /* 1.0  */
} tn_adam_params;

typedef struct tn_ftrl_params {
    float learning_rate;   /* 0.01 */
    float show_decay_rate; /* 0.98 */
    float show_threshold;  /* 0.0  */
    float beta;            /* 1    */
    float lambda1;         /* 0.1  */
    float lambda2;         /* 1    */
    float initial_scale;   /* 1.0  */
} tn_ftrl_params;

void tn_adagrad_params_default(tn_adagrad_params* p);
void tn_adam_params_default(tn_adam_params* p);
void tn_ftrl_params_default(tn_ftrl_params* p);

/* Optimizer objects are immortal and may be shared by several tables
 * (core/main/py_wrapper.cc:112).  Handles are small ints starting at 0. */
typedef int32_t tn_opt_t;

/* core/main/py_wrapper.cc:82-116 (AdaGrad factory). elimination_logic must be 0 or 1. */
int tn_opt_create_adagrad(const tn_adagrad_params* p, tn_opt_t* out);
/* core/main/py_wrapper.cc:117-133 (Adam factory). */
int tn_opt_create_adam(const tn_adam_params* p, tn_opt_t* out);
/* core/main/py_wrapper.cc:146-162 (Ftrl factory). */
int tn_opt_create_ftrl(const tn_ftrl_params* p, tn_opt_t* out);
/* OptimizerBase::SetSparseZeroInit, core/ps/optimizer/optimizer.h:49
 * (py: set_sparse_init_mode(opt, is_training) == set_sparse_zero_init(opt, !is_training)). */
int tn_opt_set_sparse_zero_init(tn_opt_t opt, int zero_init);
/* OptimizerBase::SetSchedule(float), core/ps/optimizer/optimizer.h:61. */
int tn_opt_set_learning_rate(tn_opt_t opt, float lr);
/* py get_opt_learning_rate, core/main/py_wrapper.cc:134-145 (constant schedule only). */
int tn_opt_get_learning_rate(tn_opt_t opt, float* lr);

/* ------------------------------------------------------------ sparse table */
/*
 * Record of one distinct sign of a push, byte-identical to
 * SparsePushSignInfo (core/ps_interface/ps_raw_interface.h:22-35): 16 bytes.
 */
typedef struct tn_sign_info {
    uint64_t sign;
    int32_t batch_show;
    int32_t batch_click;
} tn_sign_info;

/*
 * CreateSparseTable (core/ps/table/sparse_table.cc:169-186) as called from
 * create_sparse_table (core/main/py_wrapper.cc:169-181): a non-empty
 * embedding_group that already exists returns the existing table's handle.
 * use_cvm follows SetUseCvm (optimizer.h:51): rows of an AdaGrad table then
 * carry two extra floats (show, log(click+1)-log(show+1)) after the weights
 * and pull/push use dim = dimension + 2.
 * The table lives in HBM as an open-addressing hash table on the current HIP
 * device.  It is allocated on first use with room for
 * tn_sparse_table_reserve()'s key count (default 8 x 15485863 slots, the
 * reference's own no-rehash bucket count, optimizer_kernel.h:257-263) and
 * grows by re-insertion when its load factor would pass 0.75
 * (optimizer_kernel.h:266).
 */
int tn_sparse_table_create(tn_opt_t opt, const char* name, int dimension, int use_cvm, int shard_num,
                           int self_shard_id, const char* embedding_group, uint32_t* handle);

/* Size the HBM table for at least max_keys resident keys at load factor <= 0.75. */
int tn_sparse_table_reserve(uint32_t handle, uint64_t max_keys);

/*
 * Drops every row of the table and gives its device memory back (the table itself, its handle and its
 * settings stay; the next call allocates an empty table again).  The reference's tables live in host hash maps
 * until the process ends (SparseTableRegistry, core/ps/table/sparse_table.cc:150-186) and have no such call;
 * a table that fills most of a GPU's memory needs one, for hosts that rebuild their tables (and for tests).
 * Waits for the table's pending work first.
 */
int tn_sparse_table_clear(uint32_t handle);

/* Seed of the on-device row initialiser (the reference seeds from the wall
 * clock, core/utility/random.h:30-42; here new rows are a pure function of
 * (seed, sign)). */
int tn_sparse_table_set_seed(uint32_t handle, uint64_t seed);

/* SparseOptimizerKernelBase::KeyCount, core/ps/optimizer/optimizer_kernel.h:540-547. */
int tn_sparse_table_key_count(uint32_t handle, uint64_t* count);

/* Number of HBM hash slots currently allocated (0 before first use). */
int tn_sparse_table_capacity(uint32_t handle, uint64_t* slots);

/* Floats per row: weights (dimension, +2 with cvm) and optimizer state.
 * State layout (float words; integers stored bitwise):
 *   AdaGrad: g2sum, show, click, no_show_days(int32)        (ada_grad_kernel.h:76-83)
 *   Adam:    m[dim], v[dim], show, delta_show(int32)        (adam_kernel.h:72-86, data_struct.h:54-58)
 *   Ftrl:    z[dim], n[dim], show, delta_show(int32)        (ftrl_kernel.h:73-88) */
int tn_sparse_table_row_layout(uint32_t handle, int* weight_floats, int* state_floats);

/*
 * SparseTable::Pull (core/ps/table/sparse_table.cc:52-66): for each of the n
 * device signs, in request order, look the row up -- inserting and
 * initialising it if absent (optimizer_kernel.h:299-308) -- and write its
 * `dim` floats to out[i*dim .. i*dim+dim) (device).  dim must equal the
 * table's weight_floats.
 */
int tn_sparse_table_pull(uint32_t handle, const uint64_t* signs, int64_t n, int dim, float* out, void* stream);

/*
 * The same pull for callers that cannot allocate device memory (tight serving loops, harnesses that forbid
 * hipMalloc, code that runs between the captures of HIP graphs -- the call itself waits for its stream and
 * copies its status to the host, so it cannot be recorded into a graph).  No counterpart in the reference.
 * It calls no hipMalloc / hipFree:
 * the row numbers and the new-row list of the call live in a static device array of the library (8 MiB + 256 B,
 * held by every GPU the library runs on until the process ends), so
 *   - n is at most 1048576 signs per call (TN_ERR_UNSUPPORTED beyond that);
 *   - the table's storage must already exist (any earlier call through another entry point creates it) and
 *     must have room for n more signs without growing (TN_ERR_UNSUPPORTED / TN_ERR_TABLE_FULL otherwise:
 *     size it with tn_sparse_table_reserve first);
 *   - the current device must be the table's.
 * Calls are serialised by a lock of the library and each waits for its own work before it returns, so calls
 * from several host threads do not race on the array; results are those of tn_sparse_table_pull, bit for bit.
 */
int tn_sparse_table_pull_static(uint32_t handle, const uint64_t* signs, int64_t n, int dim, float* out, void* stream);

/*
 * SparseTable::Push (core/ps/table/sparse_table.cc:68-83): apply n records
 * (device infos[n], device grads[n*dim]) in ARRAY ORDER; a sign occurring k
 * times gets k sequential optimizer Applies.  A sign that was never pulled is
 * TN_ERR_UNKNOWN_KEY (that record is skipped, the others are applied).
 */
int tn_sparse_table_push(uint32_t handle, const tn_sign_info* infos, const float* grads, int64_t n, int dim,
                         void* stream);

/*
 * Snapshot injection / read-back: what the reference does through the mutable
 * pointer returned by SparseOptimizerKernelBase::GetWeight
 * (optimizer_kernel.h:84) and through bin Serialized/DeSerialized
 * (optimizer_kernel.h:341-351,399-408).  All pointers are device memory.
 * load_rows inserts (or overwrites) n rows; w is [n, weight_floats], state is
 * [n, state_floats] or NULL for freshly-constructed state.
 * export_rows writes the rows of n signs; found[i] = 0 and zeros for absent signs.
 */
int tn_sparse_table_load_rows(uint32_t handle, const uint64_t* signs, const float* w, const float* state,
                              int64_t n, void* stream);
int tn_sparse_table_export_rows(uint32_t handle, const uint64_t* signs, int64_t n, float* w, float* state,
                                uint8_t* found, void* stream);

/*
 * SparseTablePull op (core/ops/sparse_table_ops.cc:21-43, kernel
 * core/kernels/sparse_table_ops.cc:170-265).  N slots; slot s has
 * value_lens[s] int64 signs at device pointer values[s], a device variable
 * vars[s] of shape [var_rows[s], var_dim] row-major, and a device output
 * mapped_values[s] of value_lens[s] int64.  values/vars/mapped_values/
 * value_lens/var_rows are HOST arrays of length N.
 * Writes mapped_values[s][i] = rank of values[s][i]'s first occurrence among
 * the distinct signs of slot s (sparse_table_ops.cc:122-131) and copies the
 * pulled row of the j-th distinct sign into vars[s][j, :]; rows >= U_s are
 * left untouched.  U_s >= var_rows[s] is TN_ERR_VAR_CAPACITY.
 * The call returns when the per-slot counts and the errors of the call are
 * known on the host (the reference op blocks on a semaphore until the pulled
 * rows are there, sparse_table_ops.cc:236).  The outputs are complete in
 * stream order, as the outputs of a GPU op kernel are: on large batches the
 * copy of the pulled rows into vars may still be running on `stream` when the
 * call returns; work enqueued on `stream` afterwards sees them, a host that
 * reads them synchronises the stream (or calls tn_sparse_table_sync) first.
 */
int tn_sparse_table_pull_op(uint32_t table_handle, int N, const int64_t* const* values, const int64_t* value_lens,
                            float* const* vars, const int64_t* var_rows, int var_dim,
                            int64_t* const* mapped_values, void* stream);

/*
 * SparseTablePush op (core/ops/sparse_table_ops.cc:45-53, kernel
 * core/kernels/sparse_table_ops.cc:317-368).  grads[s] is a device matrix
 * [grad_rows[s], grad_dim] whose row j belongs to the j-th distinct sign of
 * slot s; feature_labels[s] holds value_lens[s] int64 labels.  Per distinct
 * sign batch_show = occurrences and batch_click = sum of labels
 * (sparse_table_ops.cc:283-296); records are applied slot-major, so a sign
 * present in k slots receives k sequential Applies, slot 0 first.
 * Enqueues the updates and returns without waiting for them, like the
 * reference op (sparse_table_ops.cc:363-367); errors of the enqueued work are
 * reported by the next synchronising call on the table or by
 * tn_sparse_table_sync().  One wait remains: a push that follows the pull op
 * of the same batch reuses what that pull worked out about the batch once the
 * device has confirmed that the signs are the same, and the call returns when
 * that comparison (one pass over the signs, queued ahead of the updates) has
 * reported to the host.
 */
int tn_sparse_table_push_op(uint32_t table_handle, int N, const int64_t* const* values, const int64_t* value_lens,
                            const float* const* grads, const int64_t* grad_rows, int grad_dim,
                            const int64_t* const* feature_labels, void* stream);

/*
 * The step TensorFlow runs between the two ops for every slot -- the combiner
 * of tf.nn.embedding_lookup_sparse, reached by the reference through
 * embedding_column.get_dense_tensor (tensornet/layers/embedding_features.py:278-280)
 * with the mapped ids of tensornet/feature_column/category_column.py:42-51 --
 * done on the device on both sides of the table.
 *
 * Forward: out[s] is a device matrix [batch, dim]; example_ids[s] holds, for
 * every lookup of slot s, the index of its example (SparseTensor.indices[:, 0]:
 * non-decreasing, in [0, batch)); mapped_values[s] are the ids the pull op
 * returned and vars[s] ([var_rows[s], dim]) the variable it filled.
 *   out[s][b, :] = (sum over the lookups of example b, in order, of vars[s][mapped, :]) / d(n_b)
 *   d(n) = 1 (TN_COMBINER_SUM), n (MEAN), sqrt(n) (SQRTN); examples without lookups give zeros.
 * Returns after the stream work has completed; ids outside the variable are
 * TN_ERR_VAR_CAPACITY, unsorted or out-of-range example ids TN_ERR_INVALID_ARGUMENT.
 */
enum { TN_COMBINER_SUM = 0, TN_COMBINER_MEAN = 1, TN_COMBINER_SQRTN = 2 };
int tn_sparse_table_combine_op(uint32_t table_handle, int N, const int64_t* const* mapped_values,
                               const int64_t* value_lens, const int64_t* const* example_ids, const float* const* vars,
                               const int64_t* var_rows, int dim, int64_t batch, int combiner, float* const* out,
                               void* stream);

/*
 * Backward: SparseTablePush (as tn_sparse_table_push_op) fed with the gradient
 * of the combiner's output instead of per-distinct-sign rows.  pooled_grads[s]
 * is a device matrix [batch, grad_dim]; the gradient row of the j-th distinct
 * sign of slot s -- what TensorFlow hands the reference's op as grads[s][j, :],
 * core/kernels/sparse_table_ops.cc:336-352 -- is
 *   sum over the lookups of that sign, in order, of pooled_grads[s][example, :] * (1 / d(n_example))
 * computed on the device (the segmented reduction of the per-lookup gradients)
 * and applied like a push.  Enqueues and returns like tn_sparse_table_push_op.
 */
int tn_sparse_table_push_pooled_op(uint32_t table_handle, int N, const int64_t* const* values,
                                   const int64_t* value_lens, const int64_t* const* example_ids,
                                   const float* const* pooled_grads, int64_t batch, int grad_dim, int combiner,
                                   const int64_t* const* feature_labels, void* stream);

/*
 * SparseTable::ShowDecay (core/ps/table/sparse_table.h:59, sparse_table.cc:139,
 * bound to Python as tn.core.show_decay, core/main/py_wrapper.cc:259-262): every
 * resident row ages by delta_days -- AdaGrad: show and click times
 * show_decay_rate, no_show_days += delta_days (ada_grad_kernel.cc:191-195);
 * Ftrl: show times show_decay_rate (ftrl_kernel.cc:124); Adam: nothing
 * (adam_kernel.h:67).  One streaming pass over the table, enqueued on `stream`.
 */
int tn_sparse_table_show_decay(uint32_t handle, int delta_days, void* stream);

/*
 * Value::DeleteByShow (ada_grad_kernel.cc:197-204, ftrl_kernel.cc:126,
 * adam_kernel.h:69), the feature-elimination test the reference applies to every
 * row when it saves a table (optimizer_kernel.h:332,345): out[i] (device) = 1 if
 * the row of signs[i] (device) would be left out, 0 if it is kept or absent.
 * Returns after the stream work has completed.
 */
int tn_sparse_table_delete_by_show(uint32_t handle, const uint64_t* signs, int64_t n, uint8_t* out, void* stream);

/*
 * SparseTable::Save / Load (core/ps/table/sparse_table.h:55-57, sparse_table.cc:84-137; Python
 * tn.core.save_sparse_table / load_sparse_table, core/main/py_wrapper.cc:211-220) in the
 * reference's on-disk formats: eight gzip files
 * <filepath>/sparse_table/<name or handle>/rank_0/block_<i>.gz, a row in file
 * (sign >> 32 | sign << 32) % 8, mode "txt" (default of the reference) or "bin"
 * (optimizer_kernel.h:324-420,462-538; value formats ada_grad_kernel.cc:131-189,
 * adam_kernel.cc:127-167, ftrl_kernel.cc:82-122).  Rows for which DeleteByShow holds are not
 * saved.  Load derives prefix, suffix and mode from the first file name as the reference does
 * (a name without _bin / _txt suffix is read as text) and adds the rows to the table.
 * Both work on the default stream and return when done.
 */
int tn_sparse_table_save(uint32_t handle, const char* filepath, const char* mode);
int tn_sparse_table_load(uint32_t handle, const char* filepath, const char* mode);

/*
 * Building blocks of the two above (no counterpart in the reference, whose table lives in host
 * memory).  export_range: every resident row among the table slots
 * [first_slot, first_slot + n_slots), compacted into signs / w [.., weight_floats] /
 * state [.., state_floats] (device, room for n_slots rows) in no particular order;
 * skip_eliminated leaves out rows for which DeleteByShow holds; *count (host) = rows written.
 * name / optimizer: what the table was created with (optimizer kind 0 AdaGrad, 1 Adam, 2 Ftrl).
 */
int tn_sparse_table_export_range(uint32_t handle, uint64_t first_slot, uint64_t n_slots, int skip_eliminated,
                                 uint64_t* signs, float* w, float* state, uint64_t* count, void* stream);
int tn_sparse_table_name(uint32_t handle, char* name, int cap);
int tn_sparse_table_optimizer(uint32_t handle, int* kind, int* use_cvm);

/* Wait for the table's enqueued work and return (and clear) its latched error. */
int tn_sparse_table_sync(uint32_t handle);

/* U_s of the last pull_op / synchronised push_op on the table (host array of N). */
int tn_sparse_table_last_unique_counts(uint32_t handle, int N, int64_t* counts);

/* Keep pull_op from waiting on the stream (for callers that order work on the
 * stream themselves); its errors are then latched like push_op's. */
int tn_sparse_table_set_async(uint32_t handle, int async_pull);

/* Whether small batches (every slot at most 4096 lookups, at most 128 slots and 262144 lookups) take the path
 * of few launches (the default) or the one every other batch takes.  Same results either way; a switch for
 * measurements and tests, without a counterpart in the reference. */
int tn_sparse_table_set_small_batch_path(uint32_t handle, int enable);

/* How a push_op recognises the batch of the pull_op before it on large batches (the reference has no such
 * step: every push analyses its batch itself, sparse_table_ops.cc:274-297).  By default the device compares
 * fingerprints of the signs, 16 bytes per 64 lookups (one changed sign always shows; several changed signs
 * escape only if two 64-bit hash sums agree by chance).  With exact verify the pull keeps a copy of its
 * signs (8 bytes per lookup more in the table's plan buffer) and the push compares the signs themselves,
 * as the pushes of small batches always do.  Off by default; takes effect from the next pull_op. */
int tn_sparse_table_set_exact_verify(uint32_t handle, int enable);

/* The reference's push op hands its gradients to the servers and returns; the rows are updated while the
 * worker goes on (SparseTablePushKernel::ComputeAsync, sparse_table_ops.cc:346-365: requests started, done()
 * called).  With detached updates a large push_op (3 M lookups or more, on the plan of the pull before it) does
 * the same on the device: its update kernels run on the table's own streams and `stream` does not wait for
 * them, so that what the caller queues next runs beside them -- above all the analysis of the next pull's
 * batch, which orders itself behind the updates only where it first touches what they read or write (the
 * next pull's variables hold the updated rows, as ever).  The price is the one an asynchronous op pays: the
 * gradient matrices of the push must stay as they are until the table's next pull_op, sync or other waiting
 * call has returned.  Off by default (then everything a push reads is read in the order of `stream`). */
int tn_sparse_table_set_detached_updates(uint32_t handle, int enable);

/* ------------------------------------------------------------- dense table */
/* CreateDenseTable (core/ps/table/dense_table.cc:180-186); Adam or AdaGrad.  With shard_num > 1
 * the table is worker self_shard_id's share: after Init it owns the contiguous range
 * [id * ceil(total / shard_num), ...) of the concatenated parameters (DenseTable::Init,
 * dense_table.cc:46-66); the other ranges live on other workers. */
int tn_dense_table_create(tn_opt_t opt, int shard_num, int self_shard_id, uint32_t* handle);

/*
 * DenseTableInit op (core/kernels/dense_table_ops.cc:73-118): concatenates N
 * device variables (var_lens[s] floats each, host arrays of length N) into
 * the table: DenseTable::Init(total) + SetWeight (dense_table.cc:37-87).
 * A second Init with a different total is TN_ERR_ALREADY_INIT.
 */
int tn_dense_table_init(uint32_t handle, int N, const float* const* vars, const int64_t* var_lens, void* stream);

/*
 * DenseTablePushPull op (core/kernels/dense_table_ops.cc:130-252): applies
 * the concatenated gradient with this step's learning rate
 * (DenseOptimizerKernel::Apply, optimizer_kernel.h:192-204 ->
 * DenseAdamValue::Apply adam_kernel.cc:46-55 or DenseAdaGradValue::Apply
 * ada_grad_kernel.cc:42-48) and writes the new weights back into the
 * variables.  vars[s] may be NULL to skip the write-back of a variable.
 */
int tn_dense_table_push_pull(uint32_t handle, int N, float* const* vars, const float* const* grads,
                             const int64_t* lens, float learning_rate, void* stream);

/* DenseTable::TotalElements (core/ps/table/dense_table.h:44). */
int tn_dense_table_total_elements(uint32_t handle, int64_t* total);

/* DenseOptimizerKernelBase::OffsetBegin / OffsetEnd (optimizer_kernel.h:55-57): the range of
 * the table this shard holds; [0, total) with one shard, empty for a shard past the end. */
int tn_dense_table_range(uint32_t handle, int64_t* begin, int64_t* end);

/* DenseOptimizerKernelBase::GetWeight / SetWeight (optimizer_kernel.h:63-65)
 * over the shard's range; device pointers of end - begin floats. */
int tn_dense_table_get_weight(uint32_t handle, float* w, void* stream);
int tn_dense_table_set_weight(uint32_t handle, const float* w, void* stream);
/* Optimizer state read-back for tests: Adam m,v ; AdaGrad d2sum,g2sum,m (device, end - begin floats each; NULL skips). */
int tn_dense_table_get_state(uint32_t handle, float* s0, float* s1, float* s2, void* stream);

/*
 * DenseTable::Save / Load (core/ps/table/dense_table.cc:103-157; py_wrapper.cc:221-230):
 * one text file <filepath>/dense_table/<handle>/<self_shard_id> holding the total, the
 * shard count and, per block of ceil(range / 8) elements of the shard's range, the optimizer's name, the
 * block length, Adam's beta powers and one line of w and state per element, printed as
 * operator<< prints a float (6 significant digits).  Save of a table that was never
 * initialised writes nothing.  Load initialises the table to the file's total (an
 * initialised table of another size: TN_ERR_ALREADY_INIT) and refuses a file of another
 * optimizer or shard count.  Synchronous, host code.
 */
int tn_dense_table_save(uint32_t handle, const char* filepath);
int tn_dense_table_load(uint32_t handle, const char* filepath);

/* --------------------------------------------------------------- profiling */
/*
 * Measurement hooks with no counterpart in the reference (which instruments
 * nothing on this path).  While enabled, every kernel launch of the library is
 * bracketed by two HIP events on the stream it is launched on.
 * tn_profile_summary waits for the recorded events and writes one line per
 * kernel name, "name<TAB>launches<TAB>total_ms", into buf (NUL-terminated).
 * tn_profile_reset drops the records.
 */
int tn_profile_enable(int on);
int tn_profile_reset(void);
int tn_profile_summary(char* buf, size_t cap);

#ifdef __cplusplus
}
#endif
#endif /* TENSORNET_AMD_H_ */
