/*
 * mrb.h — C ABI of the MI355X (gfx950) replay-buffer library, libmrb.so.
 *
 * The library replaces the MindSpore primitives that the reference's replay
 * buffer classes call into (the classes themselves hold no arithmetic):
 *   - uniform FIFO buffer: P.BufferAppend / P.BufferGetItem / P.BufferSample
 *     (mindspore_rl/core/uniform_replay_buffer.py:82-89, used at :114,:128,:139)
 *   - prioritized buffer:  PriorityReplayBufferCreate/Push/Sample/Update/Destroy
 *     (mindspore_rl/core/priority_replay_buffer.py:21-27, used at :62-76,:90,:106,:120)
 *
 * Conventions (the in-repo precedent for a C operator ABI is
 * mindspore_rl/utils/mcts/cpu/cpu_mcts_ops.cc:25,51-97: plain pointers,
 * a device stream argument, int status, int64 handles from a registry,
 * mindspore_rl/utils/mcts/mcts_factory.h:32,39-82):
 *   - every function returns 0 on success and a non-zero MRB_E* code on error;
 *     mrb_last_error() returns a thread-local message for the last failure.
 *     Nothing throws or aborts across this boundary.
 *   - a buffer is an opaque int64 handle (> 0) owned by a process-wide
 *     registry; the library owns row storage, trees and scratch in HBM.
 *   - all row data pointers (src_fields, dst_fields, indices, priorities,
 *     uniforms, outputs) are DEVICE pointers; the caller owns them and keeps
 *     them alive until the work enqueued on `stream` has completed.
 *   - `stream` is a hipStream_t (NULL = the null stream). All device work is
 *     enqueued on it in program order. Only *_create, *_destroy, mrb_per_state
 *     (when the running max is asked for), *_check and mrb_per_export_tree wait
 *     for the device (and, around the option "device_counters", what mrb_set_option
 *     says there); only *_create allocates device memory, with one exception:
 *     an mrb_per_update of more entries than the buffer has rows and than any
 *     earlier call had enlarges its scratch (hipMalloc; nothing is freed before
 *     *_destroy). Calls that change one handle must be serialised by the caller
 *     (the reference orders them with side_effect_io,
 *     priority_replay_buffer.py:67-76); sample / gather calls on one handle may
 *     run at the same time on different streams as long as no call that changes
 *     the handle is in flight; different handles are independent.
 *   - calls that neither wait nor allocate may be recorded into a HIP graph. A replay repeats the call
 *     as it was recorded: the ring position, the row count and the generator's call counter are host-side
 *     state that becomes kernel arguments, so a replayed push writes the slots it wrote when recorded and
 *     a replayed sample without `uniforms` draws the numbers it drew then. mrb_per_gather and an
 *     mrb_per_update of at most 1024 entries replay correctly against whatever the buffer holds at replay
 *     time; so does mrb_per_sample with `uniforms` while the number of stored rows is what it was when
 *     recorded (a full buffer). With the option "device_counters" (mrb_set_option) the counters live on the
 *     device and a recorded push / sample / update loop replays as the same calls made again would run.
 *   - storage is structure-of-arrays: field i is one [capacity, field_bytes[i]]
 *     byte matrix (reference layout: uniform_replay_buffer.py:26-47).
 */
#ifndef MRB_H_
#define MRB_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MRB_OK 0
#define MRB_EINVAL 1   /* bad argument (size, count, NULL pointer, alignment) */
#define MRB_EHANDLE 2  /* unknown or destroyed handle (cf. kErrorCode = 2, cpu_mcts_ops.cc:25) */
#define MRB_EHIP 3     /* a HIP runtime call failed */
#define MRB_ESTATE 4   /* operation not valid in the buffer's state (e.g. sample from empty) */
#define MRB_EDEVICE 5  /* a kernel recorded a data error (see mrb_per_check) */

#define MRB_MAX_FIELDS 16

/* Bits of the device-side data-error word reported by mrb_per_check. */
#define MRB_DERR_INDEX 1u     /* update_priorities: index outside [0, capacity) — entry skipped */
#define MRB_DERR_PRIORITY 2u  /* update_priorities/push: negative or non-finite priority — entry skipped */
#define MRB_DERR_TOTAL 4u     /* sample: tree total not finite or <= 0 */
#define MRB_DERR_UNFILLED 8u  /* sample: descent ended on a slot >= size */

/* ---- library ---------------------------------------------------------- */

/* Message of the calling thread's last failed call ("" if none). */
const char *mrb_last_error(void);
/* 1 = HIP/gfx950. (There is no CPU backend in this library.) */
int mrb_backend(void);
/* ABI version of this header: the library returns the MRB_ABI_VERSION it was built with; a binding
 * compares the two before it makes any other call. History: 1 = mrb_set_option(name, value);
 * 2 = mrb_set_option(handle, name, value), mrb_per_sample_many / _next / _update_noalloc added;
 * 3 = mrb_per_update_push, mrb_field_layout and mrb_bench_launch added, library-wide options (handle 0), updates
 * of more than 1024 entries refuse stream capture; 4 = mrb_per_update_push_sample added. */
#define MRB_ABI_VERSION 4
int mrb_version(void);
/* Tuning knobs of ONE buffer (any kind of handle); they change how its kernels are launched, never a
 * result. Unknown names return MRB_EINVAL. Set them while no call on the handle is in progress.
 *   "row_split"    least number of workgroups per row in the wide-row kernel (0 = auto, max 64)
 *   "row_wave"     prioritized buffers: the wave-per-row sample kernel (rows of at most 4 KB in 16-byte fields and 256
 *                  narrow bytes) is taken 0 = for launches of at least 2048 rows, 1 = whenever the rows fit it, 2 = never
 *   "sample_path"  prioritized buffers: 0 = choose by row size, 1 = wide-row kernel, 2 = LDS-top kernel
 *   "lds_levels"   prioritized buffers: tree levels staged in LDS by the LDS-top kernel (0 = auto, max 12)
 *   "device_counters" prioritized and uniform buffers: 1 = the ring position, the number of stored rows and the generator's
 *                  call counter are kept in device memory, read there by the kernels and advanced there - by
 *                  the push's own last launch, and by a one-thread kernel after a generator-driven sample - for
 *                  callers that record push / sample / update into a HIP graph: every replay then continues
 *                  where the last one stopped (pushes land in the next slots, draws differ, weights use the
 *                  current row count). While it is on: a push takes at most `capacity` rows, an update at most
 *                  1024 entries, and mrb_per_state and
 *                  the checkpoint calls wait for the device to read the counters back. Switching it (either
 *                  way) waits for the device. 0 (default) = host-side counters, passed as kernel arguments.
 *                  Uniform buffers: count, head and the generator's call counter; an append takes at most
 *                  `capacity` rows, a sample at most 65,536 (its slots are drawn into a device array that
 *                  overlapping sample / get_item calls on one handle would share), mrb_urb_append_from is
 *                  refused, and mrb_urb_state, mrb_urb_reset, mrb_urb_seed and the checkpoint calls wait.
 *   "fused_rebuild" prioritized buffers: 1 (default) = an update of <= 16 entries or a push under <= 16 leaf tiles
 *                  rebuilds the tree in one launch where the tree has one round of levels below its top;
 *                  0 = one launch per round */
/* Library-wide default, set with handle 0 and taken by buffers created afterwards:
 *   "packed_rows"  N > 0: a buffer whose packed row - every field at the next multiple of its own copy granule
 *                  (the largest power of two <= 16 that divides its size), the row padded to the widest granule -
 *                  takes at most N bytes (N <= 4096) keeps its rows packed in ONE [capacity, packed row] array
 *                  instead of one [capacity, field_bytes[i]] array per field (the reference's layout,
 *                  uniform_replay_buffer.py:26-47). A sampled row's fields then share cache lines instead of
 *                  costing a 128-byte line each; results never differ. 0 (default): one array per field.
 *                  mrb_field_layout tells where a field lies either way. */
int mrb_set_option(int64_t h, const char *name, int64_t value);
/* Where field `field` of buffer `h` (any kind) lies in device memory: row r of the field starts at
 * *dev_ptr + r * *row_stride (row_stride = field_bytes[field] unless the rows are packed). Backs the `.buffer`
 * attribute, read directly by callers (mindspore_rl/core/msrl.py:550). Either output may be NULL. */
int mrb_field_layout(int64_t h, int field, void **dev_ptr, int64_t *row_stride);

/* ---- uniform FIFO ring buffer ----------------------------------------- */

/* Replaces UniformReplayBuffer.__init__ storage + count/head
 * (uniform_replay_buffer.py:75-80). Storage is zero-filled. */
int mrb_urb_create(int64_t capacity, int nfields, const int64_t *field_bytes, int64_t *out_handle);
/* Replaces P.BufferAppend (uniform_replay_buffer.py:82,114): FIFO append of
 * nrows rows; src_fields[i] is a contiguous [nrows, field_bytes[i]] matrix.
 * nrows > capacity keeps the last `capacity` rows. */
int mrb_urb_append(int64_t h, const void *const *src_fields, int64_t nrows, void *stream);
/* Buffer-to-buffer append in one launch: the n rows of `src` at logical positions first_logical ..
 * first_logical + n - 1 (0 = oldest, negative counts back from the newest) are appended to `h` with
 * mrb_urb_append's semantics. Replaces the get_item + insert loop of NStepBuffer.get_data
 * (mindspore_rl/utils/n_step_buffer.py:85-92). Both buffers need the same fields. */
int mrb_urb_append_from(int64_t h, int64_t src, int64_t first_logical, int64_t n, void *stream);
/* Replaces P.BufferGetItem (uniform_replay_buffer.py:83,128): row at LOGICAL
 * position (0 = oldest, negative counts back from the newest) copied to
 * dst_fields[i] ([field_bytes[i]] each). */
int mrb_urb_get_item(int64_t h, int64_t logical_index, void *const *dst_fields, void *stream);
/* Gather half of P.BufferSample (uniform_replay_buffer.py:87-89,139):
 * dst_fields[i][k] = storage_i[indices[k]] for k < n, indices being physical
 * slot numbers in [0, count). Out-of-range indices are clamped into range and
 * reported by mrb_urb_check. */
int mrb_urb_gather(int64_t h, const int64_t *indices, int64_t n, void *const *dst_fields, void *stream);
/* Whole P.BufferSample: draws n slots uniformly in [0, count) with replacement
 * from the buffer's counter-based generator (seeded at create-time by
 * mrb_urb_seed; each call advances the counter, so successive calls differ),
 * optionally writes them to out_indices (may be NULL), and gathers. */
int mrb_urb_sample(int64_t h, int64_t n, int64_t *out_indices, void *const *dst_fields, void *stream);
int mrb_urb_seed(int64_t h, uint64_t seed);
/* count / head as the reference's int32 Parameters (uniform_replay_buffer.py:78-79). */
int mrb_urb_state(int64_t h, int32_t *count, int32_t *head);
/* Replaces UniformReplayBuffer.reset (uniform_replay_buffer.py:141-150): count = 0, head untouched. */
int mrb_urb_reset(int64_t h);
/* Synchronises `stream` and returns the device error word (MRB_DERR_INDEX) since the last check. */
int mrb_urb_check(int64_t h, uint32_t *flags, void *stream);
/* Device pointer of field storage [capacity, field_bytes[field]] (backs the `.buffer` attribute,
 * read directly by callers: mindspore_rl/core/msrl.py:550). */
int mrb_urb_field_ptr(int64_t h, int field, void **dev_ptr);
int mrb_urb_destroy(int64_t h);

/* ---- prioritized replay buffer ---------------------------------------- */

/* Replaces PriorityReplayBufferCreate (priority_replay_buffer.py:62-66).
 * Trees have next_pow2(capacity) leaves; max priority starts at 1.0. */
int mrb_per_create(int64_t capacity, float alpha, int nfields, const int64_t *field_bytes,
                   uint64_t seed, int64_t *out_handle);
/* Replaces PriorityReplayBufferPush (priority_replay_buffer.py:67-69,90), batched:
 * equals nrows sequential pushes. Row j goes to slot (pushes + j) mod capacity.
 * opt_priorities == NULL: each new leaf takes the running max priority (not
 * raised to alpha). Otherwise (device f32[nrows]) the push is followed by
 * update_priorities(new slots, opt_priorities). */
int mrb_per_push(int64_t h, const void *const *src_fields, int64_t nrows, const float *opt_priorities,
                 void *stream);
/* Replaces PriorityReplayBufferSample (priority_replay_buffer.py:70,106).
 * Stratified proportional sampling of `batch` rows: seg = total / batch,
 * mass_k = (k + u_k) * seg, sum-tree descent (go left when mass <= left sum),
 * weight_k = (p_k / total * size)^-beta / (p_min / total * size)^-beta,
 * then the row gather. `uniforms` is device f32[batch] in [0,1) supplied by
 * the caller, or NULL to use the buffer's counter-based generator.
 * Outputs: out_indices int64[batch], out_weights f32[batch],
 * out_fields[i] = [batch, field_bytes[i]]. */
int mrb_per_sample(int64_t h, int64_t batch, float beta, const float *uniforms, int64_t *out_indices,
                   float *out_weights, void *const *out_fields, void *stream);
/* `nbatch` stratified batches in one call: exactly what nbatch successive mrb_per_sample calls with the
 * same beta would return on an unchanged buffer (batch i uses uniforms[i * batch .. (i + 1) * batch), or
 * the generator's next call counter), written batch after batch into outputs of nbatch * batch rows.
 * No counterpart among the reference's primitives: it is for learners that draw several batches per
 * update of the priorities (prefetching); one launch then amortises the launch and the tree descent. */
int mrb_per_sample_many(int64_t h, int64_t nbatch, int64_t batch, float beta, const float *uniforms,
                        int64_t *out_indices, float *out_weights, void *const *out_fields, void *stream);
/* mrb_per_sample and, in the same launch, field `row_field` of the row whose slot number each sampled row holds
 * in its field `slot_field` (8 bytes: one int64 per row), written to out_next_rows ([batch, field_bytes[row_field]],
 * 16-byte aligned): what mrb_per_sample followed by mrb_per_gather at out_fields[slot_field] would leave in that
 * field's matrix. No counterpart among the reference's primitives: it serves transitions that keep the next
 * observation as a slot number (frame-shared storage) - a learner needs both observations, and one launch pays
 * the launch and the tree descent for both. row_field must be a field whose rows are multiples of 16 bytes.
 * Slot numbers outside [0, size) are clamped and reported by mrb_per_check (MRB_DERR_INDEX). */
int mrb_per_sample_next(int64_t h, int64_t batch, float beta, const float *uniforms, int slot_field, int row_field,
                        int64_t *out_indices, float *out_weights, void *const *out_fields, void *out_next_rows,
                        void *stream);
/* Replaces PriorityReplayBufferUpdate (priority_replay_buffer.py:71-73,120):
 * leaf[indices[j]] = priorities[j]^alpha for j in order (last write wins on
 * duplicates), every ancestor of a touched leaf recomputed from its final
 * children; max priority = max(old, all priorities[j]^alpha). */
int mrb_per_update(int64_t h, const int64_t *indices, const float *priorities, int64_t n, void *stream);
/* mrb_per_update(h, indices, priorities, n) followed by mrb_per_push(h, src_fields, nrows, opt_push_priorities),
 * as ONE call: what a learner does after every step - the new priorities of the batch it has just used
 * (priority_replay_buffer.py:108-120), then the transitions the actors have produced meanwhile (:78-90); the
 * reference's training loop issues them back to back (mindspore_rl/algorithm/dqn/dqn_trainer.py:76-87). Same
 * result, bit for bit, as the two calls (a pushed row without a priority takes the running max AFTER the
 * update). No counterpart among the reference's primitives: it exists because each of these operations is
 * bound by kernel launches, and together they need fewer - one launch for up to 384 entries and one row on a
 * tree of at most 14 levels (or up to 64 entries on one of at most 25), two launches (instead of three) for up
 * to 1024 entries and a few rows on a tree of 13 to 21 levels; other sizes run as the two calls would. */
int mrb_per_update_push(int64_t h, const int64_t *indices, const float *priorities, int64_t n,
                        const void *const *src_fields, int64_t nrows, const float *opt_push_priorities,
                        void *stream);
/* mrb_per_update_push(h, indices, priorities, n, src_fields, nrows, opt_push_priorities) followed by
 * mrb_per_sample(h, batch, beta, uniforms, out_indices, out_weights, out_fields), as ONE call: a learner's whole
 * step on the buffer - the priorities of the batch it has just used (priority_replay_buffer.py:108-120), the
 * transition the actor has just produced (:78-90) and the batch it uses next (:92-106); the reference's loop
 * issues the three in this order from one iteration to the next (mindspore_rl/algorithm/dqn/dqn_trainer.py:76-87).
 * Same results, bit for bit, as the calls one after the other (the sample sees the update and the pushed row). No
 * counterpart among the reference's primitives: on a small buffer each of the three is a launch of a few
 * microseconds, and here they are ONE launch of one workgroup when the update has at most 384 entries, the tree 2
 * to 14 levels (capacity 3 to 16,384), one row of at most 128 copy granules (2 KB in 16-byte fields) is pushed,
 * the batch has at most 512 rows of together at most 32,768 copy granules (with the option device_counters the
 * kernel takes the ring position, the row count and the generator's call counter from the device and moves them on
 * itself: a loop of such calls can be recorded into a HIP graph); any other call runs as mrb_per_update_push and
 * mrb_per_sample would. Arguments that either of them refuses
 * are refused before anything is changed. out_indices may be the array `indices` points to (a loop that updates the
 * rows it sampled the step before): the update has read its entries when the sample writes. */
int mrb_per_update_push_sample(int64_t h, const int64_t *indices, const float *priorities, int64_t n,
                               const void *const *src_fields, int64_t nrows, const float *opt_push_priorities,
                               int64_t batch, float beta, const float *uniforms, int64_t *out_indices,
                               float *out_weights, void *const *out_fields, void *stream);
/* mrb_per_update for callers that cannot allocate: code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc. It has no counterpart in the reference. Same arguments, same result
 * bit for bit; the scratch that mrb_per_update keeps per buffer (p^alpha of the call's entries) lives
 * here in a static device array of the library, 1 MiB per GPU, so n is limited to 262,144 entries
 * (larger n: MRB_EINVAL). The call allocates and frees nothing. All buffers on one GPU share that
 * array: calls of this function that may run at the same time on one GPU (different streams) race;
 * calls ordered on one stream do not. The buffer must live on the current device. */
int mrb_per_update_noalloc(int64_t h, const int64_t *indices, const float *priorities, int64_t n, void *stream);
/* Rows at the given physical slots (device int64[n], each in [0, size)), gathered like mrb_urb_gather:
 * dst_fields[i][k] = storage_i[indices[k]]. No counterpart among the reference's primitives; it serves
 * transitions that store a slot number instead of a copy of the next observation (a frame-shared
 * next_obs index): the caller samples, then gathers field rows at the sampled next_idx values.
 * Out-of-range slots are clamped and reported by mrb_per_check (MRB_DERR_INDEX). */
int mrb_per_gather(int64_t h, const int64_t *indices, int64_t n, void *const *dst_fields, void *stream);
/* Parity hook: copies both trees in canonical heap order (root at 1, leaf i at
 * leaves + i, element 0 unused) to HOST arrays of 2 * leaves floats each.
 * Either pointer may be NULL. Synchronises `stream`. */
int mrb_per_export_tree(int64_t h, float *sum_heap, float *min_heap, int64_t *leaves, void *stream);
/* Synchronises `stream`; size, next slot (pushes mod capacity) and running max priority. */
int mrb_per_state(int64_t h, int64_t *size, int64_t *head, float *max_priority, void *stream);
/* Synchronises `stream` and returns (then clears) the device error word. */
int mrb_per_check(int64_t h, uint32_t *flags, void *stream);
int mrb_per_field_ptr(int64_t h, int field, void **dev_ptr);
/* Replaces PriorityReplayBufferDestroy (priority_replay_buffer.py:74-76,138). */
int mrb_per_destroy(int64_t h);

/* ---- reservoir replay buffer --------------------------------------------- */

/* Replaces ReservoirReplayBufferCreate
 * (mindspore_rl/core/reservoir_replay_buffer.py:61-63). */
int mrb_res_create(int64_t capacity, int nfields, const int64_t *field_bytes, uint64_t seed, int64_t *out_handle);
/* Replaces ReservoirReplayBufferPush (reservoir_replay_buffer.py:64,68-79), batched: equals nrows
 * sequential pushes of Algorithm R. Row number t (counted from 0 over the buffer's life) goes to slot
 * t while t < capacity; afterwards it draws r uniformly in [0, t] from the buffer's counter-based
 * generator and replaces slot r if r < capacity (else it is dropped). Rows of one call that pick the
 * same slot: the later row wins. */
int mrb_res_push(int64_t h, const void *const *src_fields, int64_t nrows, void *stream);
/* Replaces ReservoirReplayBufferSample (reservoir_replay_buffer.py:65,81-89): n slots drawn uniformly
 * in [0, size) with replacement (n may exceed size), optionally written to out_indices, and gathered. */
int mrb_res_sample(int64_t h, int64_t n, int64_t *out_indices, void *const *dst_fields, void *stream);
/* Rows held and rows ever pushed. */
int mrb_res_state(int64_t h, int64_t *size, int64_t *total);
int mrb_res_field_ptr(int64_t h, int field, void **dev_ptr);
/* Replaces ReservoirReplayBufferDestroy (reservoir_replay_buffer.py:66,91-100). */
int mrb_res_destroy(int64_t h);

/* ---- checkpoint hooks ----------------------------------------------------- */

/* Host-side bookkeeping of a buffer as int64[4], for saving a buffer and loading it into a fresh one
 * of the same construction (the reference never persists its buffers; the row data itself is reached
 * through the *_field_ptr views):
 *   uniform   {count, head, seed, calls}      prioritized {size, pushes, seed, calls}
 *   reservoir {size, total, seed, calls}
 * set_counters validates the values against the capacity. */
int mrb_urb_get_counters(int64_t h, int64_t *out4);
int mrb_urb_set_counters(int64_t h, const int64_t *in4);
int mrb_per_get_counters(int64_t h, int64_t *out4);
int mrb_per_set_counters(int64_t h, const int64_t *in4);
int mrb_res_get_counters(int64_t h, int64_t *out4);
int mrb_res_set_counters(int64_t h, const int64_t *in4);
/* Sets the leaves of slots [0, n) of both trees to `leaves` (device f32[n], values as stored, i.e.
 * already raised to alpha), every other leaf to empty (sum 0, min FLT_MAX), rebuilds all internal
 * nodes and sets the running max priority. */
int mrb_per_load_leaves(int64_t h, const float *leaves, int64_t n, float max_priority, void *stream);

/* ---- measurement aids ---------------------------------------------------- */

/* What a machine charges for the steady-state calls above before any of their work: no counterpart in
 * the reference, no part of any buffer operation. kind 0: one launch of a kernel that does nothing
 * (calls back to back on one stream give the cost of a launch); kind 1: hipMemcpyDtoDAsync of `bytes`
 * bytes from src to dst, the runtime's own contiguous device-to-device copy (a gather of the same bytes
 * is priced against it). Neither waits nor allocates. */
int mrb_bench_launch(int kind, void *dst, const void *src, int64_t bytes, void *stream);

/* ---- discounted return --------------------------------------------------- */

/* Replaces the fused DiscountedReturn primitive and the loop it stands for
 * (mindspore_rl/utils/discounted_return.py:71,84-92): backwards over time,
 *   last = reward[t] + (1 - done[t]) * gamma * last;  out[t] = last.
 * reward and out are [timesteps, batch, inner] float32, done is [timesteps, batch] (one byte per
 * flag), last_value is [batch, inner] float32; all device pointers. */
int mrb_discounted_return(const float *reward, const uint8_t *done, const float *last_value, float *out,
                          int64_t timesteps, int64_t batch, int64_t inner, float gamma, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* MRB_H_ */
