/* tandem_hip.h -- C ABI of libtandem_hip.so: tandem's data-parallel reduction
 * path on one AMD MI355X (gfx950).
 *
 * Plain pointers and sizes only; no torch, pybind or CUDA types. Device pointers
 * are raw HIP device addresses (torch: tensor.data_ptr()); a tdm_stream is a
 * hipStream_t (torch: torch.cuda.current_stream().cuda_stream; NULL is the
 * default stream). Every function returns 0 on success and a non-zero code on
 * failure, with the message available from tdm_last_error() on the same thread.
 * Launchers enqueue work on the given stream and return without waiting.
 *
 * The citations name what each entry point replaces in the reference
 * (Shakhtar-Sankur/tandem): the Python engine's per-piece torch calls and the
 * C++ engine's pybind surface (tandem/csrc/engine.cpp:53-123).
 */
#ifndef TANDEM_HIP_H
#define TANDEM_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif
/* The library is built with hidden visibility; what this header declares is all it exports. */
#if defined(__GNUC__) || defined(__clang__)
#pragma GCC visibility push(default)
#endif

typedef void* tdm_stream;

/* The element types the reducing kernels know. Integer sums wrap around, as ATen's add_ does; 16-bit
 * floats are widened to fp32, added and rounded to nearest even once per add (tandem/csrc/reduce.cu:27-36).
 * A NaN result of a 16-bit sum or average is the type's canonical quiet NaN (bf16 0x7fc0, f16 0x7e00): sign and
 * payload of a NaN are not preserved, as they are not across torch builds either; elements that a collective
 * only copies keep the bits they came with.
 * The reference's engine reduces any further ATen dtype by falling back to add_
 * (tandem/csrc/collectives.cpp:254-256); here every entry point that adds (tdm_k1_reduce_step, tdm_local_*,
 * tdm_k2_*, tdm_all_reduce, tdm_reduce_scatter, tdm_direct_*) refuses any other code with TDM_EINVAL
 * ("unknown dtype"): bool, the unsigned types wider than a byte, complex and the 8-bit floats are not
 * summed. Entry points that only copy (tdm_all_gather, tdm_broadcast, tdm_sendrecv, tdm_unit_gather) also
 * take TDM_BYTES (code 6, declared with them), which covers every dtype. */
enum tdm_dtype {
  TDM_F32 = 0, TDM_F64 = 1, TDM_F16 = 2, TDM_BF16 = 3, TDM_I64 = 4, TDM_I32 = 5,
  TDM_I16 = 7, TDM_I8 = 8, TDM_U8 = 9
};

enum { TDM_MAX_PAIRS = 16, TDM_MAX_WORLD = 8 };

enum tdm_status {
  TDM_OK = 0,
  TDM_EINVAL = 1,   /* bad argument: maps to ValueError / std::invalid_argument (engine.cpp:54) */
  TDM_ERUNTIME = 2, /* HIP or engine failure: RuntimeError */
  TDM_ETIMEOUT = 3  /* a peer did not answer in time: TimeoutError (engine.cpp:55) */
};

/* One (destination, source, element count) stream of a launch. */
typedef struct tdm_pair {
  void* dst;
  const void* src;
  int64_t count;
} tdm_pair;

/* ---- library ------------------------------------------------------------ */

/* Message of the last failure on the calling thread ("" if none). */
const char* tdm_last_error(void);

/* Bumped when a signature in this header changes. */
int tdm_abi_version(void);

/* Name, compute-unit count and memory of HIP device `device`. */
int tdm_device_info(int device, char* name, int name_len, int* compute_units, int64_t* total_bytes);

/* Launch geometry knob for measurements: workgroups per compute unit used by the
 * streaming kernels before their grids start to stride, 1..16384 (0 restores the built-in default, 16384: one
 * workgroup per tile up to 16 GiB per launch and stream on 256 compute units). Not needed for correctness; the
 * reference has no counterpart. */
int tdm_set_blocks_per_cu(int blocks);

/* Launch geometry knob for measurements: which tile a workgroup takes. Consecutive workgroups
 * go to the GPU's 8 XCDs in turn; with shift s each XCD takes (1 << s) consecutive tiles out of
 * every group of (8 << s), so its L2 sees runs of (tile << s) bytes per stream. `kind` names the
 * kernel family (TDM_XCD_*, -1: all), `shift` is 0..12 (0: tile = workgroup index) or -1 for the
 * built-in default of that family. Process-wide; results never depend on it. The reference has no counterpart. */
#define TDM_XCD_REDUCE 0      /* K1 ring-step reduce */
#define TDM_XCD_COPY 1        /* ring copy step, pack, unit gather */
#define TDM_XCD_FOLD 2        /* fold with the table by value (one collective) */
#define TDM_XCD_FOLD_TABLE 3  /* K2 bucket fold over a device table */
#define TDM_XCD_ADAMW 4       /* K3 */
#define TDM_XCD_STEP 5        /* K2 + K3: the one-launch ZeRO-2 step */
int tdm_set_xcd_group(int kind, int shift);
/* Launch geometry knob for measurements: bytes of LDS that the launches of kernel family `kind`
 * (TDM_XCD_*, -1: all) reserve per workgroup without using them, which caps how many workgroups
 * share a compute unit (160 KiB of LDS each); 0: no cap, -1: the built-in default of that family
 * (24 KiB for TDM_XCD_STEP and TDM_XCD_ADAMW, whose many streams do better with 3 waves per SIMD;
 * beyond the caches also 24 KiB for a by-value fold (TDM_XCD_FOLD), 16 KiB for the one-launch
 * all-gather (TDM_XCD_COPY) and 16 to 32 KiB, by world size, for the one-launch reduce-scatter
 * (TDM_XCD_REDUCE); 0 otherwise). At most 65536. Process-wide; results never depend on it. The reference has
 * no counterpart. */
int tdm_set_occupancy_pad(int kind, int bytes);
/* The tile that workgroup `index` of a launch over `total` tiles takes at group shift `shift` (the
 * kernels' own function, evaluated on the host: for tests of the mapping). -1 for arguments out of range. */
int64_t tdm_tile_of(int64_t index, int64_t total, int shift);

/* Bytes of every stream that one record of the K2 and K2+K3 device tables covers (a build constant). */
int tdm_table_tile_bytes(void);

/* Build constants of the launch geometry, for records that must name the build they were measured
 * on: bytes of every stream that one workgroup of K1 and of the copy kernel takes, lanes per
 * workgroup, bytes of every stream per table record (= tdm_table_tile_bytes()). The reference has
 * no counterpart. */
int tdm_build_geometry(int* k1_tile_bytes, int* workgroup_lanes, int* table_tile_bytes);

/* ---- K1: one ring step -------------------------------------------------- */

/* The reduce half of a ring reduce-scatter step, for up to TDM_MAX_PAIRS
 * (receiver chunk, sender chunk) pairs in ONE launch:
 *
 *     d = scale_dst ? dst[i] / world : dst[i]
 *     s = scale_src ? src[i] / world : src[i]
 *     dst[i] = d + s;      if (writeback_src) src[i] = s
 *
 * in the tensor's own precision (16-bit floats: widen to fp32, operate, round to
 * nearest even after each operation), with a true division and no multiply-add
 * contraction. world <= 1 means no division. Replaces `flat.div_(size)` +
 * `into.add_(slot)` per 4 MiB piece (tandem/comm.py:269-285,336-343) and the
 * C++ engine's take()/add_into (tandem/csrc/collectives.cpp:241-260,
 * tandem/csrc/reduce.cu:47-58,75-102). scale_src is set on the first step only,
 * when the sender's chunk is still undivided; writeback_src leaves the sender's
 * chunk holding x / world, as div_ of the whole tensor does. Integer dtypes
 * reject scaling. Pointers need only element alignment; 16-byte-aligned pairs
 * take the dwordx4 path. */
int tdm_k1_reduce_step(const tdm_pair* pairs, int npairs, int dtype, int world, int scale_dst, int scale_src,
                       int writeback_src, tdm_stream stream);

/* The copy half of a ring step (all-gather, broadcast, flatten): dst[i] = src[i],
 * or dst[i] = src[i] / world when world > 1. Replaces `into.copy_(slot)`
 * (tandem/comm.py:282-283) and cudaMemcpyAsync in take()
 * (tandem/csrc/collectives.cpp:247-250). */
int tdm_k1_copy_step(const tdm_pair* pairs, int npairs, int dtype, int world, tdm_stream stream);

/* ---- a whole group in one process: rank r is bufs[r] in this GPU's HBM ----- */

/* tandem's ring collectives over `world` equally sized, non-overlapping device
 * buffers, one per rank, with ONE launch of the K1 kernels per ring step carrying
 * every rank's (receiving chunk, neighbour's chunk) pair. In place; the results,
 * including the partial sums a bare reduce_scatter leaves in the other chunks
 * (keep_sent != 0), are bit for bit those of Group.reduce_scatter / all_gather /
 * all_reduce run as `world` processes (tandem/comm.py:301-385). sizes / nsizes
 * as for the engine's collectives (nsizes == 0: torch.tensor_split). */
int tdm_local_reduce_scatter(void* const* bufs, int world, int64_t numel, int dtype, const int64_t* sizes, int nsizes,
                             int average, int keep_sent, tdm_stream stream);
int tdm_local_all_gather(void* const* bufs, int world, int64_t numel, int dtype, const int64_t* sizes, int nsizes,
                         tdm_stream stream);

/* Which form tdm_local_reduce_scatter / tdm_local_all_gather (and tdm_local_all_reduce with
 * TDM_ALLREDUCE_RING) take: 0 the ring's W-1 steps, one launch each; 1 the whole reduce-scatter as one
 * launch (world sizes 2..8: every tile runs the ring's chain of additions for its chunk and stores each
 * partial sum where the ring would have left it; a call whose ranks' copies of a chunk disagree within
 * 16 bytes takes the steps all the same) and the whole all-gather as one launch (world sizes 2..8: every
 * chunk read once from its owner and stored into the other ranks' buffers); -1 (default) both one-launch
 * forms from world size 3 on, the steps at world size 2 and beyond 8. Memory ends bit for bit the
 * same either way, partial sums included. Process-wide; for measurements and tests. The reference has no
 * counterpart. */
int tdm_set_ring_form(int form);

enum tdm_allreduce_algorithm {
  TDM_ALLREDUCE_RING = 0, /* reduce-scatter then all-gather: 2 (world - 1) launches */
  TDM_ALLREDUCE_FOLD = 1  /* one launch: every element read from all ranks, folded in the ring's
                           * order for its chunk, written to all ranks (world <= 8); same bits */
};
int tdm_local_all_reduce(void* const* bufs, int world, int64_t numel, int dtype, int average, int algorithm,
                         tdm_stream stream);

/* ---- K2: bucket flatten + average + unflatten ---------------------------- */

/* One segment of a bucket: `count` elements that lie in ring chunk `chunk` of the
 * bucket's flat buffer, held by every rank at src[r]; the averaged value is
 * written to every non-NULL dst[r] (the rank's gradient itself, or its view in
 * the bucket). */
/* Entries of ranks beyond the world size must be NULL. When every pointer of a segment lies at the same
 * distance from a 16-byte boundary, the kernels peel the few elements before the boundary and run the
 * rest on 16-byte vectors; pointers that disagree within 16 bytes cost the element-wise path. */
typedef struct tdm_fold_seg {
  const void* src[TDM_MAX_WORLD];
  void* dst[TDM_MAX_WORLD];
  int64_t count;
  int32_t chunk;
  int32_t reserved;
} tdm_fold_seg;

/* The device table holds one record per tile (tdm_table_tile_bytes() of every stream) of every segment. Number of tiles
 * and bytes of device memory the table of these segments needs (-1: bad arguments). */
int64_t tdm_k2_table_tiles(const tdm_fold_seg* segs, int nseg, int dtype);
int64_t tdm_k2_table_bytes(const tdm_fold_seg* segs, int nseg, int dtype);

/* Writes the device image of the table into host memory `image`
 * (tdm_k2_table_bytes(...) bytes); the caller copies it to the device once. */
int tdm_k2_table_build(const tdm_fold_seg* segs, int nseg, int world, int dtype, void* image);

/* For every element of every segment, in one launch over `ntiles` tiles:
 *     y_q = average ? src[q][i] / world : src[q][i]
 *     acc = y[(chunk+1) % world];  acc = y[(chunk+k) % world] + acc,  k = 2..world
 *     dst[r][i] = acc  for every rank r with a non-NULL dst   (accumulate: dst[r][i] = dst[r][i] + acc)
 * which is bit for bit what DDP's per-parameter `view.copy_(p.grad)` followed by
 * the bucket's ring all_reduce(op="avg") leaves in every rank's gradient views
 * (tandem/ddp.py:22-33,89-109; ring order tandem/comm.py:301-311). With a dst only for
 * the chunk's owner and accumulate set, a segment is ZeRO-2's reduce_scatter of that chunk
 * followed by `grad_shard[...].add_(mine)` (tandem/zero.py:141,150-153). */
int tdm_k2_bucket_fold(const void* table_dev, int64_t ntiles, int dtype, int world, int average, int accumulate,
                       tdm_stream stream);

/* tdm_k2_bucket_fold for callers that cannot allocate device memory or copy a table to the
 * device: code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.
 * It has no counterpart in the reference. The per-tile table that tdm_k2_table_build +
 * tdm_k2_bucket_fold keep in a buffer of the caller's is written here by a small kernel
 * (the segments travel in its launch arguments, 16 per launch) into a fixed array inside the
 * library, tdm_k2_static_max_tiles() records = 16,384 tiles = 64 MiB of every rank's stream
 * per call, 2.25 MiB of device memory that every GPU the library runs on holds until the
 * process ends; then the same fold kernel runs over it, on `stream`. Same arguments
 * otherwise, same bits. Segments that need more records are refused (TDM_EINVAL) before
 * anything is launched: split the call. The call allocates nothing on the device and makes no
 * host-to-device copy. All calls on one GPU share the array, and the library orders them: calls on
 * one stream are ordered by the stream; a call on another stream than the one before it first makes
 * its stream wait (on the GPU, hipStreamWaitEvent on an event created at set-up) for that call's
 * fold; host threads take turns while they enqueue. Two such calls therefore never overlap on the
 * GPU, whatever streams they are on. The one exception is a stream under capture, where neither the
 * wait nor the event record is issued (they would become nodes of the caller's graph): replays of a
 * graph that holds such a call, and any other call on the same GPU, must be ordered by the caller. */
int64_t tdm_k2_static_max_tiles(void);
int tdm_k2_bucket_fold_static(const tdm_fold_seg* segs, int nseg, int world, int dtype, int average, int accumulate,
                              tdm_stream stream);

/* ---- K3: sharded AdamW --------------------------------------------------- */

/* The step's constants, each already rounded to fp32 from the Python-double
 * expressions of tandem/optim.py:28-37. */
typedef struct tdm_adamw_scalars {
  int32_t use_decay; /* weight_decay != 0 */
  float decay;       /* 1 - lr * weight_decay */
  float w1;          /* 1 - beta1 */
  float beta2;
  float one_m_b2;    /* 1 - beta2 */
  float bc2_sqrt;    /* (1 - beta2**t) ** 0.5 */
  float eps;
  float neg_step;    /* -(lr / (1 - beta1**t)) */
  float inv_bc2_sqrt; /* 1 / ((1 - beta2**t) ** 0.5), divided in double: TDM_ADAMW_DEVICE_ORDER only */
} tdm_adamw_scalars;

enum tdm_adamw_order {
  /* torch's CPU kernels, i.e. the reference's CPU engine:
   *   v = fma((1-beta2)*g, g, v*beta2);  p = p + (neg_step*m)/d */
  TDM_ADAMW_HOST_ORDER = 0,
  /* torch's GPU kernels: addcmul_/addcdiv_ compute a + value*(t1 op t2), contracted,
   * and tensor / scalar multiplies by the scalar's reciprocal:
   *   v = fma(1-beta2, g*g, v*beta2);  d = sqrt(v) * inv_bc2_sqrt + eps;
   *   p = fma(neg_step, m/d, p) */
  TDM_ADAMW_DEVICE_ORDER = 1
};

/* One fused AdamW step over a flat fp32 shard, in place (p, m, v); replaces the
 * seven elementwise torch passes of ShardedAdamW.update (tandem/optim.py:28-37):
 *     p *= decay;  m = fma(w1, g - m, m);  v = fma(one_m_b2 * g, g, v * beta2);
 *     d = sqrt(v) / bc2_sqrt + eps;  p += (neg_step * m) / d
 * with IEEE sqrt and division. */
int tdm_k3_adamw(float* p, const float* g, float* m, float* v, int64_t n, const tdm_adamw_scalars* s, int order,
                 tdm_stream stream);

/* The same step, and the all-gather that follows it in ZeRO's step (tandem/zero.py:160-164),
 * in one pass: the updated parameters are also written to `ncopies` (<= 7) further buffers,
 * the other ranks' copies of this shard. For ranks that are buffers in one memory; saves
 * the gather's read of p and one launch per ring step. */
int tdm_k3_adamw_gather(float* p, const float* g, float* m, float* v, int64_t n, const tdm_adamw_scalars* s, int order,
                        float* const* copies, int ncopies, tdm_stream stream);

/* The step's constants as the Python doubles of tandem/optim.py:28-37, unrounded: what an entry point that takes the
 * shard's element type needs, since a Python double is applied to a tensor in the tensor's own arithmetic. */
typedef struct tdm_adamw_hyper {
  int32_t use_decay; /* weight_decay != 0 */
  int32_t reserved;
  double decay;      /* 1 - lr * weight_decay */
  double w1;         /* 1 - beta1 */
  double beta2;
  double one_m_b2;   /* 1 - beta2 */
  double bc2_sqrt;   /* (1 - beta2**t) ** 0.5 */
  double eps;
  double neg_step;   /* -(lr / (1 - beta1**t)) */
} tdm_adamw_hyper;

/* tdm_k3_adamw / tdm_k3_adamw_gather for shards of fp32 (TDM_F32), float64 (TDM_F64), bfloat16 (TDM_BF16) or float16
 * (TDM_F16): the reference's update is seven torch operations that take any floating dtype (tandem/optim.py:28-37).
 * `copies` may be NULL with ncopies 0. fp32: the constants are rounded to fp32 once and the call is
 * tdm_k3_adamw(_gather), in either order. float64: the same operations on doubles, the constants unrounded. The
 * 16-bit types: every one of the seven operations computes in fp32 and rounds its result to the type (nearest even),
 * as ATen's kernels for such tensors do; eps is added rounded to the type (float16 turns 1e-8 into 0, as it does for
 * the reference), the other constants act as fp32; a NaN is stored as the type's canonical quiet NaN. Everything but
 * fp32 follows torch's CPU kernels (TDM_ADAMW_HOST_ORDER); TDM_ADAMW_DEVICE_ORDER is refused for it. */
int tdm_k3_adamw_typed(void* p, const void* g, void* m, void* v, int64_t n, int dtype, const tdm_adamw_hyper* h, int order,
                       void* const* copies, int ncopies, tdm_stream stream);

/* ---- K2 + K3: ZeRO-2's reduce-scatter, gradient add, AdamW and all-gather in one launch ---- */

/* One segment: `count` elements that lie in ring chunk `chunk` (= the rank that owns
 * them) of a ZeRO bucket. grad[r]: rank r's gradient (its staging buffer); param[r]: rank
 * r's copy of the parameters; exp_avg, exp_avg_sq: the owner's optimizer state. `dtype` is the element type of all
 * of them: TDM_F32 (0: what a caller that zeroes the struct and knows nothing of the field leaves there), TDM_F64,
 * TDM_BF16 or TDM_F16; the segments of one table share one dtype. */
/* Entries of ranks beyond the world size must be NULL; alignment as for tdm_fold_seg. */
typedef struct tdm_step_seg {
  const void* grad[TDM_MAX_WORLD];
  void* param[TDM_MAX_WORLD];
  void* exp_avg;
  void* exp_avg_sq;
  int64_t count;
  int32_t chunk;
  int32_t dtype;
} tdm_step_seg;

/* The device table, as for K2: tiles and bytes it needs (-1: bad arguments), its image
 * in host memory (the caller copies it to the device once). */
int64_t tdm_k23_table_tiles(const tdm_step_seg* segs, int nseg);
int64_t tdm_k23_table_bytes(const tdm_step_seg* segs, int nseg);
int tdm_k23_table_build(const tdm_step_seg* segs, int nseg, int world, void* image);

/* For every element of every segment:
 *     mine = the ring-order fold of grad[0..W) (average: each divided by W first), as tdm_k2_bucket_fold
 *     g    = 0 + mine                      (grad_shard.add_(mine) onto a zeroed shard, tandem/zero.py:150-153)
 *     p, exp_avg, exp_avg_sq updated as tdm_k3_adamw does, on the owner's copy
 *     param[r] = p for every rank r        (the all-gather of tandem/zero.py:163)
 * i.e. ZeRO stage 2's communication and optimizer step (tandem/zero.py:141-163) for ranks
 * that are buffers of one process, provided the gradient shards were zero (no accumulation
 * over several backward passes); the same bits, (8W + 20) instead of (12W + 28) bytes per element. */
int tdm_k23_zero2_step(const void* table_dev, int64_t ntiles, int world, int average, const tdm_adamw_scalars* s, int order,
                       tdm_stream stream);

/* The same launch for a table of fp32, float64, bfloat16 or float16 segments, with the step's constants as Python
 * doubles (as tdm_k3_adamw_typed takes them): fp32 is tdm_k23_zero2_step; float64 folds and steps in doubles; the
 * 16-bit types fold as tdm_k2_bucket_fold does for them (every addition rounded to the type) and step as
 * tdm_k3_adamw_typed does. Everything but fp32 in TDM_ADAMW_HOST_ORDER only. `dtype` must be the one the table was
 * built for. */
int tdm_k23_zero2_step_typed(const void* table_dev, int64_t ntiles, int world, int average, int dtype, const tdm_adamw_hyper* h,
                             int order, tdm_stream stream);

/* The same step for ONE segment of fp32, passed in the launch itself (no table in device memory):
 * what a rank that is a process of its own runs over its shard, chunk = its rank. */
int tdm_k23_zero2_step_segment(const tdm_step_seg* seg, int world, int average, const tdm_adamw_scalars* s, int order,
                               tdm_stream stream);
/* The same for one segment of any of K3's shard types (seg->dtype), the step's constants as Python doubles. */
int tdm_k23_zero2_step_segment_typed(const tdm_step_seg* seg, int world, int average, const tdm_adamw_hyper* h, int order,
                                     tdm_stream stream);

/* ---- K4: ZeRO-3 unit gather ---------------------------------------------- */

/* full[lo_q : lo_q + sizes[q]] = shards[q][0 : sizes[q]] for every rank q, in one
 * launch (lo_q = sizes[0] + ... + sizes[q-1]); a shard that already is its slice
 * of `full` is skipped. Replaces `full[lo:hi].copy_(shard)` + the ring all_gather
 * of FSDP._start_gather (tandem/zero.py:238-245, tandem/comm.py:307-311,371-385). */
int tdm_k4_unit_gather(void* full, const void* const* shards, const int64_t* sizes, int world, int dtype,
                       tdm_stream stream);

/* The same gather for EVERY rank of a group whose ranks are buffers of one process, in one launch
 * (world sizes up to 8; one launch per rank beyond): shard q is read once and stored into elements
 * [lo_q, lo_q + sizes[q]) of all `world` buffers fulls[0..world): 4 (W + 1) bytes per element of the
 * unit where W calls of tdm_k4_unit_gather move 8 W. No counterpart in the reference, which has one
 * process per rank. */
int tdm_k4_unit_gather_all(void* const* fulls, const void* const* shards, const int64_t* sizes, int world, int dtype,
                           tdm_stream stream);

/* ---- the engine: Group(backend="hip") --------------------------------------- */

/* One rank's half of a group whose ranks are processes sharing one GPU. Mirrors
 * the object the reference's Group expects from its native plug-in
 * (tandem/comm.py:149-160; constructor tandem/csrc/collectives.cpp:98-117; pybind
 * surface tandem/csrc/engine.cpp:103-122): create on every rank, wait until all
 * ranks have (the launcher's barrier), connect, then collectives. Tensors must be
 * contiguous and in the engine's GPU memory; results are written in place; the
 * caller keeps them alive until the Work has been waited for. */
typedef struct tdm_engine tdm_engine;
typedef struct tdm_work tdm_work;

/* dtype code for tensors that are only copied (all_gather, broadcast, send/recv): raw bytes */
enum { TDM_BYTES = 6 };

/* Creates this rank's outgoing slots (`slots` x `slot_bytes` of device memory per
 * peer, shared through hipIpcGetMemHandle), its interprocess events
 * (hipIpcGetEventHandle) and its shared-memory region "/tandem-<job>-<rank>-hip",
 * and starts the progress thread. Replaces Engine::Engine + CudaLinks::CudaLinks
 * (tandem/csrc/collectives.cpp:98-117, tandem/csrc/cuda_links.cpp:43-84). */
int tdm_engine_create(const char* job, int rank, int size, int slots, int64_t slot_bytes, double timeout_s, int device,
                      tdm_engine** out);

/* Opens what the other ranks created (Engine::connect, CudaLinks::connect:
 * tandem/csrc/collectives.cpp:119-126, tandem/csrc/cuda_links.cpp:86-118). */
int tdm_engine_connect(tdm_engine* e);

/* Runs what is queued, stops the thread, waits for every rank, then releases
 * handles, events and slots (tandem/csrc/collectives.cpp:132-149,
 * tandem/csrc/cuda_links.cpp:162-179). tdm_engine_destroy frees the object. */
int tdm_engine_close(tdm_engine* e);
int tdm_engine_destroy(tdm_engine* e);

/* The collectives. Each validates its arguments in the calling thread, records an
 * event on `caller` (the stream that produced the tensor), queues the work for
 * the progress thread and returns a Work at once. `average` divides by the group
 * size before summing, in the ring's rank order; `sizes` (nsizes == 0: as even as
 * torch.tensor_split) cuts the flat tensor into one chunk per rank. Replace
 * Engine::all_reduce / reduce_scatter / all_gather / broadcast / send / recv /
 * sendrecv / barrier (tandem/csrc/collectives.cpp:314-397; the Python engine's
 * tandem/comm.py:326-460). tdm_sendrecv with dst < 0 is recv, with src < 0 send. */
int tdm_all_reduce(tdm_engine* e, void* ptr, int64_t numel, int dtype, int average, tdm_stream caller, tdm_work** out);
int tdm_reduce_scatter(tdm_engine* e, void* ptr, int64_t numel, int dtype, const int64_t* sizes, int nsizes, int average,
                       tdm_stream caller, tdm_work** out);
/* The same, when the caller only wants its own chunk (ZeRO's use, tandem/zero.py:141-153):
 * the chunks this rank does not own are left as they were instead of holding the ring's
 * partial sums, which lets the engine take one handshake per pass instead of two per piece. */
int tdm_reduce_scatter_owner(tdm_engine* e, void* ptr, int64_t numel, int dtype, const int64_t* sizes, int nsizes, int average,
                             tdm_stream caller, tdm_work** out);
int tdm_all_gather(tdm_engine* e, void* ptr, int64_t numel, int dtype, const int64_t* sizes, int nsizes, tdm_stream caller,
                   tdm_work** out);
int tdm_broadcast(tdm_engine* e, void* ptr, int64_t numel, int dtype, int root, tdm_stream caller, tdm_work** out);
/* K4 for process ranks: places this rank's `shard` into its chunk of `full` and
 * ring-all-gathers the other chunks, on the engine's stream, so that a unit's
 * parameters arrive while the caller's stream still computes the previous unit.
 * Replaces `full[lo:hi].copy_(shard)` + `all_gather(full, sizes, async_op=True)` of
 * FSDP._start_gather (tandem/zero.py:238-245). */
int tdm_unit_gather(tdm_engine* e, void* full, int64_t numel, int dtype, const void* shard, const int64_t* sizes, int nsizes,
                    tdm_stream caller, tdm_work** out);
/* Shared arenas + direct gather (no counterpart in the reference, which stages every
 * gather through its slots): tdm_engine_share allocates `bytes` (< 2 GiB: one exported
 * allocation) of device memory on this rank and publishes its hipIpcMemHandle_t; peers
 * map it on first use. A rank may share up to 64 arenas. A place in a rank's arenas is
 * named by one number, its arena offset: the arena's index (0 for the first one shared)
 * times 2^31, plus the byte offset within that arena; tdm_engine_arena_offset gives it
 * for `bytes` bytes at `ptr` (-1 when they do not lie within one arena of this rank).
 * tdm_unit_gather_direct then fills `full` with W-1 copy kernels that read chunk q
 * straight from rank q's arenas at arena offset peer_offsets[q] (own chunk: from `shard`),
 * on the engine's stream, without any message. The caller must bracket every change of
 * arena contents with tdm_fence, a barrier that is also ordered against the GPU: it
 * starts once `caller` has finished what it held, and a rank's arrival is announced
 * only when its engine stream has finished as well. */
int tdm_engine_share(tdm_engine* e, int64_t bytes, void** ptr);
int tdm_engine_arena_offset(tdm_engine* e, const void* ptr, int64_t bytes, int64_t* offset);
int tdm_unit_gather_direct(tdm_engine* e, void* full, int64_t numel, int dtype, const void* shard, const int64_t* sizes,
                           int nsizes, const int64_t* peer_offsets, int noffsets, tdm_stream caller, tdm_work** out);
int tdm_fence(tdm_engine* e, tdm_stream caller, tdm_work** out);

/* The three collectives for tensors that lie in the ranks' shared arenas (this rank's
 * at `ptr`, rank q's at arena offset peer_offsets[q] of its arenas), with the results of
 * tdm_all_reduce / tdm_reduce_scatter / tdm_all_gather (tandem/comm.py:326-385) bit
 * for bit, by reading the peers' tensors where they lie instead of passing pieces
 * through slots:
 *   all_reduce      fence; this rank folds its own ring chunk out of all W tensors in
 *                   the ring's order for that chunk (the sum order of tandem/comm.py:301-305)
 *                   and writes the result into all W tensors (the arenas are mapped
 *                   writable; chunk r of every tensor is touched by rank r alone); fence.
 *   reduce_scatter  fence; the same fold, written into this rank's tensor only; fence.
 *                   Unlike the ring (tandem/comm.py:350-352), the chunks this rank does
 *                   not own are left as they were.
 *   all_gather      fence; this rank copies every other chunk from its owner; fence.
 * World sizes up to 8 for the two that reduce. The tensors must not change between
 * the call and the end of the Work on any rank. */
int tdm_direct_all_reduce(tdm_engine* e, void* ptr, int64_t numel, int dtype, int average, const int64_t* peer_offsets,
                          int noffsets, tdm_stream caller, tdm_work** out);
int tdm_direct_reduce_scatter(tdm_engine* e, void* ptr, int64_t numel, int dtype, const int64_t* sizes, int nsizes,
                              int average, const int64_t* peer_offsets, int noffsets, tdm_stream caller, tdm_work** out);
int tdm_direct_all_gather(tdm_engine* e, void* ptr, int64_t numel, int dtype, const int64_t* sizes, int nsizes,
                          const int64_t* peer_offsets, int noffsets, tdm_stream caller, tdm_work** out);

/* ZeRO stage 2's reduce_scatter (every bucket), grad_shard.add_, AdamW and all_gather
 * (tandem/zero.py:141-163) as one launch per rank, for ranks whose flat parameter buffer and
 * flat gradient buffer lie in their shared arenas. `param` and `grad` are THIS rank's shard
 * of its own two buffers (`count` fp32 elements, the rank's slice of the flat layout);
 * param_offsets[q] / grad_offsets[q] are the byte offsets of the same slice inside rank q's
 * arena; exp_avg / exp_avg_sq are this rank's optimizer state for the shard (ordinary device
 * memory). The Work: fence (every rank's gradients are complete and nobody computes with
 * the old parameters any more); tdm_k23_zero2_step_segment with chunk = this rank over
 * all ranks' gradients, writing the new parameters into every rank's buffer; fence.
 * `total` (the flat buffer's length) only serves to find ranks that disagree. The same
 * bits as the separate calls provided the gradient shard was zero before (no accumulation
 * over several backward passes). World sizes up to 8. */
int tdm_direct_zero2_step(tdm_engine* e, void* param, const int64_t* param_offsets, const void* grad, const int64_t* grad_offsets,
                          int noffsets, void* exp_avg, void* exp_avg_sq, int64_t count, int64_t total, int average,
                          const tdm_adamw_scalars* s, int order, tdm_stream caller, tdm_work** out);
/* The same for buffers and optimizer state of `dtype` (TDM_F32, TDM_F64, TDM_BF16, TDM_F16; `count` elements of it),
 * the step's constants as Python doubles: tdm_k23_zero2_step_segment_typed between the two fences. */
int tdm_direct_zero2_step_typed(tdm_engine* e, void* param, const int64_t* param_offsets, const void* grad, const int64_t* grad_offsets,
                                int noffsets, void* exp_avg, void* exp_avg_sq, int64_t count, int64_t total, int average, int dtype,
                                const tdm_adamw_hyper* h, int order, tdm_stream caller, tdm_work** out);
int tdm_sendrecv(tdm_engine* e, const void* send, int64_t send_numel, int dst, void* recv, int64_t recv_numel, int src,
                 int dtype, tdm_stream caller, tdm_work** out);
int tdm_barrier(tdm_engine* e, tdm_work** out);

/* Work handle (tandem/csrc/collectives.h:43-66, tandem/csrc/engine.cpp:103-107).
 * wait: blocks the host until the collective's GPU work has been enqueued, then
 * makes `caller` wait for it on the GPU; returns the collective's error, if any.
 * (With the default host ordering between ranks, a collective's last launch is
 * enqueued only when the GPU has finished the hand-over before it, so wait returns
 * about when that last kernel starts, not right after submission. With TANDEM_HIP_WAIT=stream
 * in the environment at tdm_engine_create, wait on a collective that has not run yet makes
 * `caller` wait for a word the engine sets behind the collective's last kernel and returns at
 * once; a failure of that collective is then returned by the next call on the engine.)
 * done: 1 once the GPU has finished it. times: when the progress thread started and
 * finished it, seconds on CLOCK_MONOTONIC (Python's time.perf_counter clock); for a
 * collective submitted while tdm_engine_set_timing was on, when the GPU started it
 * (inputs ready, first kernel not yet begun) and finished its last kernel instead, on
 * the same clock: this form blocks the host until the GPU has finished it. */
int tdm_work_wait(tdm_work* w, tdm_stream caller);
/* wait for callers that only need the ORDER: if the collective has not run yet, `caller` is made to wait for
 * the word the engine sets behind the collective's last kernel and the call returns at once, whatever
 * TANDEM_HIP_WAIT says (where the device cannot park a stream on a value, and when the collective has already run,
 * this is tdm_work_wait). The host can then queue work behind a collective that is still in flight; a failure of
 * that collective is returned by the next call on the engine instead of by this one. The wait is a kernel of the
 * library's own with a time limit (the engine's time limit and ten seconds, or TANDEM_HIP_PARK_LIMIT_S): a stream
 * that gives up goes on, and the next call on the engine fails and says so. The wait is queued BEFORE
 * the write that ends it, so `caller` and the engine's stream must not share a hardware queue (the runtime's wait
 * spins at the head of its queue): in a process limited to fewer than four (GPU_MAX_HW_QUEUES=1..3; HIP's default is 4)
 * nothing is parked and this is tdm_work_wait too. No counterpart in the
 * reference, whose CUDA engine orders its hand-over on the GPU and so never blocks a waiting host for it. */
int tdm_work_wait_stream(tdm_work* w, tdm_stream caller);
int tdm_work_done(tdm_work* w);
int tdm_work_times(tdm_work* w, double* started, double* finished);
int tdm_work_free(tdm_work* w);

/* Device time stamps for the collectives submitted from now on (on != 0) or host
 * time stamps as the reference's engine keeps them (tandem/csrc/collectives.cpp:203-223;
 * the default). Feeds Group.trace (tandem/comm.py:101-102) so that tandem/profile.py's
 * summarize and chrome_trace see the GPU's span of each collective. */
int tdm_engine_set_timing(tdm_engine* e, int on);

#if defined(__GNUC__) || defined(__clang__)
#pragma GCC visibility pop
#endif
#ifdef __cplusplus
}
#endif
#endif /* TANDEM_HIP_H */
