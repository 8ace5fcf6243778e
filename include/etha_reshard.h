/*
 * etha_reshard.h — C ABI of the MI355X (gfx950) redistribute hot path.
 *
 * The library sits exactly under the two methods the reference's executor calls on
 * every bucket: Bucket.prepare() (assemble the send bucket from strided chunks of
 * the source shard, src/etha/comm/ir.py:229-264 with Chunk.prepare ir.py:101-132)
 * and Bucket.finalize() (scatter a received bucket into the target shard,
 * ir.py:300-310 with Chunk.finalize ir.py:134-141).  The host planner describes
 * every chunk once ("plan once, transfer N times"); the library compiles the
 * descriptors into a device-resident tile program and each transfer is then one
 * batched kernel launch per bucket, per run of buckets, or per set of buckets that
 * do not depend on each other (etha_launch_segments).
 *
 * Conventions
 *  - plain C types only; every function returns 0 on success or a negative
 *    ETHA_ERR_* code and never throws; etha_last_error() gives the message of the
 *    calling thread's last failure.
 *  - `stream` arguments are a hipStream_t passed as void* (NULL = default stream).
 *    Launches are asynchronous; ordering is stream ordering, as in the reference
 *    where all device work of a transfer goes to the current stream
 *    (ir.py:262-275, comm_methods.py:119).
 *  - the library never writes a tensor outside the described chunk regions and
 *    never writes a source tensor at all (pinned by the reference's
 *    tests/test_communication_replicate_shard.py:166-170,189-192).
 */
#ifndef ETHA_RESHARD_H
#define ETHA_RESHARD_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ETHA_ABI_VERSION 6
#define ETHA_MAX_NDIM 8

/* status codes */
#define ETHA_OK 0
#define ETHA_ERR_INVALID (-1)     /* bad argument / descriptor rejected by validation */
#define ETHA_ERR_UNSUPPORTED (-2) /* legal in the reference but not implemented here */
#define ETHA_ERR_HIP (-3)         /* a HIP runtime call failed */
#define ETHA_ERR_NOMEM (-4)

/* element types.  Same-type transfers are byte moves and work for every type.  Conversions
 * (Chunk.prepare / Chunk.finalize call buffer.to(dtype), ir.py:125-126,137-138) are implemented between all
 * value types: vectorised between the four IEEE-style floats, element by element when an integer, bool or
 * 8-bit float is involved.  Semantics are ATen's: round to nearest even into floats, truncation toward zero
 * into integers (values that do not fit, and NaN, give what ATen's x86 kernels give: INT32_MIN / INT64_MIN,
 * narrower results the low bits, uint8 through int64), != 0 into bool.  Opaque types can only be moved. */
enum {
  ETHA_F16 = 0,
  ETHA_BF16 = 1,
  ETHA_F32 = 2,
  ETHA_F64 = 3,
  ETHA_B8 = 4,   /* opaque 1-byte element */
  ETHA_B16 = 5,  /* opaque 2-byte element */
  ETHA_B32 = 6,  /* opaque 4-byte element */
  ETHA_B64 = 7,  /* opaque 8-byte element (complex64/...) */
  ETHA_I8 = 8,
  ETHA_U8 = 9,
  ETHA_I16 = 10,
  ETHA_I32 = 11,
  ETHA_I64 = 12,
  ETHA_BOOL = 13,
  ETHA_F8E4M3 = 14, /* float8_e4m3fn */
  ETHA_F8E5M2 = 15  /* float8_e5m2 */
};

/*
 * Launch flags.  By default a launch is ordered after everything enqueued on its stream before it, like any
 * kernel.  ETHA_LAUNCH_UNORDERED declares that this launch depends on none of the launches enqueued on the
 * stream since the last launch without the flag: it may start while they are still running, which hides the
 * drain/ramp gap between kernels.  (On a stream under capture the flag is ignored: a captured stream records a
 * chain.)  The next launch without the flag (of this library or any other kernel on
 * the stream) waits for all of them.  The caller owns the dependency analysis: two launches that touch the
 * same bucket buffer, or a launch that reads bytes another one writes, must be separated by an ordered
 * launch.  The reference needs no such notion because each of its buckets is many small ATen launches on one
 * stream (ir.py:246-259); here a bucket is one launch and the gap between launches is what is left to hide.
 */
#define ETHA_LAUNCH_UNORDERED 1u

/* reduce ops of a Partial source (ir.py:51-57) */
enum { ETHA_SUM = 0, ETHA_AVG = 1, ETHA_MAX = 2, ETHA_MIN = 3, ETHA_PRODUCT = 4 };
/*
 * Partial mesh dims with different ops.  The reference all-reduces once per Partial mesh dim, each with its own
 * op, in mesh-dim order (tensor_bus/agent.py:46-70, ir.py:123-124).  ETHA_REDUCE_LEVELS describes that as nested
 * levels: the peers are listed with the first-applied mesh dim varying fastest; op0 combines each run of g0
 * peers, op1 each run of g1 such results, op2 what is left (n_partials / (g0 * g1) of them; pass g1 = 1 and
 * op2 = op1 for two levels).  All levels accumulate in fp32 (f64 for f64 inputs) and the result is rounded
 * once; an ETHA_AVG level divides by its own member count.
 */
#define ETHA_REDUCE_LEVELS(op0, g0, op1, g1, op2) \
  ((uint32_t)(op0) | ((uint32_t)(op1) << 3) | ((uint32_t)(op2) << 6) | ((uint32_t)(g0) << 16) | ((uint32_t)(g1) << 24))

/*
 * One chunk = one strided region of a local shard plus its place in a bucket.
 * Information content of the reference's Chunk (ir.py:60-99) and of the bucket
 * byte offset Bucket.offsets[i] (ir.py:189-194).
 */
typedef struct EthaChunkDesc {
  uint64_t tensor_ptr;            /* device address of the parent tensor's element [0,..,0] (Tensor.data_ptr()) */
  uint64_t tensor_lo, tensor_hi;  /* byte range [lo,hi) the library may touch on the tensor side; both 0 = unchecked */
  uint64_t bucket_ptr;            /* device address of this chunk's first byte inside its bucket buffer */
  uint64_t bucket_lo, bucket_hi;  /* byte range [lo,hi) of that bucket buffer; both 0 = unchecked */
  int64_t start[ETHA_MAX_NDIM];   /* slice start per dim: src_slice when packing, dst_slice when unpacking */
  int64_t shape[ETHA_MAX_NDIM];   /* chunk_shape */
  int64_t stride[ETHA_MAX_NDIM];  /* parent tensor strides, in elements (non-contiguous parents are legal) */
  uint32_t ndim;                  /* <= ETHA_MAX_NDIM; 0 = scalar (one element) */
  uint32_t tensor_dtype;          /* ETHA_* element type of the tensor */
  uint32_t wire_dtype;            /* ETHA_* element type inside the bucket (Chunk.transfer_dtype) */
  uint32_t n_partials;            /* 0 = plain chunk.  >0 = Partial source: reduce this many peers (pack only) */
  uint32_t partial_first;         /* index into partial_ptrs of the first peer's data_ptr(); peers in rank order */
  uint32_t reduce_op;             /* ETHA_SUM.. or ETHA_REDUCE_LEVELS(...) when n_partials > 0 */
} EthaChunkDesc;

typedef struct EthaTable EthaTable; /* compiled, device-resident tile program */

typedef struct EthaTableInfo {
  uint32_t n_chunks;
  uint32_t n_run_tiles;   /* tiles that are one contiguous run on both sides */
  uint32_t n_row_tiles;   /* tiles that walk rows (short/ragged rows, strided elements, reduce) */
  uint32_t tile_threads;  /* units (work-items) per tile; one tile = tile_threads / 64 workgroups of one wavefront */
  uint64_t device_bytes;  /* device memory held by the table */
  uint64_t payload_bytes; /* sum over chunks of numel * wire element size */
  uint32_t n_trans_tiles; /* square blocks (up to 64-256 elements a side, by element size) of transposing chunks, staged through LDS */
  uint32_t reserved;
} EthaTableInfo;

typedef struct EthaIpcHandle {
  uint8_t handle[64]; /* hipIpcMemHandle_t */
  uint64_t offset;    /* byte offset of the exported pointer from its allocation base */
  uint64_t size;      /* size of the whole allocation */
} EthaIpcHandle;

int etha_abi_version(void);
const char* etha_last_error(void);
/* digest of the sources (kernel file + this header) the library was built from, as the build recipe passed it;
 * lets a harness notice a library that is older than the tree.  No counterpart in the reference. */
const char* etha_source_hash(void);
/* kernels this process has launched through the library so far (one call may launch several); for benchmarks
 * that report time per launch.  No counterpart in the reference. */
uint64_t etha_kernel_launches(void);

/*
 * Compile chunk descriptors into a tile program.
 *  descs/n_chunks     host array, chunk order = bucket order (chunks of one bucket adjacent,
 *                     so that a bucket is a [first, first+count) range).
 *  partial_ptrs       host array of peer data_ptr() values referenced by reduce chunks (may be NULL).
 *  upload             non-zero: copy the program to the current HIP device (needed to launch);
 *                     zero: keep it on the host only (planning/inspection without a GPU).
 * Replaces the per-transfer Python work of Bucket.__post_init__/prepare (ir.py:189-194,246-259).
 */
int etha_table_create(const EthaChunkDesc* descs, uint32_t n_chunks, const uint64_t* partial_ptrs,
                      uint32_t n_partial_ptrs, int upload, EthaTable** out);

/*
 * Same-rank (LOCAL transport) chunks: copy src region i to dst region i directly, no bucket.
 * bucket_* fields are ignored; shapes must match pairwise; src.tensor_dtype is converted to
 * dst.tensor_dtype.  Replaces the self-copy bucket path (ir.py:238-244,254-257,136-140).
 */
int etha_selfcopy_table_create(const EthaChunkDesc* src, const EthaChunkDesc* dst, uint32_t n_chunks, int upload,
                               EthaTable** out);

/*
 * Region-to-region copies where producer and consumer tensors sit on one device and no bucket buffer is wanted:
 * src region i is copied (converted) straight into dst region i.  A src with n_partials > 0 is a Partial
 * source: its peers (partial_ptrs, as in etha_table_create) are combined as in etha_reduce_pack_bucket and the
 * result is rounded to src.wire_dtype and then converted to dst.tensor_dtype, the two roundings of the bucket
 * path (Chunk.prepare's cast to transfer_dtype, ir.py:125-126, then Chunk.finalize's cast, ir.py:137-138).
 * For plain chunks wire_dtype is ignored.  Run with etha_selfcopy_bucket; a launched range must be all plain or
 * all Partial chunks.  etha_selfcopy_table_create is this function without Partial sources.
 * No counterpart in the reference (its buckets always cross a process group).
 */
int etha_direct_table_create(const EthaChunkDesc* src, const EthaChunkDesc* dst, uint32_t n_chunks,
                             const uint64_t* partial_ptrs, uint32_t n_partial_ptrs, int upload, EthaTable** out);

int etha_table_destroy(EthaTable* table);
int etha_table_info(const EthaTable* table, EthaTableInfo* out);

/*
 * Inspection of the compiled program (host copies), for CPU-side checking.
 * which: 0 = run tiles (uint64 a, b; uint32 n, meta), 1 = row tiles, 2 = transposing tiles (see etha_reshard.hip).
 * A tile holds up to tile_units units and is executed by tile_units / 64 workgroups of 64 work-items.
 * Copies up to cap_bytes into out and stores the full size in *need_bytes.
 */
int etha_table_read_tiles(const EthaTable* table, int which, void* out, uint64_t cap_bytes, uint64_t* need_bytes);
/* per-chunk first-tile indices, n_chunks+1 entries each */
int etha_table_read_ranges(const EthaTable* table, uint32_t* run_begin, uint32_t* row_begin);
int etha_table_read_trans_ranges(const EthaTable* table, uint32_t* trans_begin);

/*
 * Declare that chunks [first, first+count) are always launched together by etha_unpack_bucket (or
 * etha_selfcopy_bucket).  The library then keeps a second copy of that range's tiles ordered by the
 * address they write, and uses it for launches of exactly this range.  Tiles are independent, so the
 * result is unchanged; what changes is that rows of a target tensor that arrive through different
 * buckets are written at the same time, which keeps DRAM pages open (measured +15 % on short-row
 * scatters).  No counterpart in the reference, whose finalize runs chunk by chunk (ir.py:306-308).
 */
int etha_table_optimize_range(EthaTable* table, uint32_t first, uint32_t count);
/* host copy of an optimized range's tiles, in launch order; same conventions as etha_table_read_tiles, plus
 * which = 3: the piece addresses (uint64) of the range's gather tiles - row tiles that assemble each
 * destination row from the pieces of several chunks, so that whole lines are written at once.  They follow
 * the plain row tiles in which = 1 and run in a kernel of their own. */
int etha_table_read_ordered(const EthaTable* table, uint32_t first, uint32_t count, int which, void* out,
                            uint64_t cap_bytes, uint64_t* need_bytes);

/*
 * Gather chunks [first, first+count) of the table from their tensors into their bucket
 * positions, converting tensor_dtype -> wire_dtype.  One kernel launch.
 * Replaces Bucket.prepare() for a source bucket (ir.py:229-264; Chunk.prepare ir.py:112-126).
 * The range must not contain reduce chunks.
 */
int etha_pack_bucket(const EthaTable* table, uint32_t first, uint32_t count, void* stream, uint32_t flags);

/*
 * Scatter chunks [first, first+count) from their bucket positions into their tensors,
 * converting wire_dtype -> tensor_dtype.  One kernel launch.
 * Replaces Bucket.finalize() for a target bucket (ir.py:300-310; Chunk.finalize ir.py:134-141).
 */
int etha_unpack_bucket(const EthaTable* table, uint32_t first, uint32_t count, void* stream, uint32_t flags);

/*
 * Partial-source buckets: for every chunk combine the n_partials peer regions element-wise
 * (fp32 accumulation in rank order for f16/bf16/f32 inputs, f64 for f64), convert to
 * wire_dtype once, and write the bucket.  One kernel launch; the peers are only read.
 * Replaces the clone + all_reduce + cast of Chunk.prepare (ir.py:116-126).
 * Every chunk of the range must be a reduce chunk.
 */
int etha_reduce_pack_bucket(const EthaTable* table, uint32_t first, uint32_t count, void* stream, uint32_t flags);

/* Run chunks [first, first+count) of a self-copy or direct table.  One kernel launch. */
int etha_selfcopy_bucket(const EthaTable* table, uint32_t first, uint32_t count, void* stream, uint32_t flags);

/*
 * Several bucket launches that do not depend on each other, issued as one unit: what one sweep of the
 * reference's bucket_comm loop prepares and finalizes over all its channels (comm_methods.py:85-116) -
 * packs of the next candidates, unpacks of the arrived buckets, same-rank copies - in as few kernel
 * launches as possible.  Segment i runs chunks [first, first+count) of its table as the entry point named
 * by kind would (ETHA_SEG_PACK = etha_pack_bucket, ...).  No byte written by one segment may be read or
 * written by another: the segments run concurrently.  flags apply to the set as a whole (with
 * ETHA_LAUNCH_UNORDERED the whole set is unordered against earlier launches of the stream).  Segments of one
 * direction and of similar size share a launch (up to ETHA_MAX_SEGMENTS each; the segment is picked by the
 * workgroup's second grid index); transposing and reduce tiles keep their own kernels.  Saves the cost of a
 * launch (about 1.8 us) per segment that joins another's launch.  No counterpart in the reference, whose
 * buckets are many small ATen launches each.
 */
#define ETHA_SEG_PACK 0u
#define ETHA_SEG_UNPACK 1u
#define ETHA_SEG_REDUCE_PACK 2u
#define ETHA_SEG_SELFCOPY 3u
#define ETHA_MAX_SEGMENTS 16u
typedef struct EthaSegment {
  const EthaTable* table;
  uint32_t kind; /* ETHA_SEG_* */
  uint32_t first, count;
  uint32_t reserved; /* 0 */
} EthaSegment;
int etha_launch_segments(const EthaSegment* segments, uint32_t n_segments, void* stream, uint32_t flags);

/*
 * A transfer as one call.  The reference plans once and transfers N times (tensor_bus/batch_state.py:38-40), and
 * every transfer of a planned batch walks the same buckets in the same order through bucket_comm's loop
 * (comm_methods.py:81-117).  A schedule is that walk recorded: the launch calls one transfer made, in order -
 * each an etha_launch_segments call (segments [first_segment, +n_segments) of the segment array with its flags)
 * or, with single = 1, one chunk range run as etha_pack_bucket / etha_unpack_bucket / etha_reduce_pack_bucket /
 * etha_selfcopy_bucket would run it.  etha_schedule_create validates the calls and resolves them into ready-made
 * kernel launches; etha_schedule_launch re-issues them on a stream with no planning left on the host.  The caller
 * owns the claim that the recorded order is still right (same buckets, same readiness order).  The library checks
 * what it can: a schedule whose tables have been destroyed, or changed by etha_table_optimize_range since it was
 * created, refuses to launch with ETHA_ERR_INVALID ("stale schedule") - create a new one.
 */
typedef struct EthaSchedule EthaSchedule;
typedef struct EthaScheduleCall {
  uint32_t first_segment, n_segments; /* range of the segment array */
  uint32_t flags;                     /* launch flags of the call */
  uint32_t single;                    /* 1: n_segments == 1, run as the single-range entry point of its kind */
} EthaScheduleCall;
typedef struct EthaScheduleInfo {
  uint32_t n_calls;
  uint32_t n_kernel_launches; /* kernels one etha_schedule_launch issues */
  uint32_t n_tables;
  uint32_t reserved;
} EthaScheduleInfo;
int etha_schedule_create(const EthaSegment* segments, uint32_t n_segments, const EthaScheduleCall* calls, uint32_t n_calls,
                         EthaSchedule** out);
int etha_schedule_launch(const EthaSchedule* schedule, void* stream);
int etha_schedule_info(const EthaSchedule* schedule, EthaScheduleInfo* out);
int etha_schedule_destroy(EthaSchedule* schedule);

/*
 * Region copies for callers that cannot allocate device memory (tight serving loops, harnesses that forbid
 * hipMalloc).  No counterpart in the reference.
 * etha_copy_regions_noalloc does what etha_selfcopy_table_create + etha_selfcopy_bucket + etha_table_destroy
 * do - copy src region i into dst region i, converting between their dtypes; no Partial sources - but keeps
 * the compiled tile program in a fixed array inside the library instead of in memory from hipMalloc, and calls
 * no hipMalloc / hipFree.  The program of one call may take at most ETHA_NOALLOC_SCRATCH_BYTES (24 bytes per
 * 16 KiB of contiguous payload, 64 bytes per 16 KiB of short-row payload: roughly 1-2.8 GB per call); larger
 * requests are refused with ETHA_ERR_UNSUPPORTED before anything is launched.  Every call on a GPU shares that
 * GPU's array and upload buffer.  Calls from several host threads are serialised by the library; on the device,
 * calls must be issued on one stream, or otherwise ordered so that one call's launches have finished before the
 * next call's begin - calls that overlap on one GPU race.  A stream under HIP graph capture is refused
 * (ETHA_ERR_UNSUPPORTED): the upload would be replayed from a buffer that later calls overwrite.
 * etha_noalloc_setup must have been called once with the device current (it looks up the array's device
 * address and allocates the pinned upload buffer; it is the only part that allocates).
 */
#define ETHA_NOALLOC_SCRATCH_BYTES (4u << 20)
int etha_noalloc_setup(void);
int etha_copy_regions_noalloc(const EthaChunkDesc* src, const EthaChunkDesc* dst, uint32_t n_chunks, void* stream);

/*
 * Bucket-pool memory that can cross a process boundary on the same GPU (the worker <-> agent
 * hand-off the reference does with CUDA-IPC pickling, tensor_bus/client.py:314,
 * tensor_bus/agent.py:608, tensor_bus/utils.py:14-69).  etha_arena_create is a plain
 * hipMalloc so that the allocation base can be exported.
 */
int etha_arena_create(uint64_t nbytes, void** out_ptr);
int etha_arena_destroy(void* ptr);
int etha_ipc_export(const void* dev_ptr, EthaIpcHandle* out);
int etha_ipc_open(const EthaIpcHandle* handle, void** out_ptr); /* returns base + offset */
int etha_ipc_close(void* opened_ptr);

#ifdef __cplusplus
}
#endif
#endif /* ETHA_RESHARD_H */
