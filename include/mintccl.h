/* mintccl.h - C ABI of libmintccl.so, the MI355X (gfx950) data path.
 *
 * The reference (huangs0/mintccl) has no FFI: its Python host functions launch
 * Triton-JIT kernels directly, passing raw 64-bit device addresses with 0
 * meaning "absent" (common.py:71), a byte count and rank/world integers.  Each
 * entry point below names the reference launch it stands for.  A Python caller
 * binds them with ctypes (see mintccl_amd/_lib.py).
 *
 * Conventions
 *  - plain C types only; device addresses are void* / uint64_t, 0 = absent;
 *  - every function returns 0 on success or a negative mint_error; none throws;
 *  - all work is enqueued on the hipStream_t passed as void* (NULL = the
 *    default stream); no call synchronises with the host, with one exception:
 *    mint_device_info asked for the XCD count (see there);
 *  - the caller owns every buffer and keeps it alive until the stream drains;
 *  - the library keeps no per-call state: calls on different streams are
 *    independent as long as their buffers are.
 */
#ifndef MINTCCL_H
#define MINTCCL_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MINT_MAX_RANKS 8
#define MINT_LINE_BYTES 128u     /* protocol.py:47 BYTES_LL128_MSG */
#define MINT_LINE_PAYLOAD 120u   /* protocol.py:48 BYTES_LL128_RAW */
#define MINT_SECTOR_BYTES 64u    /* unit that becomes visible as a whole */
#define MINT_BLOCK_LINES 8u      /* lines one 64-lane access carries */
#define MINT_BLOCK_MSG 1024u
#define MINT_BLOCK_RAW 960u

typedef enum {
    MINT_OK = 0,
    MINT_ERR_ARG = -1,        /* bad argument (null, range, unknown enum) */
    MINT_ERR_ALIGN = -2,      /* address not 16-byte aligned (staging; buffers of the stand-alone
                                 copy, codec and sum entry points; ring buffers need none) */
    MINT_ERR_GEOMETRY = -3,   /* slot / wave geometry does not divide */
    MINT_ERR_RESIDENCY = -4,  /* grid would not be co-resident on the device */
    MINT_ERR_HIP = -5,        /* a HIP runtime call failed */
    MINT_ERR_TOO_LARGE = -6,  /* a row does not fit a 32-bit offset window; or, for
                                 mint_ring_launch_static, the geometry does not fit
                                 the library's static scratch array */
    MINT_ERR_STAGING = -7,    /* staging_bytes is smaller than mint_ring_staging_bytes() */
    MINT_ERR_NOT_READY = -8   /* mint_ring_launch_static on a stream under capture before the
                                 library has looked up its static array on this device:
                                 call mint_static_init() (or one launch) first */
} mint_error;

typedef enum { MINT_LAYOUT_PAIR = 0, MINT_LAYOUT_WAVE64 = 1 } mint_layout;
typedef enum { MINT_F16 = 0, MINT_BF16 = 1, MINT_F32 = 2, MINT_BYTES = 3 } mint_dtype;
typedef enum { MINT_PROTO_LL128 = 0, MINT_PROTO_SIMPLE = 1 } mint_protocol;
typedef enum {
    MINT_OP_SENDRECV = 0,      /* 2_sendrecv_indirect.py:44-93, 3_sendrecv_buffer.py:23-74 */
    MINT_OP_BROADCAST = 1,     /* 4_broadcast.py:27-76 */
    MINT_OP_REDUCE = 2,        /* 5_reduce.py:36-95 */
    MINT_OP_ALLGATHER = 3,     /* 6_allgather.py:79-138 (spatial variant) */
    MINT_OP_REDUCESCATTER = 4, /* 7_reducescatter.py:13-79 */
    MINT_OP_ALLREDUCE = 5,     /* the reference's planned 8_allreduce (README.md:23):
                                  reducescatter and allgather in one pass round the ring */
    MINT_OP_ALLTOALL = 6,      /* the reference's planned 9_alltoall (README.md:24,50):
                                  row d of rank s goes into row s of rank d, every
                                  row straight to its destination through the
                                  destination's staging (input[] and output[] must
                                  not overlap) */
    MINT_OP_TREE_BROADCAST = 7, /* broadcast and reduce over a binary tree, an open */
    MINT_OP_TREE_REDUCE = 8,    /* item of the reference's roadmap (README.md:52-55).
                                  The tree is laid over ring[] turned so that the
                                  root comes first: node h (0 = root) has parent
                                  (h - 1) / 2 and children 2h + 1, 2h + 2.  Buffers
                                  as for BROADCAST / REDUCE; a node's sum is
                                  (own + first subtree) + second subtree, one
                                  rounding per addition.  LL128 only.  slot_bytes
                                  of a TREE_REDUCE holds two shares (one per
                                  child). */
    MINT_OP_HYPERCUBE_REDUCESCATTER = 10, /* reduce-scatter and allgather over a */
    MINT_OP_HYPERCUBE_ALLGATHER = 11,     /* hypercube, the last open topology of the
                                  reference's roadmap (README.md:52-55): recursive
                                  halving / doubling, log2(world) exchanges instead
                                  of world - 1 hops; world is 2, 4 or 8.  Node i is
                                  rank ring[i]; in exchange k = 0.. nodes i and
                                  i ^ (world >> (k + 1)) split the rows they still
                                  hold.  Buffers as for REDUCESCATTER / ALLGATHER;
                                  the value a node passes on is
                                  ((own + partner 0) + partner 1) + partner 2, one
                                  rounding per addition.  LL128 only.  slot_bytes
                                  holds world - 1 shares (the streams a rank
                                  receives). */
    MINT_OP_ALLGATHER_TEMPORAL = 9 /* 6_allgather.py:25-77, the schedule the
                                  reference's allgather launches (:157): the whole
                                  grid moves rank 0's row round the ring, then rank
                                  1's, ...; one pipeline, so slot_bytes holds one
                                  row's share.  Same descriptor and same result as
                                  MINT_OP_ALLGATHER.  LL128 only. */
} mint_op;
typedef enum {
    MINT_PLACE_SPREAD = 0,  /* ring neighbours on consecutive blocks (adjacent XCDs) */
    MINT_PLACE_LOCAL = 1    /* every hop of a channel on the same XCD: each block takes its
                               work from the XCD it runs on; needs a device that deals
                               every 8 consecutive blocks to 8 different XCDs
                               (mint_device_info reports 8, mint_xcd_map shows the order) */
} mint_placement;

typedef enum {
    MINT_FETCH_INLINE = 0,  /* every wave-channel loads its own rows itself, one
                               group ahead, into registers */
    MINT_FETCH_LDS = 1      /* reducing ops on LL128: one more wavefront per thread
                               block streams the own rows of the block's
                               wave-channels from HBM into LDS several groups
                               ahead and the wave-channels read them there, so
                               that a poll of staging never queues behind an HBM
                               fetch (vector-memory loads of one wavefront
                               return in issue order).  Ignored by the ops and
                               the protocol that have no such kernel. */
} mint_row_fetch;

/* Status block written by the ring kernel (device memory, 4 x uint64, zeroed
 * by the caller before launch).  word 0: 0 = OK, else 1 = a bounded wait ran
 * out; word 1: (pipeline << 32 | position << 16 | wave) of the first waiter
 * that gave up; word 2: step it waited for; word 3: low half = abort flag
 * polled by all other waits, high half = number of launches that started
 * with the flag already set (they give up at their first wait).  Error code 2: MINT_PLACE_LOCAL met an XCD number beyond 7; word 2
 * then holds that number.  Error code 3: MINT_PLACE_LOCAL, and a thread block
 * found every seat of its XCD taken or waited in vain for its compute unit's
 * number: the device did not deal an eighth of the grid to every XCD (blocks
 * may be dealt over the compute units of an XCD in any way - a stream with a
 * CU mask, compute units busy with other kernels, a grid that is resident in
 * parts).  The same launch with MINT_PLACE_SPREAD (cache_policy 0) will do.
 * The words stay set until the caller zeroes them: every launch that finds
 * word 3 set gives up at its first wait (after at most 64 polls) and leaves
 * unspecified output, and only the first failure is recorded.  After a
 * non-zero word 0 the caller synchronises the stream, zeroes the block and
 * treats the outputs of every launch since the last clean check as lost;
 * under MINT_PLACE_LOCAL it also zeroes the staging before it is used again
 * (a launch that ends early can leave seat counters behind; the slots
 * themselves need no clearing: the next launch brings its own epoch).
 * The reference has no abort path (common.py:106 is unused). */
#define MINT_STATUS_WORDS 4

/* One ring collective over `world` virtual ranks of one GPU.  It stands for the
 * argument lists (recvbuff, sendbuff, inputbuff, outputbuff, count[, rank,
 * dest, world_size, root]) of the reference kernels, for all ranks at once. */
typedef struct {
    int32_t op;            /* mint_op */
    int32_t protocol;      /* mint_protocol */
    int32_t dtype;         /* mint_dtype; MINT_BYTES for the copying ops */
    int32_t world;         /* number of virtual ranks, 1..MINT_MAX_RANKS */
    int32_t ring[MINT_MAX_RANKS + 1]; /* rank sequence, ring[world] == ring[0]
                              (topology.py:56-93); for SENDRECV the route
                              src..dst of route_len ranks */
    int32_t route_len;     /* SENDRECV only: number of ranks on the route */
    int32_t root;          /* BROADCAST / REDUCE / TREE_* root rank */
    uint64_t input[MINT_MAX_RANKS];   /* per rank; 0 = absent */
    uint64_t output[MINT_MAX_RANKS];  /* per rank; 0 = absent */
    uint64_t staging[MINT_MAX_RANKS]; /* per rank, mint_ring_staging_bytes() each */
    uint64_t staging_bytes; /* bytes the caller allocated behind every staging[r];
                              a launch whose slots and credit words would not
                              fit is refused with MINT_ERR_STAGING (the credit
                              words sit behind the slots, outside a buffer
                              that only holds nslots * slot_bytes) */
    uint64_t count_bytes;  /* SENDRECV/BROADCAST/REDUCE/ALLREDUCE/TREE_*: bytes of the
                              buffer; ALLGATHER(_TEMPORAL)/REDUCESCATTER/ALLTOALL/HYPERCUBE_*:
                              bytes of one row */
    uint64_t row_stride;   /* ALLGATHER/REDUCESCATTER/ALLTOALL/HYPERCUBE_*: bytes between rows */
    uint32_t slot_bytes;   /* staging bytes of one step over all pipelines;
                              multiple of 1024, >= 1024 per pipeline (per
                              pipeline and phase for ALLREDUCE, which has 2;
                              per source rank for ALLTOALL) */
    uint32_t nslots;       /* slots in the circular staging buffer */
    uint32_t waves_per_channel_group; /* wave-channels per (pipeline, hop) */
    uint32_t threads_per_block;       /* multiple of 64 */
    int32_t placement;     /* mint_placement */
    int32_t cache_policy;  /* how staging is accessed: 0 agent scope (sc1),
                              1 system scope (sc0 sc1), 2 XCD-local (stores
                              stay in the XCD's L2; needs MINT_PLACE_LOCAL) */
    uint32_t flag_epoch;   /* 1..4095; must differ from every earlier launch
                              that used the same staging memory since that
                              memory was last zeroed */
    uint32_t spin_budget;  /* polls before a wait gives up; 0 = default */
    uint64_t status;       /* device address of MINT_STATUS_WORDS uint64 */
    int32_t row_fetch;     /* mint_row_fetch: who reads the ranks' own rows */
    uint32_t credit_offset; /* byte offset of the credit words inside each rank's
                               staging; 0 = right after the slots.  A caller
                               that changes slot geometry between launches on
                               the same staging keeps this fixed (beyond its
                               largest nslots * slot_bytes, multiple of 256) so
                               that credit words and payload never share bytes */
    uint64_t total_bytes;  /* ALLGATHER / REDUCESCATTER: 0, or the rows are the
                              pieces of one buffer of total_bytes bytes, cut
                              every row_stride bytes: row p ends where the
                              buffer ends (short or empty last rows), and
                              count_bytes is the length of a full row.  This
                              is how an allreduce runs as a reducescatter
                              followed by an allgather.  Other ops: 0. */
    uint64_t epoch_ptr;    /* 0, or the device address of a uint32 that holds
                              the epoch: the kernel reads it there and
                              flag_epoch is ignored.  For launches that are
                              captured into a HIP graph and replayed: put a
                              mint_epoch_advance on the same word in front of
                              every launch. */
    uint32_t origin_cus;   /* 0, or of the 32 compute units of an XCD so many
                              hold nothing but origins (the positions that
                              read the caller's rows from HBM): SENDRECV,
                              BROADCAST, TREE_BROADCAST, ALLGATHER(_TEMPORAL) and ALLTOALL under MINT_PLACE_LOCAL
                              with at least 64 thread blocks per position
                              and 16 steps, below 32; ignored elsewhere, and
                              where the larger grid it needs (blocks with
                              nothing to do fill the rounds) would not be
                              resident.  A matter of speed only: a compute
                              unit keeps a bounded number of loads in flight,
                              and an eighth of them cannot feed an 8-rank
                              ring.  No counterpart in the reference. */
    uint32_t reserved1;    /* 0 */
} mint_ring_op;

/* 100 * major + minor of this interface: 102 = mint_build_flags, mint_static_init,
 * mint_step_mix_deep, mint_ring_seat, MINT_OP_HYPERCUBE_*; mint_epoch_advance takes
 * the protocol; every rank's staging grew by the seat counters; status word 3 counts
 * launches that started aborted (101 = mint_ring_op with origin_cus).  A binding checks it against the
 * version it was written for before it passes a descriptor. */
int mint_version(void);
/* What the library was compiled with, as bits.  A product build returns 0.
 *   MINT_BUILD_RING_STATS   -DMINT_RING_STATS: the ring kernels collect wait
 *                           accounting (mint_ring_debug.stats); results are right,
 *                           times a few per cent longer
 *   MINT_BUILD_ROW_NOLOAD   -DMINT_ROW_NOLOAD: whole blocks of the callers' rows
 *                           are not loaded (their block numbers travel instead):
 *                           WRONG RESULTS BY DESIGN, for timing a collective
 *                           without its reads from HBM
 * No counterpart in the reference. */
#define MINT_BUILD_RING_STATS 1
#define MINT_BUILD_ROW_NOLOAD 2
int mint_build_flags(void);
const char* mint_strerror(int err);

/* Compute units, XCDs and wavefront size of the current device (the reference
 * asks torch for the multiprocessor count, common.py:72; XCDs have no
 * counterpart there).  Any pointer may be NULL.  Asking for `xcds` is the one
 * call of this library that allocates and synchronises: it runs a 64-block
 * probe on the default stream and waits for it - a set-up call, not one for a
 * serving loop or a stream under capture (mint_xcd_map is the asynchronous
 * form).  `xcds` is the number of distinct XCDs the probe's blocks landed on;
 * when that is 8 but some aligned group of 8 consecutive blocks did not land
 * on 8 different XCDs - the dealing MINT_PLACE_LOCAL is built on - it is
 * reported as 0 and MINT_PLACE_SPREAD is the placement to use.  (A launch
 * with MINT_PLACE_LOCAL on a device that deals otherwise loses no data
 * silently: some (channel, position) is then served twice and another not at
 * all, the neighbours' bounded waits run out, status word 0 says 1 and
 * in-place buffers are left partly updated.) */
int mint_device_info(int* compute_units, int* xcds, int* wave_size);

/* XCC_ID of the XCD each of `blocks` thread blocks of a 1-D launch lands on
 * (device uint32[blocks]).  No counterpart in the reference; documents the block -> XCD dealing order that the
 * placement option relies on: round-robin, starting at an XCD that depends on
 * the hardware queue behind the stream. */
int mint_xcd_map(int blocks, void* out, void* stream);

/* Simple-protocol copy, 16 bytes per lane, persistent grid.
 * Stands for recv_kernel (1_sendrecv_direct.py:31-54); also the HBM
 * copy-bandwidth yardstick.  blocks = 0 picks a device-filling grid. */
int mint_copy_simple(const void* src, void* dst, size_t nbytes, int blocks, int threads,
                     void* stream);

/* Read-only pass over a buffer: XORs every whole 16-byte vector of
 * src[0, nbytes) into out (device uint32[4], which the caller has zeroed; the
 * kernel only XORs into it).  No counterpart in the reference: it is the HBM
 * read-bandwidth yardstick beside mint_copy_simple, and its result can be
 * checked.  blocks = 0 picks a device-filling grid. */
int mint_read_xor(const void* src, size_t nbytes, void* out, int blocks, int threads,
                  void* stream);

/* The memory traffic of the ring kernels' inner loop without the ring: `waves`
 * wavefronts each run `iters` steps of, as `what` selects (bits),
 *   1  a 16-byte-per-lane streaming load of the wave's own 960-byte block from
 *      `rows` (block i * waves + w in step i: needs waves * iters * 960 bytes),
 *   2  a 16-byte-per-lane agent-scope load of 1 KiB from one of the wave's two
 *      private slots in `staging` (needs waves * 2048 bytes, 16-byte aligned),
 *   4  a 16-byte-per-lane store of the f16 sum of the two into the other slot,
 *   8  (with 1) the own block is loaded straight into LDS (buffer_load ... lds)
 *      and read from there, instead of into registers,
 *  16  (without 1 and 8) a streaming store of the block back into `rows`, as a
 *      copying position saves what it received (`rows` is written),
 * 256 * k (k = 2, 4, 5, 6, 8 or 12, with 1 + 2 + 4 only) k times sixteen scalar
 *      additions between the loads and the store of a step: the bookkeeping
 *      of a ring step without the ring,
 * with no flags and nobody waiting for anybody.  The launch takes what the
 * device needs for that mix of accesses however well a ring schedules them:
 * the yardstick beside mint_copy_simple and mint_read_xor.  `sink` (device
 * uint32, may hold anything) is only written when no store is selected.  No
 * counterpart in the reference. */
int mint_step_mix(const void* rows, size_t rows_bytes, void* staging, size_t staging_bytes,
                  int waves, int iters, int what, void* sink, void* stream);

/* mint_step_mix with several steps in flight per wavefront.  mint_step_mix has
 * one: a step's loads are waited for and its store is issued before the next
 * step's loads go out, so its time is steps x (load latency + store latency)
 * and need not be what the device can do with the mix.  Here (`what` bits 1,
 * 2, 4 as above) the loads run `ahead` = 1..3 steps ahead of their use and go
 * out before the store of the step in hand: ahead + 1 steps of loads in flight
 * per wavefront, the stores never waited for.  A wavefront owns ahead + 2 slots
 * of 1 KiB in `staging` (needs waves * (ahead + 2) * 1024 bytes); with
 * `partner` != 0 it loads what the same wavefront of the thread block 8
 * further on stores (the same XCD, another compute unit - a line is written
 * by one compute unit and read by another, as in a ring), else what it stored
 * itself ahead + 1 steps earlier.  `iters` is a multiple of ahead + 1.  No
 * counterpart in the reference. */
int mint_step_mix_deep(const void* rows, size_t rows_bytes, void* staging, size_t staging_bytes,
                       int waves, int iters, int what, int ahead, int partner, void* sink,
                       void* stream);

/* Standalone LL128 codec (load_ll128 + send_ll128 / recv_ll128 + save_ll128,
 * protocol.py:57-137).  Line L (0-based) carries flag_base + L * flag_stride:
 * MINT_LAYOUT_PAIR is the reference's wire format (120 payload bytes, then the
 * flag as 8 little-endian bytes); MINT_LAYOUT_WAVE64 is the format the ring
 * kernels use (per 64-byte sector 60 payload bytes, then the low 32 bits of
 * the flag).
 * msg must hold mint_ll128_packed_bytes(nbytes, layout).  bad_flags (device
 * uint64, may be 0) is incremented once per line whose flag is not the
 * expected one. */
size_t mint_ll128_packed_bytes(size_t nbytes, int layout);
int mint_ll128_pack(const void* raw, void* msg, size_t nbytes, uint64_t flag_base,
                    uint64_t flag_stride, int layout, void* stream);
int mint_ll128_unpack(const void* msg, void* raw, size_t nbytes, uint64_t flag_base,
                      uint64_t flag_stride, int layout, void* bad_flags, void* stream);

/* out = rn(a + b) elementwise with the reduction's own device function
 * (SumFP16, primitive.py:232-247; comp_ll128, protocol.py:142-156). */
int mint_elementwise_sum(const void* a, const void* b, void* out, size_t nelem, int dtype,
                         void* stream);

/* Bytes of staging each rank needs for this op (slots plus credit words). */
size_t mint_ring_staging_bytes(const mint_ring_op* op);
/* Blocks the launch will use; negative mint_error if the geometry is bad. */
int mint_ring_grid_blocks(const mint_ring_op* op);
/* The chunk schedule of one wave-channel, listed on the host by the code the
 * kernels walk (the reference computes it inline in every kernel: sendrecv
 * 2_sendrecv_indirect.py:61,76-77, buffered 3_sendrecv_buffer.py:32-34,46-47,
 * reducescatter 7_reducescatter.py:23-34,43-44,75-77, allgather
 * 6_allgather.py:42,57-59,91-102).  For wave-channel `wave` at `position`
 * (0 = origin .. hops = sink) of `pipeline`, in the order it handles them:
 * step[i], block[i] (block number inside the row: 960 raw bytes for LL128,
 * 1024 for Simple), recv_offset[i] / send_offset[i] (byte offset of the
 * block's 1 KiB message inside the staging of the rank it is received in /
 * sent to).  Any output array may be NULL; at most max_entries are written,
 * *n_entries is the full count.  Needs no GPU.  The tree ops and the temporal
 * allgather are not listed (MINT_ERR_ARG). */
int mint_ring_schedule(const mint_ring_op* op, int pipeline, int position, int wave,
                       uint32_t max_entries, uint32_t* step, uint32_t* block,
                       uint32_t* recv_offset, uint32_t* send_offset, uint32_t* n_entries);
/* Which seat a thread block takes under MINT_PLACE_LOCAL, computed on the host
 * by the code the kernels run.  The reference maps program_id to its work
 * directly (7_reducescatter.py:23-25: every rank is a GPU of its own); here a
 * block claims an entry of the list of the XCD it finds itself on: the
 * compute unit that was the `cu_rank`-th of XCD `xcd` to show up wants, with
 * its `nth` block (0-based), entry nth * 32 + cu_rank; a block beyond a
 * compute unit's share, of a compute unit beyond the 32nd, or whose entry is
 * taken, draws a ticket and takes the first free entry from its ticket's
 * place in the last, partial round (later tickets: from the head of the list)
 * upwards.  A launch of at most 32 entries per XCD (no compute
 * unit gets a second block) takes the whole list by ticket.  `state` is the
 * XCD's counters, MINT_SEAT_STATE_WORDS words that the caller zeroes before
 * the first block of a simulated launch and passes to every call for that
 * XCD, in the order in which the blocks arrive.  Returns 1 and the seat
 * (pipeline, position, block of the position's group of thread blocks), 0 if
 * the block has nothing to do, or a negative mint_error.  Needs no GPU: the
 * test of "every seat exactly once however the blocks are dealt". */
#define MINT_SEAT_STATE_WORDS 17
int mint_ring_seat(const mint_ring_op* op, int xcd, int cu_rank, int nth, uint64_t* state,
                   int* pipeline, int* position, int* block_of_group);

/* Validate and enqueue one fused launch that runs every rank's kernel: the
 * Triton launches kernel[(NUM_BLOCKS,)](recvbuff, sendbuff, inputbuff,
 * outputbuff, count, ...) of 2_sendrecv_indirect.py:165-166,
 * 3_sendrecv_buffer.py:150-151, 4_broadcast.py:100-101, 5_reduce.py:120-121,
 * 6_allgather.py:157-158 and 7_reducescatter.py:97-98, for all ranks at once. */
int mint_ring_launch(const mint_ring_op* op, void* stream);

/* Test hooks, kept out of the descriptor.  skip_origin != 0: the origin hop of
 * every pipeline sends nothing, so every other wait runs out (exercises the
 * bounded waits and the status block).  stats: 0, or - in a library built
 * with -DMINT_RING_STATS only, others refuse it - the device address of
 * (hops + 1) x 8 zeroed uint64 that receive, per position, {groups, re-polls,
 * ticks waiting for credit, ticks polling, ticks total, wavefronts, ticks
 * waiting for own rows fetched ahead (LL128 copying walks and the walk with
 * own rows through LDS), ticks issuing a step's loads and stores (LL128
 * copying walks; the LDS walk: its fetchers' wait for room)}; a tick is
 * 10 ns.  No counterpart in the reference. */
typedef struct {
    uint32_t skip_origin;
    uint32_t reserved0;
    uint64_t stats;
} mint_ring_debug;
int mint_ring_launch_debug(const mint_ring_op* op, const mint_ring_debug* dbg, void* stream);

/* mint_ring_launch for callers that cannot allocate device memory: code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.
 * It has no counterpart in the reference (whose host functions allocate their
 * staging with torch on every call, e.g. 7_reducescatter.py:93).
 * The descriptor is the one of mint_ring_launch, except that staging[],
 * staging_bytes, credit_offset, flag_epoch and epoch_ptr are ignored: slots,
 * credit words and the launch epoch live in a static device array inside the
 * library, MINT_STATIC_SCRATCH_BYTES on every GPU the library runs on, held
 * until the process ends.  The caller still passes input[], output[] and
 * status.  Every rank gets MINT_STATIC_RANK_BYTES of it: a geometry with
 * nslots * slot_bytes > MINT_STATIC_SLOT_BYTES or with more than
 * MINT_STATIC_CHANNELS wave-channels per rank (pipelines x phases x
 * waves_per_channel_group) is refused with MINT_ERR_TOO_LARGE.
 * The call enqueues, on `stream`, a one-block kernel that advances the epoch
 * kept in the array and the ring launch; it calls no hipMalloc / hipFree and no
 * allocating library routine.  The epoch kernel clears the array (a fill of
 * its own, no memset) on first use, when the 12-bit count starts over, and when
 * an LL128 launch follows a Simple one - which it decides on the device, from
 * a word in the array that holds the protocol of the launch before, so a
 * launch captured into a graph decides anew at every replay, whatever ran
 * between the replays.  All calls on a GPU share that GPU's array: two calls
 * that overlap in time on one GPU (different streams, or threads) race - keep
 * them on one stream.  The first call on a device looks the array's address up
 * (hipGetSymbolAddress) with that device current; a stream under capture is
 * no place for that, so a caller that captures calls mint_static_init() on
 * the device beforehand (MINT_ERR_NOT_READY otherwise). */
#define MINT_STATIC_SCRATCH_BYTES (16u << 20)
#define MINT_STATIC_HEADER_BYTES 4096u
#define MINT_STATIC_RANK_BYTES ((MINT_STATIC_SCRATCH_BYTES - MINT_STATIC_HEADER_BYTES) / MINT_MAX_RANKS)
#define MINT_STATIC_CHANNELS 1024u
#define MINT_STATIC_SLOT_BYTES (MINT_STATIC_RANK_BYTES - MINT_STATIC_CHANNELS * 256u - 32768u)
int mint_ring_launch_static(const mint_ring_op* op, void* stream);
/* Looks up the address of the static array on the current device (once; later
 * calls return at once).  Enqueues nothing and allocates nothing.  For callers
 * of mint_ring_launch_static that capture their first launch. */
int mint_static_init(void);

/* Advances the epoch word a mint_ring_op points to with epoch_ptr (device
 * uint32, zero before its first use): 1, 2, ..., 4095, 1, ...  Whenever the
 * count starts over (and on first use) the kernel also zeroes
 * staging[0, staging_bytes) - the whole staging allocation of all ranks - as
 * the epoch contract demands.  `protocol` = -1, or the mint_protocol of the
 * launch that follows: then `epoch_word` points to TWO uint32 (both zero
 * before their first use), the second remembers the protocol of the launch
 * before, and the staging is also cleared when an LL128 launch follows a
 * Simple one on it (raw payload of a Simple launch could pass for LL128 sector
 * tags).  Enqueued on `stream` like a launch; it is what makes a captured
 * sequence of collectives replayable, because a replay then sees fresh epochs
 * and takes the clearing decision itself, on the device.  No counterpart in the
 * reference (its flags restart with every launch and it clears nothing). */
int mint_epoch_advance(void* epoch_word, void* staging, size_t staging_bytes, int protocol,
                       void* stream);

/* Torn-line probe: `pairs` producer wavefronts each rewrite 1 KiB blocks of
 * their own `iters` times; every 64-byte sector carries a tag and a payload
 * that is a function of the tag.  The paired consumer wavefronts poll until
 * the tags appear and count 128-byte lines holding bytes that do not belong to
 * the tag.  per_sector = 1: all 16 sector tags of a block are tested (the ring
 * kernels' format); per_sector = 0: only the tag of the second sector of each
 * line is tested (one flag per 128-byte line, the reference's assumption,
 * protocol.py:31-35).  counters: device uint64[8] = {lines checked, torn
 * lines, polls, timeouts, torn lines whose first sector alone was stale, 0..}.
 * flag_epoch is 1..4095.  With MINT_PLACE_LOCAL the pair count must be a
 * multiple of 32 (whole blocks per XCD). */
int mint_torn_line_probe(void* staging, size_t staging_bytes, int pairs, int iters,
                         int cache_policy, int placement, int per_sector, uint32_t flag_epoch,
                         uint32_t spin_budget, void* counters, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* MINTCCL_H */
