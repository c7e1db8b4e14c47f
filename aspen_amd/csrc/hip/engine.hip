// Host side of the flat C ABI (include/aspen_hip.h): device setup, memory, graph upload, the
// per-layer launch path and the persistent dataflow engine.
//
// The dataflow engine is the device-side counterpart of the reference's scheduler:
//   ready pool  (reference src/rpool.c:611-685)  -> one ticket queue in HBM, a slot per tile
//   dse_schedule (reference src/dse.c:20-108)    -> loop of a persistent workgroup
//   update_children (reference src/dse.c:363-401)-> atomic decrement of the children's dependency
//                                                   counters; the last parent publishes the child
//   push_first_layer_to_rpool (src/dse.c:443)    -> arm kernel seeds the queue with the root tiles
#include <hip/hip_runtime.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include "tile_kernels.h"

#define QUEUE_EMPTY 0xffffffffu
typedef unsigned long long qentry_t;      // ready-queue entry / child-record entry, see arm_kernel
#define ST_DONE 64
#define ST_ABORT 96
#define ST_TWICE 128
#define ST_SINKS 160
// Up to one ready queue per XCD (NUM_QUEUES = 8), chosen per run (ASPEN_HIP_FLAG_XCD_QUEUES); by default all tiles go
// through queue 0.  With XCD queues workgroup b, which the dispatcher places on XCD b % 8, serves queue b % 8, and a
// tile's home queue is the eighth of its layer's tile range it lies in, i.e. a fixed eighth of the layer's columns for
// all but the smallest layers.  Tiles that read the same activations (neighbouring output positions, the row tiles and
// split-K slices of one column block, a tile and the tile below it) then run on one XCD and find them in its L2 instead
// of fetching them over the fabric once per XCD: ResNet-50 batch 32 reads 4.9 instead of 8.7 GB per inference.  It is
// not the default because a free workgroup can no longer take a ready tile of another XCD: the same run is 3 % slower
// (transformer graphs, whose layers have fewer tiles than there are workgroups, 6-11 %).
#define NUM_QUEUES 8u
#define ST_QHEAD(q) (192u + 64u * (q))      // pop tickets of queue q
#define ST_QTAIL(q) (224u + 64u * (q))      // push cursor of queue q
#define ST_WORDS (192u + 64u * NUM_QUEUES)
// Co-scheduled networks ("groups", aspen_hip_layer_t.graph_id): each counts its finished tiles without children on a
// line of its own behind the state words; ST_SINKS counts the groups that have finished.
#define MAX_GROUPS 64u
#define ST_GROUP(g) (ST_WORDS + 32u * (g))
#define ST_ALL_WORDS (ST_WORDS + 32u * MAX_GROUPS)
#define HOST_DONE_WORD 16u      // pinned host block: [0] abort flag, [HOST_DONE_WORD + g] = serial of the last run group g finished in
#define NUM_EVENTS 16
#define DEFAULT_SPIN_LIMIT (1ull << 26)
#define ORDERED_BELOW 128.0     // average parallelism (tiles) under which a dataflow run takes its tiles in index order

struct aspen_hip_graph_t
{
    uint32_t num_layers, num_ninst, num_roots, num_edges;
    aspen_hip_layer_t *h_layers;
    aspen_hip_layer_t *d_layers;
    uint32_t *d_ninst_layer, *d_num_parents, *d_child_off, *d_child_idx, *d_roots;
    uint32_t *d_ninst_home;         // per tile: its home queue (0 .. NUM_QUEUES - 1)
    uint32_t *d_root_pos;           // per root: its position among the roots of its home queue
    uint32_t root_count[NUM_QUEUES];
    uint32_t root_shift;            // the XCD grouping (see nq_shift) d_root_pos / root_count were computed for
    uint32_t queue_row, queue_cap;  // see queue_slot
    uint32_t *d_dep;        // remaining-parent counters, re-armed before every dataflow run
    uint32_t *d_dep_spread; // the same, one per cache line, for ordered runs (allocated at the first one), see dep_slot
    uint32_t dep_stride;
    int spread_armed;       // an ordered run has left d_dep_spread and the sink counters armed for the next one (tiles set their own
                            // counters back, see wait_until_ready): no arming pass is needed unless a run was given up since
    qentry_t *d_queue;      // ready queue: slot t is written once, by whoever makes a tile ready
    qentry_t *d_child_rec;  // per tile: child count + its first CHILD_REC-1 children with their layers
    uint32_t *d_state;      // one counter per 128-byte line: [ST_QHEAD (q)] pop tickets, [ST_QTAIL (q)] push cursor of queue q, [ST_DONE] tiles done,
                            // [ST_ABORT] abort flag, [ST_TWICE] tiles executed more than once, [ST_SINKS] finished tiles without children
    uint32_t *d_ran;        // per-tile execution count (sanity: every tile exactly once)
    uint32_t *d_arrivals;   // split-K arrival counters, see run_tile
    uint32_t num_sinks;     // tiles without children
    uint32_t num_groups;    // co-scheduled networks (largest graph_id + 1)
    uint32_t live_groups;   // those of them that have tiles
    uint32_t *d_group_sinks;    // per group: its tiles without children
    uint32_t run_serial;    // number of the last dataflow run (never 0): what a group's host word holds once it has finished in that run
    int last_run_dataflow;  // the host words describe the last run
    int last_run_ordered;   // the last dataflow run took its tiles in index order (no ready queue)
    int prefer_ordered;     // -1: decided from the graph's parallelism; 0 / 1: the caller's choice, see aspen_hip_graph_set_ordered
    unsigned features;      // TILES_* bits of the tile kinds the graph contains: picks the persistent kernel's variant
    int variant;            // index into dataflow_kernels of the smallest variant that has all of them
    uint32_t epoch;         // tag of the last run's queue entries, cycles 1..EPOCH_MAX
    uint32_t queue_config;  // grid, flags and queue grouping of the last run (they decide which queue slots a run rewrites), see run_dataflow
    unsigned long long *d_prof;
    uint32_t default_workgroups;    // grid of a dataflow run when the caller names none, see graph_parallelism
    double parallelism;             // average parallelism of the tile graph, see graph_parallelism
    int cached_loads;       // 1: no cache line of an activation is shared by two producer tiles
    unsigned long long *d_trace;    // [2*tile] start, [2*tile+1] end time stamps (allocated on first traced run)
    uint32_t *h_abort;              // pinned host word the persistent kernel raises when it gives this graph's run up
};

static hipStream_t g_stream = nullptr;
static hipStream_t g_side_stream = nullptr;       // read-outs that must not queue behind a running persistent kernel
static hipEvent_t g_events[NUM_EVENTS];
static int g_inited = 0;
static int g_num_cu = 0;
static int g_resident_wg = WG_PER_CU;     // workgroups of the dataflow kernel's largest variant that fit one compute unit
static int g_variant_wg[8][2];            // the same per variant of the kernel ([variant][coherent / cached loads]), see dataflow_kernels
static char g_err[512] = "";
static uint32_t g_flags = 0;

static int fail (hipError_t e, const char *what)
{
    snprintf (g_err, sizeof (g_err), "%s: %s", what, hipGetErrorString (e));
    fprintf (stderr, "aspen_hip: %s\n", g_err);
    return (int)e;
}
#define CHECK(call) do { hipError_t e_ = (call); if (e_ != hipSuccess) return fail (e_, #call); } while (0)

// ------------------------------------------------------------------------------------------------
// kernels
// ------------------------------------------------------------------------------------------------

// Per-layer launch: workgroup -> tile with contiguous tile ranges per XCD (workgroups are dealt to
// the 8 XCDs round-robin), so tiles that share activation rows meet in the same L2.
__global__ void __launch_bounds__ (WG_THREADS, WG_PER_CU) layer_kernel (const aspen_hip_layer_t *layers, uint32_t l, uint32_t first_tile, uint32_t *arrivals)
{
    extern __shared__ __align__ (16) float smem[];
    const uint32_t nt = gridDim.x, bid = blockIdx.x;
    const uint32_t xcd = bid & 7, local = bid >> 3, chunk = nt >> 3, rem = nt & 7;
    const uint32_t t = first_tile + xcd * chunk + (xcd < rem ? xcd : rem) + local;
    bool more_rows;
    uint32_t row_rep = 0;
    do
    {
        more_rows = false;
        run_tile<0> ([=] () { return scalar_layer (layers + l); }, t, false, smem, [=] () { return arrivals; }, NoHook (), row_rep++, &more_rows);
    } while (more_rows);
}

// Second launch of a split-K layer in launch-per-layer mode: one workgroup per output tile adds the slices up.
__global__ void __launch_bounds__ (WG_THREADS, WG_PER_CU) finish_kernel (const aspen_hip_layer_t *layers, uint32_t l)
{
    extern __shared__ __align__ (16) float smem[];
    const aspen_hip_layer_t L = scalar_layer (layers + l);
    finish_tile<0> (L, blockIdx.x, smem);
}

// Re-arm: counters back to the parent counts, queues seeded with the roots.  A queue entry is 64 bits:
// tile [31:0], layer [47:32], the run's epoch [63:48] (a child record's entries carry the child's home queue in [55:48] instead).
// An entry left over from an earlier run does not match the current epoch, so a poll cannot mistake an old entry for
// a new one and a run does not clear the queues.  Which slots a run rewrites depends on its grid, its flags and the
// queue grouping (kept tiles never enter a queue), so a slot may keep an old entry over many runs: the host clears
// all queues whenever the epoch wraps around and whenever one of those settings differs from the graph's previous
// run (clear_queue_kernel), which is what makes "an old entry never matches" hold.  Carrying the layer saves the
// consumer a dependent lookup.  All writes are device-scope (write-through) stores, the same path the persistent
// kernel's polls and atomics use.
#define EPOCH_SHIFT 48
#define EPOCH_MAX 0xffffu
#define QUEUE_ID_BITS 24
#define QUEUE_ID_MASK ((1u << QUEUE_ID_BITS) - 1u)
#define MAX_GRAPH_LAYERS 65535u
__device__ __forceinline__ qentry_t make_entry (uint32_t epoch, uint32_t layer, uint32_t tile)
{
    return ((qentry_t)epoch << EPOCH_SHIFT) | ((qentry_t)layer << 32) | tile;
}
// Ticket t of a queue lives in that queue's entry (t % QUEUE_LANES) * row + t / QUEUE_LANES, row >= QUEUE_MIN_ROW
// entries: the workgroups that wait hold consecutive tickets and each polls its entry, so neighbouring tickets
// are placed at least 4 KiB apart and the polls spread over all memory channels instead of
// hammering the one or two that would hold a dense array's next few lines.  Queue q starts QUEUE_LANES * row entries
// behind queue q - 1.
#define QUEUE_LANES 128u
#define QUEUE_MIN_ROW 512u
#define QUEUE_SLACK 8192u       // tickets beyond a queue's tiles: one "leave" entry per workgroup that may still wait
__device__ __forceinline__ size_t queue_slot (uint32_t q, uint32_t ticket, uint32_t row)
{
    return ((size_t)q * QUEUE_LANES + ticket % QUEUE_LANES) * row + ticket / QUEUE_LANES;
}
static uint32_t queue_row (uint32_t capacity)
{
    const uint32_t r = (capacity + QUEUE_LANES) / QUEUE_LANES;
    return r < QUEUE_MIN_ROW ? QUEUE_MIN_ROW : r;
}

struct queue_counts_t { uint32_t n[NUM_QUEUES]; };

// Where tile id's dependency counter lives.  stride = 0: dep[id] (the counters of a layer's tiles share cache lines, which
// is what the countdowns of a full device like best).  Ordered mode gives every counter a 128-byte line of its own and
// puts neighbouring tiles' counters `stride` words (at least 4 KiB) apart: there a workgroup POLLS its tile's counter
// while the tile's parents count it down, and the polls of a level's hundreds of tiles would otherwise all land on
// the two or three memory channels that hold the level's lines, in front of the very countdowns they wait for.
__host__ __device__ __forceinline__ size_t dep_slot (uint32_t id, uint32_t stride)
{
    return stride ? (size_t)(id & 31u) * stride + (size_t)(id >> 5) * 32u : (size_t)id;
}

// every entry of every queue back to "no run's" (epoch 0), see make_entry
__global__ void clear_queue_kernel (qentry_t *queue, size_t entries)
{
    const size_t step = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < entries; i += step)
        __hip_atomic_store (&queue[i], (qentry_t)0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// nq_mask = number of queues in use - 1 (7 or 0); root_pos / counts describe the 8-queue seeding
__global__ void arm_kernel (uint32_t *dep, const uint32_t *num_parents, qentry_t *queue, uint32_t *ran,
    const uint32_t *roots, const uint32_t *ninst_layer, const uint32_t *ninst_home, const uint32_t *root_pos, queue_counts_t counts,
    uint32_t num_ninst, uint32_t num_roots, uint32_t *state, uint32_t epoch, uint32_t qrow, uint32_t nq_mask, uint32_t nq_shift,
    uint32_t *arrivals, uint32_t dep_stride)
{
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < num_ninst)
    {
        __hip_atomic_store (&dep[dep_slot (i, dep_stride)], num_parents[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (i < num_roots)
        {
            const uint32_t r = roots[i], q = (ninst_home[r] >> nq_shift) & nq_mask, pos = nq_mask ? root_pos[i] : i;
            __hip_atomic_store (&queue[queue_slot (q, pos, qrow)], make_entry (epoch, ninst_layer[r], r), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        __hip_atomic_store (&ran[i], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store (&arrivals[i], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    if (i < NUM_QUEUES)
    {
        __hip_atomic_store (&state[ST_QHEAD (i)], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store (&state[ST_QTAIL (i)], nq_mask ? counts.n[i] : (i == 0 ? num_roots : 0u), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    if (i == 0)
    {
        __hip_atomic_store (&state[ST_DONE], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store (&state[ST_ABORT], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store (&state[ST_TWICE], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store (&state[ST_SINKS], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    if (i < MAX_GROUPS) __hip_atomic_store (&state[ST_GROUP (i)], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

struct dataflow_args_t
{
    const aspen_hip_layer_t *layers;
    const uint32_t *ninst_layer, *ninst_home, *child_off, *child_idx;
    const qentry_t *child_rec;      // [num_ninst][CHILD_REC]: [0] = number of children | the tile's group << 32, then the first CHILD_REC-1 as (home << 48 | layer << 32 | tile)
    qentry_t *queue;
    uint32_t *dep, *state, *ran;
    uint32_t *arrivals;             // per split-K group (at its first tile's index): slices that have finished, see run_tile
    uint32_t *host_abort;           // pinned host block, see HOST_DONE_WORD
    const uint32_t *group_sinks;    // per co-scheduled network: its tiles without children
    uint32_t num_groups, run_serial;
    uint32_t dep_stride;            // ordered mode: see dep_slot (0: counters packed)
    const uint32_t *num_parents;    // ordered mode: what a tile's counter is set back to once the tile has seen it reach zero
    unsigned long long *trace;      // per-tile start / end time stamps when ASPEN_HIP_FLAG_TRACE is set
    unsigned long long *prof;       // 8 counters of summed 100 MHz ticks, see aspen_hip_dataflow_profile
    uint32_t num_ninst;
    uint32_t num_sinks;             // tiles without children: when all of them have finished, so has every tile
    uint32_t epoch;                 // 1..EPOCH_MAX, tag of this run's queue entries
    uint32_t flags;                 // ASPEN_HIP_FLAG_*
    uint32_t queue_row;             // see queue_slot
    uint32_t queue_cap;             // tickets a queue can hold
    uint32_t nq_mask;               // queues in use - 1: NUM_QUEUES - 1, or 0 when the grid is not a multiple of NUM_QUEUES
    uint32_t nq_shift;              // XCDs per queue, as a power of two
    unsigned long long spin_limit;
};

#define CHILD_REC 64     // entries per child record: one per lane of the publishing wavefront
#define QENTRY_EMPTY (~(qentry_t)0)

// Waits until queue slot `ticket` holds an entry of this run and returns it; QENTRY_EMPTY when all tickets
// are taken or the run was aborted.  An entry whose tile is QUEUE_EMPTY tells the workgroup to leave: the
// workgroup that finishes the run's last tile writes it to the slots that will never be served, see
// schedule_step.  The wait polls with relaxed device-scope loads (an
// acquire here would invalidate this XCD's L2 on every poll).
__device__ __forceinline__ qentry_t wait_for_slot (const dataflow_args_t &a, uint32_t q, uint32_t ticket)
{
    if (ticket >= a.queue_cap) return QENTRY_EMPTY;
    unsigned long long spins = 0;
    for (;;)
    {
        const qentry_t e = __hip_atomic_load (&a.queue[queue_slot (q, ticket, a.queue_row)], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if ((uint32_t)(e >> EPOCH_SHIFT) == a.epoch) return e;
        ++spins;
        if ((spins & 63) == 0 && __hip_atomic_load (&a.state[ST_ABORT], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0) return QENTRY_EMPTY;
        if (spins > a.spin_limit)
        {
            __hip_atomic_store (&a.state[ST_ABORT], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store (a.host_abort, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
            return QENTRY_EMPTY;
        }
        __builtin_amdgcn_s_sleep (2);
    }
}

// Workgroup-local scheduler state.  It lives in LDS so that nothing of it occupies registers while a
// tile runs: the tile code is inlined into the persistent loop and owns the whole register budget.
struct sched_lds_t
{
    dataflow_args_t a;
    uint32_t tile, layer;                // tile to run next (QUEUE_EMPTY: leave) and its layer
    uint32_t complete;                   // 0: the tile just run was a split-K slice that did not finish its group
    uint32_t may_keep;                   // the tile just run releases children, one of which this workgroup may run next
    uint32_t my_queue;                   // the ready queue this workgroup serves
    uint32_t next_ordered;               // ordered mode: the tile this workgroup takes next
    unsigned long long t0, ticks[6];     // profiling: last time stamp; tile / drain / scheduling / publish / ticket / slot-wait ticks
    unsigned long long p0, phase[5];     // profiling of contraction tiles: last phase stamp; set-up / K loop / epilogue / split-K ticks
};
__shared__ sched_lds_t s_sched;

__device__ __forceinline__ void prof_lap (int which)
{
    if ((s_sched.a.flags & ASPEN_HIP_FLAG_PROFILE) && threadIdx.x == 0)
    {
        const unsigned long long t = wall_clock64 ();
        s_sched.ticks[which] += t - s_sched.t0; s_sched.t0 = t;
    }
}

__device__ void tile_phase_lap (int which)
{
    if ((s_sched.a.flags & ASPEN_HIP_FLAG_PROFILE) && threadIdx.x == 0)
    {
        const unsigned long long t = wall_clock64 ();
        s_sched.phase[which - 8] += t - s_sched.p0; s_sched.p0 = t;
    }
    // traced runs also stamp a contraction tile's end of the K loop (9) and end of the epilogue's stores (10, 11)
    if ((s_sched.a.flags & ASPEN_HIP_FLAG_TRACE) && threadIdx.x == 0 && which >= 9 && which <= 11)
        s_sched.a.trace[2 * (size_t)s_sched.a.num_ninst + 2 * (size_t)s_sched.tile + (which == 9 ? 0 : 1)] = wall_clock64 ();
}

// Puts a tile that has become ready into the queue.
__device__ __forceinline__ void push_ready (const dataflow_args_t &a, uint32_t child, uint32_t layer, uint32_t home)
{
    const uint32_t q = (home >> a.nq_shift) & a.nq_mask, slot = atomicAdd (&a.state[ST_QTAIL (q)], 1u);
    __hip_atomic_store (&a.queue[queue_slot (q, slot, a.queue_row)], make_entry (a.epoch, layer, child), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// One scheduling step of a workgroup, as a real function call (it needs few registers, all of them
// caller-saved, so the call costs no register traffic).  done == QUEUE_EMPTY: nothing to publish (first
// step).  `rec` is this lane's entry of the finished tile's child record, fetched by wavefront 0 before the
// tile ran, so publishing starts with the atomics right away.  Returns the tile to run next; its layer is
// left in s_sched.layer.
//
// Publish: one child per lane of wavefront 0, a relaxed device-scope countdown of the child's counter.  The
// FIRST child whose counter this brings to zero is kept: it is this workgroup's next tile, with no trip
// through the queue (the reference's depth-first hand-off: the thread that completes a ninst's last parent
// runs that ninst next and pushes only the others it made ready, src/dse.c:363-401).  It saves the two
// atomic round trips and the poll of a pop on the chain parent -> child, and the child finds its parent's
// output in this XCD's L2.  Only a workgroup that kept nothing draws a ticket and waits for its queue slot.
// A tile that cannot release anything (no children, or a split-K slice that was not the last of its group)
// pops while it is being accounted, as before.
// Kept tiles never enter the queue, so fewer than num_ninst tickets are ever served.  Tiles without children
// count themselves when they finish; the last of them (then every tile has finished, for every tile has a
// descendant without children) writes a leave entry into the next gridDim.x slots behind the tail: every
// workgroup holds at most one ticket, so these are all the slots anyone can still be waiting for.
// The pop half of a scheduling step, run by one wavefront: draws a ticket and waits for its slot.
// kept != QUEUE_EMPTY: the tile to run is already known.
template <bool ORDERED>
__device__ __forceinline__ void pop_next (const dataflow_args_t &a, uint32_t lane, uint32_t kept, uint32_t kept_layer, bool prof)
{
    if (lane == 0)
    {
        if (kept != QUEUE_EMPTY) { s_sched.tile = kept; s_sched.layer = kept_layer; }
        else if (ORDERED)
        {
            // ordered mode: workgroup b runs tiles b, b + grid, b + 2 grid, ... (tiles are numbered parents first); whether
            // a tile is ready is found out by the tile itself, see wait_until_ready.  A fixed assignment, no ticket
            // counter: with a grid of two workgroups per compute unit the two tiles a compute unit holds are a grid
            // apart, i.e. in neighbouring dependency levels, so one of them computes while the other is being
            // prepared, and no two tiles of one level share a matrix pipeline while other units idle.  (Every workgroup
            // of the grid must be resident: the host clamps the grid to what fits.)
            const uint32_t ticket = s_sched.next_ordered;
            s_sched.next_ordered = ticket + gridDim.x;
            const bool live = ticket < a.num_ninst && __hip_atomic_load (&a.state[ST_ABORT], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == 0;
            s_sched.tile = live ? ticket : QUEUE_EMPTY;
            s_sched.layer = live ? a.ninst_layer[ticket] : 0u;
        }
        else
        {
            // a ticket is drawn only now, when this workgroup is free.  Drawing it earlier would hide the
            // atomic's round trip but binds a (possibly already ready) tile to a busy workgroup while idle
            // ones wait on later slots.
            const unsigned long long t1 = prof ? wall_clock64 () : 0;
            const uint32_t q = s_sched.my_queue, ticket = atomicAdd (&a.state[ST_QHEAD (q)], 1u);
            const unsigned long long t2 = prof ? wall_clock64 () : 0;
            const qentry_t e = wait_for_slot (a, q, ticket);
            s_sched.tile = e == QENTRY_EMPTY ? QUEUE_EMPTY : (uint32_t)e;
            s_sched.layer = (uint32_t)(e >> 32) & 0xffffu;
            if (prof) { s_sched.ticks[4] += t2 - t1; s_sched.ticks[5] += wall_clock64 () - t2; }
        }
    }
}

template <bool ORDERED>
__device__ __noinline__ uint32_t schedule_step (uint32_t done, qentry_t rec)
{
    const dataflow_args_t &a = s_sched.a;
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (done != QUEUE_EMPTY)
    {
        prof_lap (0);
        // a tile that releases children may keep one of them: then the pop waits for the outcome of the
        // countdown; otherwise wavefront 1 pops while wavefront 0 does the accounting
        if (threadIdx.x == 0)
            s_sched.may_keep = !ORDERED && s_sched.complete && (uint32_t)rec != 0u && !(a.flags & ASPEN_HIP_FLAG_NO_HANDOFF);
        // every wave waits until its (write-through, device-coherent) stores have been acknowledged.
        // An explicit wait: a workgroup-scope fence does not have to wait for global stores.
        asm volatile ("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads ();
        prof_lap (1);
        if ((a.flags & ASPEN_HIP_FLAG_TRACE) && threadIdx.x == 0) a.trace[2 * (size_t)done + 1] = wall_clock64 ();
    }
    const bool prof = (a.flags & ASPEN_HIP_FLAG_PROFILE) && lane == 0;
    const bool may_keep = done != QUEUE_EMPTY && __builtin_amdgcn_readfirstlane (s_sched.may_keep) != 0u;
    if (wave == 0 && done != QUEUE_EMPTY)
    {
        const unsigned long long tp = prof ? wall_clock64 () : 0;
        uint32_t kept = QUEUE_EMPTY, kept_layer = 0;
        // a split-K slice that was not the last of its group leaves the children to the one that is
        const uint32_t listed = (uint32_t)__shfl (rec, 0, 64), count = s_sched.complete ? listed : 0u;
        const uint32_t child = (uint32_t)rec, layer = (uint32_t)(rec >> 32) & 0xffffu, home = (uint32_t)(rec >> 48) & 0xffu;
        bool ready = false;
        if (lane >= 1 && lane <= count)
            ready = __hip_atomic_fetch_sub (&a.dep[dep_slot (child, ORDERED ? a.dep_stride : 0u)], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == 1u;
        if (may_keep)
        {
            // only a child at home in this workgroup's queue is kept
            const unsigned long long made_ready = __ballot (ready && ((home >> a.nq_shift) & a.nq_mask) == s_sched.my_queue);
            if (made_ready)
            {
                const int keeper = __builtin_ctzll (made_ready);
                kept = (uint32_t)__shfl (child, keeper, 64);
                kept_layer = (uint32_t)__shfl (layer, keeper, 64);
                ready = ready && (int)lane != keeper;
            }
        }
        if (ready && !ORDERED) push_ready (a, child, layer, home);
        if (count > CHILD_REC - 1)
        {
            // more children than the record holds: the rest comes from the CSR lists and goes through the queue
            const uint32_t c0 = a.child_off[done] + (CHILD_REC - 1), c1 = a.child_off[done + 1];
            for (uint32_t c = c0 + lane; c < c1; c += 64)
            {
                const uint32_t ch = a.child_idx[c];
                if (__hip_atomic_fetch_sub (&a.dep[dep_slot (ch, ORDERED ? a.dep_stride : 0u)], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == 1u && !ORDERED) push_ready (a, ch, a.ninst_layer[ch], a.ninst_home[ch]);
            }
        }
        if (listed == 0u)
        {
            // a tile without children (no hand-off, so wavefront 1 is popping meanwhile): was it the run's last?
            // Its network's last?  Then that network is complete (every tile has a descendant without children, and this
            // tile's stores were acknowledged above): the host word of the network is raised, the counterpart of the
            // reference's per-nasm completion signal (src/dse.c:94-105).  The network that completes last ends the run.
            uint32_t last = 0;
            if (lane == 0)
            {
                const uint32_t grp = (uint32_t)(rec >> 32);
                if (__hip_atomic_fetch_add (&a.state[ST_GROUP (grp)], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + 1u == a.group_sinks[grp])
                {
                    __hip_atomic_store (a.host_abort + HOST_DONE_WORD + grp, a.run_serial, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
                    last = __hip_atomic_fetch_add (&a.state[ST_SINKS], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + 1u == a.num_groups;
                    if (ORDERED)
                    {
                        // (these counters too are back at their start for the next ordered run: nobody adds to them any more)
                        __hip_atomic_store (&a.state[ST_GROUP (grp)], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        if (last) __hip_atomic_store (&a.state[ST_SINKS], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    }
                }
            }
            if (__shfl (last, 0, 64) && !ORDERED)
            {
                // the run is over and nothing will be pushed any more: tell everyone who waits, this workgroup's
                // own popping wavefront included
                for (uint32_t q = 0; q <= a.nq_mask; q++)
                {
                    const uint32_t tail = __hip_atomic_load (&a.state[ST_QTAIL (q)], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    for (uint32_t t = tail + lane; t < tail + gridDim.x && t < a.queue_cap; t += 64)
                        __hip_atomic_store (&a.queue[queue_slot (q, t, a.queue_row)], make_entry (a.epoch, 0, QUEUE_EMPTY), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
            }
        }
        if (lane == 0 && (a.flags & ASPEN_HIP_FLAG_COUNT_TILES))
        {
            if (atomicAdd (&a.ran[done], 1u) != 0) atomicAdd (&a.state[ST_TWICE], 1u);
            atomicAdd (&a.state[ST_DONE], 1u);
        }
        if (prof) s_sched.ticks[3] += wall_clock64 () - tp;
        if (may_keep) pop_next<ORDERED> (a, lane, kept, kept_layer, prof);
    }
    else if (wave == 1 && !may_keep) pop_next<ORDERED> (a, lane, QUEUE_EMPTY, 0, prof);
    __syncthreads ();
    const uint32_t next = s_sched.tile;
    prof_lap (2);
    return next;
}

// Persistent workgroup = one scheduling engine (the reference's DSE thread, src/dse.c:5-108).
// No cache write-back / invalidate is needed anywhere: tiles store activations with device-scope
// write-through instructions and load them either coherently (COH = 1) or, when the host has checked
// that no cache line is shared between producer tiles, through the caches (COH = 2); see ActView.
// Ordered mode: waits until every parent of the tile this workgroup holds has finished (its dependency counter has
// been counted down to zero).  Called from inside the tile, after the set-up that needs no activation.  Every
// wavefront polls for itself (one request per poll, the word is the same for all lanes); a wait that exceeds the
// run's spin limit gives the run up like a wait on a queue slot does: the tile then runs on whatever its parents have
// written so far, inside its own buffers, and the next scheduling step ends the workgroup.
__device__ __forceinline__ void wait_until_ready ()
{
    const dataflow_args_t &a = s_sched.a;
    const uint32_t id = __builtin_amdgcn_readfirstlane (s_sched.tile);
    // one wavefront polls, the others wait at the barrier: every poll is a trip to memory, and a thousand wavefronts
    // polling at once slow down the very countdowns they are waiting for
    if (threadIdx.x < 64)
    {
        unsigned long long spins = 0;
        uint32_t *counter = &a.dep[dep_slot (id, a.dep_stride)];
        const uint32_t parents = a.num_parents[id];     // (requested before the wait)
        bool seen_zero = true;
        while (__builtin_amdgcn_readfirstlane (__hip_atomic_load (counter, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) != 0u)
        {
            ++spins;
            if ((spins & 63) == 0 && __hip_atomic_load (&a.state[ST_ABORT], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0) { seen_zero = false; break; }
            if (spins > a.spin_limit)
            {
                __hip_atomic_store (&a.state[ST_ABORT], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                __hip_atomic_store (a.host_abort, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
                seen_zero = false;
                break;
            }
            __builtin_amdgcn_s_sleep (1);
        }
        // The counter has done its work for this run (every parent has counted down): it is set back right away, so
        // that the next ordered run of the graph needs no arming pass in front of it.
        if (seen_zero && threadIdx.x == 0) __hip_atomic_store (counter, parents, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads ();
    if ((a.flags & ASPEN_HIP_FLAG_TRACE) && threadIdx.x == 0) a.trace[2 * (size_t)id] = wall_clock64 ();      // a tile "starts" when it may touch its operands
    if ((a.flags & ASPEN_HIP_FLAG_PROFILE) && threadIdx.x == 0) { const unsigned long long t = wall_clock64 (); s_sched.ticks[5] += t - s_sched.p0; s_sched.p0 = t; }
}

template <int COH, unsigned FEAT, bool ORDERED = false>
// (The variant for transformer graphs is built for three workgroups per compute unit instead of four: those graphs never
// fill the device (256 to 768 workgroups), and 168 instead of 128 registers per lane spare their attention and matmul loops
// the spills the tighter budget forces.)
#define DATAFLOW_WG_PER_CU(feat, ordered) ((feat) == TILES_TRANSFORMER ? WG_PER_CU - 1 : WG_PER_CU)
__global__ void __launch_bounds__ (WG_THREADS, DATAFLOW_WG_PER_CU (FEAT, ORDERED)) dataflow_kernel (dataflow_args_t args)
{
    extern __shared__ __align__ (16) float smem[];
    if (threadIdx.x == 0)
    {
        s_sched.a = args;
        s_sched.t0 = wall_clock64 ();
        for (int i = 0; i < 6; i++) s_sched.ticks[i] = 0;
        for (int i = 0; i < 5; i++) s_sched.phase[i] = 0;
        s_sched.may_keep = 0;
        s_sched.my_queue = ((blockIdx.x & (NUM_QUEUES - 1u)) >> args.nq_shift) & args.nq_mask;
        s_sched.next_ordered = blockIdx.x;
    }
    __syncthreads ();
    __builtin_amdgcn_s_setprio (TILE_PRIO);
    const unsigned long long t_begin = wall_clock64 (), c_begin = clock64 ();
    uint32_t id = QUEUE_EMPTY;
    uint32_t row_rep = 0;           // which row tile of a row group comes next (see run_tile); 0: a new tile
    qentry_t rec = 0;
    for (;;)
    {
        if (row_rep == 0)
        {
            id = __builtin_amdgcn_readfirstlane (schedule_step<ORDERED> (id, rec));
            if (id == QUEUE_EMPTY) break;           // all tickets taken, or aborted
            // wavefront 0 requests this tile's child record now; it arrives while the tile runs
            // (a global, not a flat load: a flat one would also count as LDS traffic the tile's first fragment wait sits out)
            if (threadIdx.x < CHILD_REC)
                rec = *(const qentry_t __attribute__ ((address_space (1))) *)(s_sched.a.child_rec + (size_t)id * CHILD_REC + threadIdx.x);
            if ((s_sched.a.flags & ASPEN_HIP_FLAG_TRACE) && threadIdx.x == 0) s_sched.a.trace[2 * (size_t)id] = wall_clock64 ();
            if ((s_sched.a.flags & ASPEN_HIP_FLAG_PROFILE) && threadIdx.x == 0) s_sched.p0 = wall_clock64 ();
        }
        // the layer's descriptor goes from memory into scalar registers (it is shared by all tiles of the layer
        // and by all workgroups, so it sits in the scalar cache or in L2)
        const auto descriptor = [] () { return scalar_layer (s_sched.a.layers + s_sched.layer); };
        bool complete, more_rows = false;
        const auto ready = [] () { if constexpr (ORDERED) wait_until_ready (); };
        if (!(s_sched.a.flags & ASPEN_HIP_FLAG_SKIP_TILES))
            complete = run_tile<COH, FEAT, ORDERED ? NARROW_PF_SLICES : 0> (descriptor, id, true, smem, [] () { return s_sched.a.arrivals; }, ready, row_rep, &more_rows);
        else
        {
            // scheduler-only run: the split-K groups still elect the member that releases the children
            ready ();
            const aspen_hip_layer_t L = descriptor ();
            const uint32_t t = id - L.ninst_start;
            complete = L.splits <= 1 || splitk_arrived_last (&s_sched.a.arrivals[id - t % L.splits], L.splits, smem);
        }
        row_rep = __builtin_amdgcn_readfirstlane (more_rows ? row_rep + 1u : 0u);
        if (threadIdx.x == 0) s_sched.complete = complete;      // read by schedule_step behind its barrier
    }
    if ((s_sched.a.flags & ASPEN_HIP_FLAG_PROFILE) && threadIdx.x == 0)
    {
        unsigned long long *prof = s_sched.a.prof;
        atomicAdd (&prof[0], s_sched.ticks[0]); atomicAdd (&prof[1], s_sched.ticks[1]); atomicAdd (&prof[2], s_sched.ticks[2]);
        atomicAdd (&prof[3], wall_clock64 () - t_begin);
        atomicAdd (&prof[4], s_sched.ticks[3]); atomicAdd (&prof[5], s_sched.ticks[4]); atomicAdd (&prof[6], s_sched.ticks[5]);
        for (int i = 0; i < 5; i++) atomicAdd (&prof[8 + i], s_sched.phase[i]);
        atomicAdd (&prof[7], (unsigned long long)(clock64 () - c_begin));     // engine clock cycles: [7] / [3] * 100 MHz = the clock the run had
    }
}

__global__ void sgemm_kernel (const aspen_hip_layer_t L);       // defined with aspen_hip_sgemm_static

// The persistent kernel's variants, smallest first: [variant][0] coherent loads, [1] cached loads.  A graph runs on the
// first variant that has all its tile kinds, see graph_features.
#define NUM_KERNEL_VARIANTS 5
static const unsigned kernel_variant_tiles[NUM_KERNEL_VARIANTS] = {TILES_TRANSFORMER, TILES_CONVNET, TILES_CONVNET | TILES_TALL, TILES_CONVNET | TILES_YOLO, TILES_ALL};
static const void *const dataflow_kernels[NUM_KERNEL_VARIANTS][2] = {
    {(const void *)dataflow_kernel<1, TILES_TRANSFORMER>, (const void *)dataflow_kernel<2, TILES_TRANSFORMER>},
    {(const void *)dataflow_kernel<1, TILES_CONVNET>, (const void *)dataflow_kernel<2, TILES_CONVNET>},
    {(const void *)dataflow_kernel<1, TILES_CONVNET | TILES_TALL>, (const void *)dataflow_kernel<2, TILES_CONVNET | TILES_TALL>},
    {(const void *)dataflow_kernel<1, TILES_CONVNET | TILES_YOLO>, (const void *)dataflow_kernel<2, TILES_CONVNET | TILES_YOLO>},
    {(const void *)dataflow_kernel<1, TILES_ALL>, (const void *)dataflow_kernel<2, TILES_ALL>}};

// Ordered mode (see aspen_hip_run_dataflow), cached loads only: for convolutional networks, for those with weight-streaming
// layers (VGG-16 at small batches), for transformer graphs, and with every tile kind.
#define NUM_ORDERED_VARIANTS 4
#define ORDERED_SMEM_BYTES CMAX (GEMM_SMEM_BYTES, NARROW_PF_SMEM_BYTES)       // the narrow tiles' weight prefetch buffers
static const unsigned ordered_variant_tiles[NUM_ORDERED_VARIANTS] = {TILES_CONVNET | TILES_YOLO | TILES_NARROW, TILES_CONVNET | TILES_TALL, TILES_TRANSFORMER, TILES_ALL};
static const void *const ordered_kernels[NUM_ORDERED_VARIANTS] = {
    (const void *)dataflow_kernel<2, TILES_CONVNET | TILES_YOLO | TILES_NARROW, true>, (const void *)dataflow_kernel<2, TILES_CONVNET | TILES_TALL, true>,
    (const void *)dataflow_kernel<2, TILES_TRANSFORMER, true>, (const void *)dataflow_kernel<2, TILES_ALL, true>};

// The tile kinds a graph contains, as TILES_* bits.
static unsigned graph_features (const aspen_hip_layer_t *layers, uint32_t num_layers)
{
    unsigned f = 0;
    for (uint32_t l = 0; l < num_layers; l++)
    {
        const aspen_hip_layer_t &L = layers[l];
        if (L.type == INPUT_LAYER || L.num_ninst == 0) continue;
        switch (L.type)
        {
        case CONV_LAYER: case FC_LAYER: case MATMUL_LAYER:
            if (L.variant == ASPEN_HIP_GEMM_NARROW) { f |= TILES_NARROW; break; }      // (brings its own operand loaders)
            f |= L.variant == ASPEN_HIP_GEMM_LARGE ? TILES_LARGE : L.variant == ASPEN_HIP_GEMM_WIDE ? TILES_WIDE : L.variant == ASPEN_HIP_GEMM_TALL ? TILES_TALL : TILES_SMALL;
            if (L.direct != ASPEN_HIP_OPERAND_DIRECT) f |= TILES_GATHER;
            break;
        case K_ATTENTION_LAYER: case V_ATTENTION_LAYER: f |= TILES_ATTENTION; break;
        case LAYERNORM_LAYER: case SOFTMAX_LAYER: f |= TILES_NORM; break;
        case MAXPOOL_LAYER: case AVGPOOL_LAYER: f |= TILES_POOL; break;
        case YOLO_LAYER: case APPEND_LAYER: f |= TILES_YOLO; break;
        case RESIDUAL_LAYER: f |= TILES_RESIDUAL; break;
        default: f |= TILES_ALL; break;
        }
    }
    return f;
}

// ------------------------------------------------------------------------------------------------
// device, memory
// ------------------------------------------------------------------------------------------------
extern "C" int aspen_hip_init (void)
{
    if (g_inited) return 0;
    int count = 0;
    CHECK (hipGetDeviceCount (&count));
    if (count < 1) { snprintf (g_err, sizeof (g_err), "no HIP device"); return -1; }
    CHECK (hipSetDevice (0));
    hipDeviceProp_t prop;
    CHECK (hipGetDeviceProperties (&prop, 0));
    g_num_cu = prop.multiProcessorCount;
    CHECK (hipStreamCreate (&g_stream));
    CHECK (hipStreamCreate (&g_side_stream));
    for (int i = 0; i < NUM_EVENTS; i++) CHECK (hipEventCreate (&g_events[i]));
    CHECK (hipFuncSetAttribute ((const void *)layer_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, GEMM_SMEM_BYTES));
    CHECK (hipFuncSetAttribute ((const void *)sgemm_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, GEMM_SMEM_BYTES));
    for (int v = 0; v < NUM_KERNEL_VARIANTS; v++)
        for (int coh = 0; coh < 2; coh++)
            CHECK (hipFuncSetAttribute (dataflow_kernels[v][coh], hipFuncAttributeMaxDynamicSharedMemorySize, GEMM_SMEM_BYTES));
    for (int v = 0; v < NUM_ORDERED_VARIANTS; v++)
        CHECK (hipFuncSetAttribute (ordered_kernels[v], hipFuncAttributeMaxDynamicSharedMemorySize, ORDERED_SMEM_BYTES));
    // how many persistent workgroups really fit a compute unit (registers, LDS), per variant: a graph's default grid
    // follows the variant it runs on
    g_resident_wg = WG_PER_CU;
    for (int v = 0; v < NUM_KERNEL_VARIANTS; v++)
        for (int coh = 0; coh < 2; coh++)
        {
            int occ = 0;
            CHECK (hipOccupancyMaxActiveBlocksPerMultiprocessor (&occ, dataflow_kernels[v][coh], WG_THREADS, GEMM_SMEM_BYTES));
            g_variant_wg[v][coh] = occ < 1 ? 1 : occ;
            if (g_variant_wg[v][coh] < g_resident_wg) g_resident_wg = g_variant_wg[v][coh];
        }
    if (getenv ("ASPEN_GPU_VERBOSE")) fprintf (stderr, "aspen_hip: %d resident dataflow workgroups per compute unit (built for %d)\n", g_resident_wg, WG_PER_CU);
    g_inited = 1;
    return 0;
}

extern "C" const char *aspen_hip_last_error (void) { return g_err; }

extern "C" void aspen_hip_tile_shapes (uint32_t shapes[13])
{
    shapes[11] = VAR4_BM; shapes[12] = VAR4_BN;
    shapes[0] = VAR0_BM; shapes[1] = VAR0_BN; shapes[2] = VAR1_BM; shapes[3] = VAR1_BN; shapes[4] = VAR2_BM; shapes[5] = VAR2_BN;
    shapes[6] = KATTN_BN; shapes[7] = VATTN_BN; shapes[8] = WG_PER_CU; shapes[9] = VAR3_BM; shapes[10] = VAR3_BN;
}

extern "C" int aspen_hip_device_info (int *num_cu, int *clock_khz, size_t *mem_bytes, char *name, int name_len)
{
    if (aspen_hip_init ()) return -1;
    hipDeviceProp_t prop;
    CHECK (hipGetDeviceProperties (&prop, 0));
    if (num_cu) *num_cu = prop.multiProcessorCount;
    if (clock_khz) *clock_khz = prop.clockRate;
    if (mem_bytes) *mem_bytes = prop.totalGlobalMem;
    if (name && name_len > 0)
    {
        // some driver stacks leave the marketing name empty: fall back to the architecture name
        strncpy (name, prop.name[0] ? prop.name : prop.gcnArchName, name_len - 1);
        name[name_len - 1] = 0;
    }
    return 0;
}

extern "C" void *aspen_hip_alloc (size_t bytes)
{
    if (aspen_hip_init ()) return nullptr;
    void *p = nullptr;
    if (bytes == 0) bytes = 256;
    hipError_t e = hipMalloc (&p, bytes + 256);      // slack: edge tiles may read (never write) a few floats past a row
    if (e != hipSuccess) { fail (e, "hipMalloc"); return nullptr; }
    e = hipMemsetAsync (p, 0, bytes + 256, g_stream);
    if (e == hipSuccess) e = hipStreamSynchronize (g_stream);
    if (e != hipSuccess) { fail (e, "hipMemset"); (void)hipFree (p); return nullptr; }
    return p;
}

extern "C" void aspen_hip_free (void *ptr) { if (ptr) (void)hipFree (ptr); }

extern "C" int aspen_hip_h2d (void *dst, const void *src, size_t bytes)
{
    if (aspen_hip_init ()) return -1;
    CHECK (hipMemcpyAsync (dst, src, bytes, hipMemcpyHostToDevice, g_stream));
    CHECK (hipStreamSynchronize (g_stream));
    return 0;
}
extern "C" int aspen_hip_d2h (void *dst, const void *src, size_t bytes)
{
    if (aspen_hip_init ()) return -1;
    CHECK (hipMemcpyAsync (dst, src, bytes, hipMemcpyDeviceToHost, g_stream));
    CHECK (hipStreamSynchronize (g_stream));
    return 0;
}
extern "C" int aspen_hip_h2d_2d (void *dst, size_t dpitch, const void *src, size_t spitch, size_t width, size_t rows)
{
    if (aspen_hip_init ()) return -1;
    CHECK (hipMemcpy2DAsync (dst, dpitch, src, spitch, width, rows, hipMemcpyHostToDevice, g_stream));
    CHECK (hipStreamSynchronize (g_stream));
    return 0;
}
extern "C" int aspen_hip_d2h_2d (void *dst, size_t dpitch, const void *src, size_t spitch, size_t width, size_t rows)
{
    if (aspen_hip_init ()) return -1;
    CHECK (hipMemcpy2DAsync (dst, dpitch, src, spitch, width, rows, hipMemcpyDeviceToHost, g_stream));
    CHECK (hipStreamSynchronize (g_stream));
    return 0;
}
extern "C" int aspen_hip_zero (void *dst, size_t bytes)
{
    if (aspen_hip_init ()) return -1;
    CHECK (hipMemsetAsync (dst, 0, bytes, g_stream));
    return 0;
}

// Dense <-> strided columns.  dense[c * rows + r] <-> strided[c * ld + r]; padding rows [rows, ld) are written as zeros.
__global__ void __launch_bounds__ (WG_THREADS) spread_columns_kernel (const float *__restrict__ dense, float *__restrict__ strided, uint32_t rows, uint32_t ld, size_t n)
{
    const size_t step = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += step)
    {
        const size_t c = i / ld;
        const uint32_t r = (uint32_t)(i - c * ld);
        strided[i] = r < rows ? dense[c * rows + r] : 0.f;
    }
}
__global__ void __launch_bounds__ (WG_THREADS) gather_columns_kernel (const float *__restrict__ strided, float *__restrict__ dense, uint32_t rows, uint32_t ld, size_t n)
{
    const size_t step = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += step)
    {
        const size_t c = i / rows;
        dense[i] = strided[c * ld + (i - c * rows)];
    }
}

// staging buffer for the two functions below; grows on demand and lives as long as the process
static float *g_stage = nullptr;
static size_t g_stage_bytes = 0;
static int stage_reserve (size_t bytes)
{
    if (bytes <= g_stage_bytes) return 0;
    CHECK (hipStreamSynchronize (g_stream));
    if (g_stage) { (void)hipFree (g_stage); g_stage = nullptr; g_stage_bytes = 0; }
    CHECK (hipMalloc ((void **)&g_stage, bytes));
    g_stage_bytes = bytes;
    return 0;
}
static unsigned stream_grid (size_t n)
{
    const size_t want = (n + WG_THREADS - 1) / WG_THREADS, cap = (size_t)g_num_cu * 16;
    return (unsigned)(want < cap ? (want ? want : 1) : cap);
}

extern "C" int aspen_hip_dense_host_to_device (float *dst, uint32_t ld, const float *src_host, uint32_t rows, size_t columns)
{
    if (aspen_hip_init ()) return -1;
    if (!dst || !src_host || rows == 0 || ld < rows) { snprintf (g_err, sizeof (g_err), "dense_host_to_device: bad arguments"); return -1; }
    if (columns == 0) return 0;
    if (ld == rows) return aspen_hip_h2d (dst, src_host, (size_t)rows * columns * sizeof (float));
    const size_t bytes = (size_t)rows * columns * sizeof (float);
    if (stage_reserve (bytes)) return -1;
    CHECK (hipMemcpyAsync (g_stage, src_host, bytes, hipMemcpyHostToDevice, g_stream));
    const size_t n = (size_t)ld * columns;
    hipLaunchKernelGGL (spread_columns_kernel, dim3 (stream_grid (n)), dim3 (WG_THREADS), 0, g_stream, g_stage, dst, rows, ld, n);
    CHECK (hipGetLastError ());
    CHECK (hipStreamSynchronize (g_stream));       // the caller may reuse its buffer, and the next call the staging buffer
    return 0;
}

extern "C" int aspen_hip_dense_device_to_host (float *dst_host, const float *src, uint32_t ld, uint32_t rows, size_t columns)
{
    if (aspen_hip_init ()) return -1;
    if (!dst_host || !src || rows == 0 || ld < rows) { snprintf (g_err, sizeof (g_err), "dense_device_to_host: bad arguments"); return -1; }
    if (columns == 0) return 0;
    if (ld == rows) return aspen_hip_d2h (dst_host, src, (size_t)rows * columns * sizeof (float));
    const size_t bytes = (size_t)rows * columns * sizeof (float), n = (size_t)rows * columns;
    if (stage_reserve (bytes)) return -1;
    hipLaunchKernelGGL (gather_columns_kernel, dim3 (stream_grid (n)), dim3 (WG_THREADS), 0, g_stream, src, g_stage, rows, ld, n);
    CHECK (hipGetLastError ());
    CHECK (hipMemcpyAsync (dst_host, g_stage, bytes, hipMemcpyDeviceToHost, g_stream));
    CHECK (hipStreamSynchronize (g_stream));
    return 0;
}

// plain streaming copy; also the yardstick the HBM byte counters of a profiler are calibrated with (its traffic is
// known: `bytes` read + `bytes` written).  A workgroup moves contiguous pieces of COPY_UNROLL x 4 KB: every lane has
// COPY_UNROLL 16-byte loads in flight before its first store (one load per lane per step leaves the memory pipeline
// mostly empty: 4.5 of 8 TB/s against 5.7 this way), and the grid is what the device holds at once.
#define COPY_UNROLL 8
__global__ void __launch_bounds__ (WG_THREADS) copy_kernel (const float4 *__restrict__ src, float4 *__restrict__ dst, size_t n4)
{
    const size_t piece = (size_t)WG_THREADS * COPY_UNROLL, step = (size_t)gridDim.x * piece;
    const floatx4 *s4 = reinterpret_cast<const floatx4 *> (src);
    floatx4 *d4 = reinterpret_cast<floatx4 *> (dst);
    for (size_t base = (size_t)blockIdx.x * piece + threadIdx.x; base < n4; base += step)
    {
        floatx4 v[COPY_UNROLL];
        #pragma unroll
        for (int u = 0; u < COPY_UNROLL; u++) if (base + (size_t)u * WG_THREADS < n4) v[u] = __builtin_nontemporal_load (&s4[base + (size_t)u * WG_THREADS]);
        #pragma unroll
        for (int u = 0; u < COPY_UNROLL; u++) if (base + (size_t)u * WG_THREADS < n4) __builtin_nontemporal_store (v[u], &d4[base + (size_t)u * WG_THREADS]);
    }
}
extern "C" int aspen_hip_copy (void *dst, const void *src, size_t bytes)
{
    if (aspen_hip_init ()) return -1;
    if (bytes % 16 || ((uintptr_t)dst | (uintptr_t)src) % 16)
    { snprintf (g_err, sizeof (g_err), "copy: size and addresses must be multiples of 16 bytes"); return -1; }
    if (bytes == 0) return 0;
    const size_t n4 = bytes / 16, piece = (size_t)WG_THREADS * COPY_UNROLL;
    const size_t want = (n4 + piece - 1) / piece;
    static int per_cu = 0;
    if (per_cu == 0)
    {
        CHECK (hipOccupancyMaxActiveBlocksPerMultiprocessor (&per_cu, copy_kernel, WG_THREADS, 0));
        if (per_cu < 1) per_cu = 1;
    }
    const size_t cap = (size_t)g_num_cu * (size_t)per_cu;
    const unsigned grid = (unsigned)(want < cap ? want : cap);
    hipLaunchKernelGGL (copy_kernel, dim3 (grid), dim3 (WG_THREADS), 0, g_stream, (const float4 *)src, (float4 *)dst, n4);
    CHECK (hipGetLastError ());
    return 0;
}

// ------------------------------------------------------------------------------------------------
// graph
// ------------------------------------------------------------------------------------------------
// {multiplier, shift} for fast_div (tile_kernels.h): division by the invariant d in its branch-free round-up form
// (T. Granlund, P. Montgomery, "Division by invariant integers using multiplication", 1994).
static void divider_for (uint32_t d, uint32_t out[2])
{
    if (d <= 1) { out[0] = 0; out[1] = 0x80u; return; }
    uint32_t lg = 31;
    while (!(d >> lg)) lg--;                                 // floor (log2 (d))
    if ((d & (d - 1)) == 0) { out[0] = 0; out[1] = lg - 1; return; }
    const uint64_t two_k = (uint64_t)1 << (32 + lg);
    uint64_t m = two_k / d;
    const uint64_t rem = two_k - m * d;
    m *= 2;
    if (2 * rem >= d) m += 1;
    out[0] = (uint32_t)(m + 1);
    out[1] = lg;
}

// the values of a layer descriptor that aspen_hip_graph_create derives for the kernels
static void fill_derived (aspen_hip_layer_t &L)
{
    divider_for (L.OH * L.OW, L.div_ohw);
    divider_for (L.OW, L.div_ow);
    divider_for (L.tiles_m, L.div_tiles_m);
    divider_for (L.splits, L.div_splits);
    if (L.type == FC_LAYER) L.in0_columns = L.N * L.IH * L.IW;
    else if (L.type == CONV_LAYER && L.OH * L.OW != 0) L.in0_columns = (L.N / (L.OH * L.OW)) * L.IH * L.IW;
    else L.in0_columns = L.N;
}

extern "C" void aspen_hip_divider_for (uint32_t d, uint32_t out[2]) { divider_for (d, out); }

template <class T> static T *upload (const T *src, size_t n)
{
    T *d = (T *)aspen_hip_alloc ((n ? n : 1) * sizeof (T));
    if (d && n && aspen_hip_h2d (d, src, n * sizeof (T))) { aspen_hip_free (d); return nullptr; }
    return d;
}

static int check_layer (const aspen_hip_layer_t &L, uint32_t idx)
{
    const char *why = nullptr;
    // buffer descriptors carry 32-bit sizes: this holds for every matrix, also one no tile of its own layer writes
    if ((uint64_t)L.N * L.ld * 4 >= 0xffffff00ull
        || (L.splits > 1 && (uint64_t)L.splits * L.tiles_m * L.tiles_n * L.tile_m * L.tile_n * 4 >= 0xffffff00ull))
    {
        snprintf (g_err, sizeof (g_err), "layer %u rejected: matrix larger than 4 GiB", idx);
        fprintf (stderr, "aspen_hip: %s\n", g_err);
        return -1;
    }
    if (L.type == INPUT_LAYER || L.num_ninst == 0) return 0;     // no tiles: written by the host, or by another layer's epilogue
    if (!L.out || !L.in0) why = "missing buffers";
    else if (L.ld % 4 || L.ld0 % 4 || (L.in1 && L.ld1 % 4)) why = "strides must be multiples of 4 floats";
    else if (L.tiles_m == 0 || L.tiles_n == 0 || L.splits == 0
        || L.num_ninst != L.tiles_m * L.tiles_n * L.splits) why = "tile grid";
    else if (L.splits > 1 && (!L.partial || L.kiters_per_split == 0 || (uint64_t)L.splits * L.kiters_per_split * GEMM_BK < L.Kp
        || !(L.type == CONV_LAYER || L.type == FC_LAYER || L.type == MATMUL_LAYER) || (L.variant != ASPEN_HIP_GEMM_SMALL && L.variant != ASPEN_HIP_GEMM_NARROW && L.variant != ASPEN_HIP_GEMM_TALL))) why = "split-K geometry";
    else if ((L.type == CONV_LAYER || L.type == MAXPOOL_LAYER || L.type == AVGPOOL_LAYER)
        && (L.stride == 0 || L.KH == 0 || L.KW == 0 || L.IH == 0 || L.IW == 0 || L.OH == 0 || L.OW == 0 || L.N % (L.OH * L.OW))) why = "window geometry";
    else if (L.type == CONV_LAYER || L.type == FC_LAYER || L.type == MATMUL_LAYER)
    {
        uint32_t shp[13];
        aspen_hip_tile_shapes (shp);
        if (L.variant < 0 || L.variant >= ASPEN_HIP_NUM_GEMM_VARIANTS) { snprintf (g_err, sizeof (g_err), "layer %u rejected: GEMM variant", idx); return -1; }
        const bool narrow = L.variant == ASPEN_HIP_GEMM_NARROW, tall = L.variant == ASPEN_HIP_GEMM_TALL;
        const uint32_t bm = narrow ? shp[9] : tall ? shp[11] : shp[2 * L.variant], bn = narrow ? shp[10] : tall ? shp[12] : shp[2 * L.variant + 1];
        if (!L.weight) why = "missing weight";
        else if ((uint64_t)((L.M + 127) / 128 * 128) * L.Kp * 4 >= 0xffffff00ull) why = "weight matrix larger than 4 GiB";
        else if (L.Kp == 0 || L.Kp % GEMM_BK) why = "Kp must be a positive multiple of 32";
        else if (L.tile_n != bn || (L.tile_m != bm && !(L.variant == ASPEN_HIP_GEMM_LARGE && L.splits == 1 && (L.tile_m == 2 * bm || L.tile_m == 4 * bm))))
            why = "tile extent does not match the GEMM variant";         // (the large shape may cover two or four row tiles per workgroup)
        else if ((uint64_t)L.tiles_m * L.tile_m < L.M || (uint64_t)L.tiles_n * bn < L.N) why = "tile grid does not cover the matrix";
        else if (L.direct != ASPEN_HIP_OPERAND_DIRECT && !L.ktab) why = "missing k-chunk table";
        else if (L.fuse_out && (!L.fuse_in || L.fuse_ld_in % 4 || L.fuse_ld_in < L.M)) why = "fused shortcut operand";
        else if (L.direct == ASPEN_HIP_OPERAND_DIRECT && (L.ld0 < L.Kp)) why = "direct operand shorter than Kp";
        else if (L.fuse_norm_stats && (!L.fuse_out || !L.fuse_norm_gamma || L.variant != ASPEN_HIP_GEMM_SMALL || L.M % 64)) why = "a normalised shortcut operand needs a fused shortcut, the norm's scale, 64 x 64 tiles and whole groups of 64 channels";
        else if (L.norm_stats && !L.norm_fold) why = "column statistics are stored by a layer with a folded layer norm";
        else if (L.norm_fold && (L.type != MATMUL_LAYER || L.direct != ASPEN_HIP_OPERAND_DIRECT || L.variant != ASPEN_HIP_GEMM_SMALL || L.splits > 1 || !L.in1 || L.K % GEMM_BK)) why = "a folded layer norm needs a direct operand, 64 x 64 tiles and an uncut K axis";
        else if (L.direct == ASPEN_HIP_OPERAND_DENSE3 && (L.IC != 3 || L.Kp > 512 || L.Kp < 3 * L.KH * L.KW || L.ld0 < 4 || bm != 64)) why = "dense three-channel operand";
        else if (L.direct < 0 || L.direct > ASPEN_HIP_OPERAND_DENSE3) why = "operand kind";
        else if (L.direct == ASPEN_HIP_OPERAND_TABLE && L.IC % GEMM_BK != 0 && L.variant != ASPEN_HIP_GEMM_SMALL) why = "a K axis that needs the k-chunk table takes 64 x 64 tiles";
        else if (L.direct == ASPEN_HIP_OPERAND_TABLE && L.IC == 0) why = "channel count";
        else if (tall && L.direct == ASPEN_HIP_OPERAND_DENSE3) why = "the dense three-channel operand takes 64-row tiles";
        else if (narrow && (L.direct == ASPEN_HIP_OPERAND_DENSE3 || (L.direct == ASPEN_HIP_OPERAND_TABLE && L.IC % GEMM_BK != 0))) why = "the 32 x 32 tile reads its operand in place or steps through taps of whole K slices";
    }
    else if (L.type == K_ATTENTION_LAYER)
    {
        if (!L.in1 || L.hd == 0 || L.hd % GEMM_BK || L.heads == 0 || L.seq == 0) why = "attention geometry";
        else if (L.ld < L.seq || L.ld % GEMM_BK) why = "probability stride must be a multiple of 32 covering seq";
        else if (L.tile_n != KATTN_BN || L.tiles_m != 1) why = "K-attention tile extent";
    }
    else if (L.type == V_ATTENTION_LAYER)
    {
        if (!L.in1 || L.hd == 0 || L.heads == 0 || L.seq == 0) why = "attention geometry";
        else if (L.tile_n != VATTN_BN || L.tile_m > 64 || L.hd % L.tile_m) why = "V-attention tile extent (queries x <=64 channels of one head)";
        else if (L.direct == ASPEN_HIP_ATTENTION_FUSED)
        {
            if (!L.fuse_in || L.fuse_ld_in % 4 || L.hd > 64 || L.hd % GEMM_BK || L.tile_m != L.hd || L.ld0 < L.heads * L.hd || L.ld1 < L.heads * L.hd || L.fuse_ld_in < L.heads * L.hd)
                why = "fused attention takes whole heads of 32 or 64 channels and Query / Key / Value matrices";
        }
        else if (L.ld0 % GEMM_BK || L.ld0 < L.seq) why = "probability stride must be a multiple of 32 covering seq";
    }
    else if (L.type == MAXPOOL_LAYER || L.type == AVGPOOL_LAYER)
    {
        if (L.tiles_m > 1 && (L.tile_m % 4 || (uint64_t)L.tiles_m * L.tile_m < L.M || (uint64_t)(L.tiles_m - 1) * L.tile_m >= L.M)) why = "pool row tiles";
        else if ((uint64_t)L.tiles_n * L.tile_n < L.N) why = "tile grid does not cover the matrix";
    }
    else if (L.type == YOLO_LAYER)
    {
        if (!L.weight || L.M < 5 || L.IC % L.M || L.IC / L.M > 3 || L.IC == 0 || L.IH == 0 || L.IW == 0 || L.tiles_m != 1 || L.ld0 < L.IC) why = "yolo geometry";
        else if (L.N % (L.IH * L.IW * (L.IC / L.M))) why = "yolo columns";
    }
    else if (L.type == APPEND_LAYER)
    {
        if (!L.in1 || L.stride == 0 || L.OH == 0 || L.OW == 0 || L.OH % L.stride || L.OW % L.stride || L.IC >= L.M || L.tiles_m != 1
            || L.ld0 < L.IC || L.ld1 < L.M - L.IC || L.N % (L.OH * L.OW)) why = "append geometry";
    }
    else if (L.type == RESIDUAL_LAYER) { if (!L.in1 || L.tiles_m != 1) why = "missing second parent, or row tiles"; }
    else if (L.type == LAYERNORM_LAYER) { if (!L.weight || L.tiles_m != 1) why = "missing gamma, or row tiles"; }
    else if (L.type == SOFTMAX_LAYER) { if (L.tiles_m != 1) why = "row tiles"; }
    if (why)
    {
        snprintf (g_err, sizeof (g_err), "layer %u rejected: %s", idx, why);
        fprintf (stderr, "aspen_hip: %s\n", g_err);
        return -1;
    }
    return 0;
}

// True when every activation some tile reads is laid out so that a 128-byte cache line belongs to
// exactly one producer tile: matrix start and column stride are multiples of 128 bytes, and a tile
// spans either all rows or a multiple of 32 rows.  Then activation loads may go through the caches
// inside the persistent kernel (see ActView, mode 2).
static bool lines_have_one_producer (const aspen_hip_layer_t *layers, uint32_t num_layers)
{
    for (uint32_t l = 0; l < num_layers; l++)
    {
        const aspen_hip_layer_t &P = layers[l];
        if (P.type == INPUT_LAYER || P.num_ninst == 0) continue;      // written by the host before the launch
        bool is_read = false;
        for (uint32_t c = 0; c < num_layers && !is_read; c++) is_read = layers[c].num_ninst != 0 && (layers[c].in0 == P.out || layers[c].in1 == P.out || layers[c].fuse_in == P.out);
        const bool aligned = (uintptr_t)P.out % 128 == 0 && ((size_t)P.ld * 4) % 128 == 0 && (P.tiles_m == 1 || (P.tile_m * 4) % 128 == 0);
        const bool ok = !(is_read && !aligned) && !(P.splits > 1 && ((uintptr_t)P.partial % 128 != 0 || !aligned))
            && !(P.fuse_out && ((uintptr_t)P.fuse_out % 128 != 0 || !aligned));
        if (!ok)
        {
            if (getenv ("ASPEN_GPU_VERBOSE"))
                fprintf (stderr, "aspen_hip: layer %u (type %d, ld %u, tile_m %u, tiles_m %u) shares cache lines between tiles: coherent loads\n",
                    l, P.type, P.ld, P.tile_m, P.tiles_m);
            return false;
        }
    }
    return true;
}

// Average parallelism of the tile graph = total tile cost / cost of the longest dependency chain, with a
// crude cost per tile (K slices of a contraction tile plus a constant for fetching and storing).  Workgroups
// beyond it only wait, and those that wait next to a working one on the same compute unit are the ones
// that get the next tile as likely as those on an idle unit: tiles then share a matrix pipeline while
// other units sit idle, which stretches exactly the chains that bound a run with little parallelism.
static double graph_parallelism (const aspen_hip_layer_t *layers, const uint32_t *ninst_layer, const uint32_t *child_off,
    const uint32_t *child_idx, uint32_t num_ninst)
{
    if (num_ninst == 0) return 0.0;
    float *dist = (float *)calloc (num_ninst, sizeof (float));
    if (!dist) return 1e30;
    double total = 0.0, longest = 0.0;
    bool ordered = true;
    for (uint32_t t = 0; t < num_ninst && ordered; t++)
    {
        const aspen_hip_layer_t &L = layers[ninst_layer[t]];
        float cost = 4.f;
        if (L.type == CONV_LAYER || L.type == FC_LAYER || L.type == MATMUL_LAYER)
        {
            cost = 8.f + (float)(L.splits > 1 ? L.kiters_per_split : L.Kp / GEMM_BK);
            if (L.variant == ASPEN_HIP_GEMM_NARROW) cost = 8.f + 0.25f * (float)(L.splits > 1 ? L.kiters_per_split : L.Kp / GEMM_BK);     // a quarter of the work, a quarter of the K axis per wavefront
        }
        else if (L.type == K_ATTENTION_LAYER || L.type == V_ATTENTION_LAYER) cost = 16.f;
        dist[t] += cost;
        total += cost;
        if (dist[t] > longest) longest = dist[t];
        for (uint32_t e = child_off[t]; e < child_off[t + 1]; e++)
        {
            const uint32_t c = child_idx[e];
            if (c <= t) { ordered = false; break; }       // not listed parents-first: no estimate
            if (dist[c] < dist[t]) dist[c] = dist[t];
        }
    }
    free (dist);
    return ordered && longest > 0.0 ? total / longest : 1e30;
}

extern "C" aspen_hip_graph_t *aspen_hip_graph_create (const aspen_hip_layer_t *layers, uint32_t num_layers,
    const uint32_t *ninst_layer, const uint32_t *num_parents, const uint32_t *child_off,
    const uint32_t *child_idx, uint32_t num_ninst, const uint32_t *roots, uint32_t num_roots)
{
    if (aspen_hip_init ()) return nullptr;
    if (num_ninst > QUEUE_ID_MASK) { snprintf (g_err, sizeof (g_err), "graph has more than %u tiles", QUEUE_ID_MASK); return nullptr; }
    if (num_layers > MAX_GRAPH_LAYERS) { snprintf (g_err, sizeof (g_err), "graph has more than %u layers", MAX_GRAPH_LAYERS); return nullptr; }
    for (uint32_t l = 0; l < num_layers; l++)
        if (check_layer (layers[l], l)) return nullptr;
    // host-side sanity of the dependency structure: every index in range, counts consistent
    const uint32_t num_edges = child_off[num_ninst];
    {
        uint32_t *seen = (uint32_t *)calloc (num_ninst ? num_ninst : 1, sizeof (uint32_t));
        if (!seen) { snprintf (g_err, sizeof (g_err), "out of host memory"); return nullptr; }
        bool ok = true;
        // the members of a split-K group carry the same child list and count as one parent
        for (uint32_t t = 0; t < num_ninst && ok; t++)
        {
            if (ninst_layer[t] >= num_layers) { ok = false; break; }
            const aspen_hip_layer_t &L = layers[ninst_layer[t]];
            const uint32_t slice = L.splits > 1 ? (t - L.ninst_start) % L.splits : 0;
            if (slice != 0 && child_off[t + 1] - child_off[t] != child_off[t - slice + 1] - child_off[t - slice]) ok = false;
            for (uint32_t e = child_off[t]; e < child_off[t + 1] && ok; e++)
            {
                if (child_idx[e] >= num_ninst) ok = false;
                else if (slice != 0) { if (child_idx[e] != child_idx[child_off[t - slice] + (e - child_off[t])]) ok = false; }
                else seen[child_idx[e]]++;
            }
        }
        for (uint32_t i = 0; i < num_ninst && ok; i++) if (seen[i] != num_parents[i] || ninst_layer[i] >= num_layers) ok = false;
        for (uint32_t r = 0; r < num_roots && ok; r++) if (roots[r] >= num_ninst || num_parents[roots[r]] != 0) ok = false;
        free (seen);
        if (!ok) { snprintf (g_err, sizeof (g_err), "inconsistent dependency arrays"); fprintf (stderr, "aspen_hip: %s\n", g_err); return nullptr; }
    }
    aspen_hip_graph_t *g = (aspen_hip_graph_t *)calloc (1, sizeof (aspen_hip_graph_t));
    if (!g) { snprintf (g_err, sizeof (g_err), "out of host memory"); return nullptr; }
    g->prefer_ordered = -1;
    g->cached_loads = lines_have_one_producer (layers, num_layers) && getenv ("ASPEN_GPU_COHERENT_LOADS") == nullptr;
    g->num_layers = num_layers; g->num_ninst = num_ninst; g->num_roots = num_roots; g->num_edges = num_edges;
    g->features = graph_features (layers, num_layers);
    uint32_t group_sinks[MAX_GROUPS] = {0};
    for (uint32_t l = 0; l < num_layers; l++)
    {
        if (layers[l].graph_id >= MAX_GROUPS) { snprintf (g_err, sizeof (g_err), "layer %u: graph_id %u, at most %u networks share a run", l, layers[l].graph_id, MAX_GROUPS); free (g); return nullptr; }
        if (layers[l].graph_id + 1 > g->num_groups) g->num_groups = layers[l].graph_id + 1;
    }
    for (uint32_t t = 0; t < num_ninst; t++)
        if (child_off[t + 1] == child_off[t]) { g->num_sinks++; group_sinks[layers[ninst_layer[t]].graph_id]++; }
    // (a group without tiles would never report: it counts as finished from the start)
    uint32_t live_groups = 0;
    for (uint32_t i = 0; i < g->num_groups; i++) live_groups += group_sinks[i] != 0;
    g->d_group_sinks = upload (group_sinks, MAX_GROUPS);
    {
        // default grid: a whole number of workgroups per compute unit, no more than the graph can keep busy
        const double par = graph_parallelism (layers, ninst_layer, child_off, child_idx, num_ninst);
        g->parallelism = par;
        static const bool all_tiles = getenv ("ASPEN_GPU_ONE_KERNEL") != nullptr;       // comparisons: always the variant with every tile kind
        g->variant = NUM_KERNEL_VARIANTS - 1;
        for (int i = NUM_KERNEL_VARIANTS - 2; i >= 0 && !all_tiles; i--) if ((g->features & ~kernel_variant_tiles[i]) == 0) g->variant = i;
        const uint32_t resident = (uint32_t)g_variant_wg[g->variant][g->cached_loads ? 1 : 0];      // of the variant this graph runs on
        uint32_t per_cu = resident;
        // measured on 256 compute units (ResNet-50 batch 1 / 32, VGG-16, BERT, GPT-2): one more workgroup per
        // unit pays once the average parallelism grows by another two tiles per unit
        if (par < 2.0 * g_num_cu * resident) per_cu = (uint32_t)(par / (2.0 * g_num_cu)) + 1;
        if (per_cu > resident) per_cu = resident;
        g->default_workgroups = per_cu * (uint32_t)g_num_cu;
        if (getenv ("ASPEN_GPU_VERBOSE"))
            fprintf (stderr, "aspen_hip: %u tiles, average parallelism %.0f: %u workgroups by default\n", num_ninst, par, g->default_workgroups);
    }
    g->h_layers = (aspen_hip_layer_t *)malloc (sizeof (aspen_hip_layer_t) * (num_layers ? num_layers : 1));
    if (!g->h_layers) { snprintf (g_err, sizeof (g_err), "out of host memory"); free (g); return nullptr; }
    memcpy (g->h_layers, layers, sizeof (aspen_hip_layer_t) * num_layers);
    for (uint32_t l = 0; l < num_layers; l++) fill_derived (g->h_layers[l]);
    g->d_layers = upload (g->h_layers, num_layers);
    g->d_ninst_layer = upload (ninst_layer, num_ninst);
    g->d_num_parents = upload (num_parents, num_ninst);
    g->d_child_off = upload (child_off, (size_t)num_ninst + 1);
    g->d_child_idx = upload (child_idx, num_edges);
    g->d_roots = upload (roots, num_roots);
    g->d_dep = (uint32_t *)aspen_hip_alloc (sizeof (uint32_t) * (num_ninst + 1));
    g->queue_cap = num_ninst + QUEUE_SLACK;
    g->queue_row = queue_row (g->queue_cap);
    g->d_queue = (qentry_t *)aspen_hip_alloc (sizeof (qentry_t) * (size_t)NUM_QUEUES * QUEUE_LANES * g->queue_row);
    {
        // home queues: the eighth of its layer's tile range a tile lies in (tiles are numbered column tile by column
        // tile, the row tiles and split-K slices of a column tile next to each other)
        uint32_t *home = (uint32_t *)malloc (sizeof (uint32_t) * (num_ninst ? num_ninst : 1));
        uint32_t *pos = (uint32_t *)malloc (sizeof (uint32_t) * (num_roots ? num_roots : 1));
        // child records: what the publishing wavefront fetches with one 64-lane load
        qentry_t *rec = (qentry_t *)calloc ((size_t)(num_ninst ? num_ninst : 1) * CHILD_REC, sizeof (qentry_t));
        if (home && pos && rec)
        {
            for (uint32_t t = 0; t < num_ninst; t++)
            {
                const aspen_hip_layer_t &L = layers[ninst_layer[t]];
                const uint64_t in_layer = t >= L.ninst_start ? t - L.ninst_start : 0;
                home[t] = L.num_ninst ? (uint32_t)(in_layer * NUM_QUEUES / L.num_ninst) % NUM_QUEUES : 0u;
                // a contraction layer whose weight matrix is larger than its input (the last stage of a deep convolutional
                // network: megabytes of weights, a few hundred columns) is divided by weight rows and K parts instead, so
                // that the tiles which read the same weights meet in the same caches
                const bool contraction = L.type == CONV_LAYER || L.type == FC_LAYER || L.type == MATMUL_LAYER;
                static const bool by_weights = getenv ("ASPEN_GPU_NO_WEIGHT_HOMES") == nullptr;
                if (contraction && by_weights && L.num_ninst && (uint64_t)L.M * L.Kp > (uint64_t)L.ld0 * g->h_layers[ninst_layer[t]].in0_columns)
                {
                    const uint64_t per_column_tile = (uint64_t)L.tiles_m * (L.splits ? L.splits : 1u);
                    home[t] = (uint32_t)((in_layer % per_column_tile) * NUM_QUEUES / per_column_tile) % NUM_QUEUES;
                }
            }
            for (uint32_t r = 0; r < num_roots; r++) pos[r] = g->root_count[home[roots[r]]]++;
            for (uint32_t t = 0; t < num_ninst; t++)
            {
                const uint32_t c0 = child_off[t], n = child_off[t + 1] - c0;
                rec[(size_t)t * CHILD_REC] = n | ((qentry_t)layers[ninst_layer[t]].graph_id << 32);
                for (uint32_t c = 0; c < n && c < CHILD_REC - 1; c++)
                {
                    const uint32_t ch = child_idx[c0 + c];
                    rec[(size_t)t * CHILD_REC + 1 + c] = ((qentry_t)home[ch] << 48) | ((qentry_t)ninst_layer[ch] << 32) | ch;
                }
            }
            g->d_ninst_home = upload (home, num_ninst);
            g->d_root_pos = upload (pos, num_roots);
            g->d_child_rec = upload (rec, (size_t)num_ninst * CHILD_REC);
        }
        free (home); free (pos); free (rec);
    }
    g->d_ran = (uint32_t *)aspen_hip_alloc (sizeof (uint32_t) * (num_ninst + 1));
    g->d_state = (uint32_t *)aspen_hip_alloc (sizeof (uint32_t) * ST_ALL_WORDS);
    g->d_arrivals = (uint32_t *)aspen_hip_alloc (sizeof (uint32_t) * (num_ninst + 1));
    g->d_prof = (unsigned long long *)aspen_hip_alloc (sizeof (unsigned long long) * 16);
    if (hipHostMalloc ((void **)&g->h_abort, sizeof (uint32_t) * (HOST_DONE_WORD + MAX_GROUPS), hipHostMallocDefault) != hipSuccess) g->h_abort = nullptr;
    else memset (g->h_abort, 0, sizeof (uint32_t) * (HOST_DONE_WORD + MAX_GROUPS));
    g->live_groups = live_groups;
    if (!g->h_abort || !g->d_group_sinks || !g->d_layers || !g->d_ninst_layer || !g->d_num_parents || !g->d_child_off || !g->d_child_idx || !g->d_roots
        || !g->d_dep || !g->d_queue || !g->d_ran || !g->d_state || !g->d_child_rec || !g->d_ninst_home || !g->d_root_pos || !g->d_arrivals || !g->d_prof)
    {
        aspen_hip_graph_destroy (g);
        return nullptr;
    }
    return g;
}

extern "C" void aspen_hip_graph_destroy (aspen_hip_graph_t *g)
{
    if (!g) return;
    (void)hipStreamSynchronize (g_stream);
    aspen_hip_free (g->d_layers); aspen_hip_free (g->d_ninst_layer); aspen_hip_free (g->d_num_parents);
    aspen_hip_free (g->d_child_off); aspen_hip_free (g->d_child_idx); aspen_hip_free (g->d_roots); aspen_hip_free (g->d_ninst_home); aspen_hip_free (g->d_root_pos);
    aspen_hip_free (g->d_child_rec); aspen_hip_free (g->d_dep); aspen_hip_free (g->d_queue); aspen_hip_free (g->d_ran); aspen_hip_free (g->d_arrivals); aspen_hip_free (g->d_state); aspen_hip_free (g->d_prof); aspen_hip_free (g->d_trace); aspen_hip_free (g->d_group_sinks); aspen_hip_free (g->d_dep_spread);
    if (g->h_abort) (void)hipHostFree (g->h_abort);
    free (g->h_layers);
    free (g);
}

// ------------------------------------------------------------------------------------------------
// execution
// ------------------------------------------------------------------------------------------------
// One layer in launch mode.  A split-K layer takes two launches: within one launch the plain (write-back)
// stores of a workgroup are not visible to workgroups on other XCDs, so the slices cannot be added up by
// whichever slice finishes last, as the persistent kernel (write-through stores) does.
static void launch_layer (const aspen_hip_graph_t *g, uint32_t l)
{
    const aspen_hip_layer_t &L = g->h_layers[l];
    hipLaunchKernelGGL (layer_kernel, dim3 (L.num_ninst), dim3 (WG_THREADS), GEMM_SMEM_BYTES, g_stream, g->d_layers, l, 0u, (uint32_t *)nullptr);
    if (L.splits > 1)
        hipLaunchKernelGGL (finish_kernel, dim3 (L.tiles_m * L.tiles_n), dim3 (WG_THREADS), EPI_FLOATS (VAR2_BM, VAR2_BN) * sizeof (float), g_stream, g->d_layers, l);
}

extern "C" int aspen_hip_run_layers (aspen_hip_graph_t *g, uint32_t first_layer, uint32_t last_layer)
{
    if (!g || first_layer > last_layer || last_layer >= g->num_layers) { snprintf (g_err, sizeof (g_err), "run_layers: bad range"); return -1; }
    g->last_run_dataflow = 0;
    for (uint32_t l = first_layer; l <= last_layer; l++)
    {
        const aspen_hip_layer_t &L = g->h_layers[l];
        if (L.type == INPUT_LAYER || L.num_ninst == 0) continue;
        launch_layer (g, l);
        CHECK (hipGetLastError ());
    }
    return 0;
}

extern "C" int aspen_hip_run_dataflow (aspen_hip_graph_t *g, uint32_t workgroups, uint64_t spin_limit)
{
    if (!g) { snprintf (g_err, sizeof (g_err), "run_dataflow: null graph"); return -1; }
    if (g->num_ninst == 0) return 0;
    const uint32_t workgroups_requested = workgroups;
    if (workgroups == 0) workgroups = g->default_workgroups;
    if (workgroups > QUEUE_SLACK) workgroups = QUEUE_SLACK;         // every waiting workgroup must find a "leave" entry within its queue
    g->epoch = g->epoch % EPOCH_MAX + 1u;
    // one queue per XCD on request, when every XCD gets the same number of workgroups (workgroup b runs on XCD b % 8)
    // (ASPEN_GPU_XCD_QUEUES=0: always one queue; any other value: one queue per XCD, in groups of 2 / 4 XCDs with
    // ASPEN_GPU_XCD_QUEUE_SHIFT = 1 / 2)
    static const char *xcd_queues_env = getenv ("ASPEN_GPU_XCD_QUEUES");
    static const bool one_queue_env = xcd_queues_env != nullptr && strcmp (xcd_queues_env, "0") == 0;
    const bool xcd_queues = (xcd_queues_env != nullptr && !one_queue_env) || (g_flags & ASPEN_HIP_FLAG_XCD_QUEUES);
    static const uint32_t shift_env = getenv ("ASPEN_GPU_XCD_QUEUE_SHIFT") ? (uint32_t)atoi (getenv ("ASPEN_GPU_XCD_QUEUE_SHIFT")) : 0u;
    uint32_t nq_shift = shift_env > 2u ? 2u : shift_env;
    // Ordered mode for graphs that can never keep the device busy (one image through a deep network): no ready queue,
    // workgroups take the tiles in index order (parents first), set each one up and request its first weights BEFORE it
    // is ready, and wait on the tile's own dependency counter.  With far more workgroups than ready tiles nothing is
    // lost by binding a workgroup to a tile early, and a dependency level no longer pays for descriptor fetch, index
    // arithmetic, the weights' memory latency and two queue round trips after its parents have finished.
    static const char *ordered_env = getenv ("ASPEN_GPU_ORDERED");
    bool ordered = ordered_env ? atoi (ordered_env) != 0 : g->prefer_ordered >= 0 ? g->prefer_ordered != 0 : g->parallelism < ORDERED_BELOW;
    if (g_flags & ASPEN_HIP_FLAG_ORDERED) ordered = true;
    if (g_flags & ASPEN_HIP_FLAG_NO_ORDERED) ordered = false;
    // (a static assignment in index order only terminates when every tile's parents have smaller indices: graph_parallelism
    // reports 1e30 for a graph that is not listed that way)
    if (!g->cached_loads || xcd_queues || g->num_ninst > (1u << 20) || g->parallelism > 1e29) ordered = false;
    size_t ordered_smem = ORDERED_SMEM_BYTES;
    if (ordered)
    {
        // tiles are assigned to workgroups beforehand: every workgroup of the grid must be running
        // (graphs without 32 x 32 tiles need no weight prefetch buffers: their workgroups take the LDS of any other tile, and
        // twice as many fit a compute unit)
        static int fits[NUM_ORDERED_VARIANTS][2];
        static bool fits_known[NUM_ORDERED_VARIANTS][2];
        const int small_lds = (g->features & TILES_NARROW) == 0;
        int ov = 0;         // (the variant the launch below takes)
        while (ov + 1 < NUM_ORDERED_VARIANTS && (g->features & ~ordered_variant_tiles[ov]) != 0) ov++;
        if (!fits_known[ov][small_lds])
        {
            int o = 0;
            CHECK (hipOccupancyMaxActiveBlocksPerMultiprocessor (&o, ordered_kernels[ov], WG_THREADS, small_lds ? GEMM_SMEM_BYTES : ORDERED_SMEM_BYTES));
            fits[ov][small_lds] = o * g_num_cu;
            fits_known[ov][small_lds] = true;
        }
        const int fit = fits[ov][small_lds];
        ordered_smem = small_lds ? GEMM_SMEM_BYTES : ORDERED_SMEM_BYTES;
        if (fit < 1) ordered = false;
        else
        {
            // by default two per compute unit (one tile computes, the next is prepared); without the prefetch buffers three
            // from an estimated parallelism of 350 and four from 600 on (YOLO-v3 batch 1, 409: 1.30 / 1.25 / 1.26 ms with
            // two / three / four; ResNet-50 batch 4, 335: 0.72 / 0.76 / 0.76; VGG-16 batch 4, 766: 1.51 / 1.40 / 1.34)
            // (transformer graphs, whose kernel fits three times: two below 600; BERT-base 8 x 128, 519: 1.96 / 2.00 ms with
            // two / three, 16 x 128, 1024: 3.49 / 3.33)
            const double three_from = (g->features & TILES_ATTENTION) ? 600.0 : 350.0;
            const uint32_t per_cu = !small_lds || g->parallelism < three_from ? 2u : g->parallelism < 600.0 ? 3u : 4u;
            if (workgroups_requested == 0) workgroups = per_cu * (uint32_t)g_num_cu < (uint32_t)fit ? per_cu * (uint32_t)g_num_cu : (uint32_t)fit;
            if (workgroups > (uint32_t)fit) workgroups = (uint32_t)fit;
        }
    }
    if (ordered && !g->d_dep_spread)
    {
        g->dep_stride = (g->num_ninst + 31u) / 32u * 32u + 1024u;
        g->d_dep_spread = (uint32_t *)aspen_hip_alloc (sizeof (uint32_t) * 32u * (size_t)g->dep_stride);
        if (!g->d_dep_spread) return -1;
    }
    uint32_t nq_mask = (xcd_queues && workgroups % NUM_QUEUES == 0) ? (NUM_QUEUES >> nq_shift) - 1u : 0u;
    // By default a graph that fills the device (every compute unit holds as many workgroups as fit) runs on TWO queues,
    // one per half of the XCDs: tiles that read the same activations then meet in one of four L2s instead of eight (a
    // tenth less memory traffic on the convolutional networks), and two pools of 512 workgroups balance as well as one of
    // 1024 (same run time; four and eight queues cost 1 % and 3 %).  Smaller grids keep one queue: their runs are bound by
    // dependency chains, and every restriction on who may take a ready tile lengthens those.
    if (!xcd_queues && !one_queue_env && !ordered && workgroups % NUM_QUEUES == 0
        && workgroups >= (uint32_t)g_variant_wg[g->variant][g->cached_loads ? 1 : 0] * (uint32_t)g_num_cu)
    { nq_shift = 2u; nq_mask = (NUM_QUEUES >> nq_shift) - 1u; }
    queue_counts_t counts;
    if (nq_mask && g->root_shift != nq_shift)
    {
        // positions of the roots inside their queues for this grouping of the XCDs
        uint32_t *home = (uint32_t *)malloc (sizeof (uint32_t) * g->num_ninst), *roots = (uint32_t *)malloc (sizeof (uint32_t) * g->num_roots), *pos = (uint32_t *)malloc (sizeof (uint32_t) * g->num_roots);
        if (!home || !roots || !pos || aspen_hip_sync () || aspen_hip_d2h (home, g->d_ninst_home, sizeof (uint32_t) * g->num_ninst) || aspen_hip_d2h (roots, g->d_roots, sizeof (uint32_t) * g->num_roots))
        { free (home); free (roots); free (pos); snprintf (g_err, sizeof (g_err), "run_dataflow: cannot regroup the roots"); return -1; }
        memset (g->root_count, 0, sizeof (g->root_count));
        for (uint32_t r = 0; r < g->num_roots; r++) pos[r] = g->root_count[(home[roots[r]] >> nq_shift) & nq_mask]++;
        const int failed = aspen_hip_h2d (g->d_root_pos, pos, sizeof (uint32_t) * g->num_roots);
        free (home); free (roots); free (pos);
        if (failed) return -1;
        g->root_shift = nq_shift;
    }
    for (uint32_t q = 0; q < NUM_QUEUES; q++) counts.n[q] = g->root_count[q];
    {
        // The slots a run rewrites depend on the grid (leave entries), the hand-off (kept tiles take no slot) and the
        // queue grouping.  A slot an earlier run with other settings wrote could otherwise survive until the epoch
        // comes round again and be taken for an entry of that run.
        const uint32_t config = workgroups ^ ((uint32_t)ordered << 15) ^ (nq_mask << 16) ^ (nq_shift << 20) ^ ((g_flags & (ASPEN_HIP_FLAG_NO_HANDOFF | ASPEN_HIP_FLAG_XCD_QUEUES | ASPEN_HIP_FLAG_SKIP_TILES)) << 24);
        if (g->epoch == 1u || config != g->queue_config)
        {
            const size_t entries = (size_t)NUM_QUEUES * QUEUE_LANES * g->queue_row;
            hipLaunchKernelGGL (clear_queue_kernel, dim3 (stream_grid (entries)), dim3 (WG_THREADS), 0, g_stream, g->d_queue, entries);
            CHECK (hipGetLastError ());
        }
        g->queue_config = config;
    }
    // An ordered run leaves its counters armed for the next one, so back-to-back ordered runs launch ONE kernel.  The
    // arming pass runs in front of the first ordered run, after a run that was given up, and whenever the per-tile
    // execution counts are kept (they are reset there).
    if (*(volatile uint32_t *)g->h_abort != 0) g->spread_armed = 0;
    const bool skip_arm = ordered && g->spread_armed && !(g_flags & (ASPEN_HIP_FLAG_COUNT_TILES | ASPEN_HIP_FLAG_SKIP_TILES));
    if (!skip_arm)
    {
        hipLaunchKernelGGL (arm_kernel, dim3 ((g->num_ninst + 255) / 256), dim3 (256), 0, g_stream,
            ordered ? g->d_dep_spread : g->d_dep, g->d_num_parents, g->d_queue, g->d_ran, g->d_roots, g->d_ninst_layer, g->d_ninst_home, g->d_root_pos, counts,
            g->num_ninst, g->num_roots, g->d_state, g->epoch, g->queue_row, nq_mask, nq_shift, g->d_arrivals, ordered ? g->dep_stride : 0u);
        CHECK (hipGetLastError ());
    }
    g->spread_armed = ordered ? 1 : 0;          // (a run on the ready queue leaves the shared counters at their final values)
    dataflow_args_t a;
    a.layers = g->d_layers; a.ninst_layer = g->d_ninst_layer; a.ninst_home = g->d_ninst_home; a.child_off = g->d_child_off; a.child_idx = g->d_child_idx; a.child_rec = g->d_child_rec;
    a.num_parents = g->d_num_parents;
    a.dep = ordered ? g->d_dep_spread : g->d_dep; a.dep_stride = ordered ? g->dep_stride : 0u; a.queue = g->d_queue; a.state = g->d_state; a.ran = g->d_ran; a.arrivals = g->d_arrivals; a.prof = g->d_prof; a.host_abort = g->h_abort;
    g->run_serial = g->run_serial + 1u ? g->run_serial + 1u : 1u;
    g->last_run_dataflow = 1;
    a.group_sinks = g->d_group_sinks; a.num_groups = g->live_groups; a.run_serial = g->run_serial;
    if ((g_flags & ASPEN_HIP_FLAG_TRACE) && !g->d_trace)
    {
        g->d_trace = (unsigned long long *)aspen_hip_alloc (sizeof (unsigned long long) * 4 * (size_t)g->num_ninst);     // start / end, then K loop / epilogue stamps
        if (!g->d_trace) return -1;
    }
    a.trace = g->d_trace;
    a.num_ninst = g->num_ninst; a.num_sinks = g->num_sinks; a.epoch = g->epoch; a.flags = g_flags; a.queue_row = g->queue_row; a.queue_cap = g->queue_cap; a.nq_mask = nq_mask; a.nq_shift = nq_shift; a.spin_limit = spin_limit ? spin_limit : DEFAULT_SPIN_LIMIT;
    CHECK (hipEventRecord (g_events[NUM_EVENTS - 2], g_stream));
    {
        const void *kernel = dataflow_kernels[g->variant][g->cached_loads ? 1 : 0];
        if (ordered)
        {
            int v = 0;
            while (v + 1 < NUM_ORDERED_VARIANTS && (g->features & ~ordered_variant_tiles[v]) != 0) v++;
            kernel = ordered_kernels[v];
        }
        g->last_run_ordered = ordered;
        void *kernel_args[] = {&a};
        CHECK (hipLaunchKernel (kernel, dim3 (workgroups), dim3 (WG_THREADS), kernel_args, ordered ? ordered_smem : GEMM_SMEM_BYTES, g_stream));
    }
    CHECK (hipGetLastError ());
    CHECK (hipEventRecord (g_events[NUM_EVENTS - 1], g_stream));
    return 0;
}

extern "C" void aspen_hip_graph_set_ordered (aspen_hip_graph_t *g, int ordered) { if (g) g->prefer_ordered = ordered < 0 ? -1 : ordered != 0; }
extern "C" int aspen_hip_graph_last_run_ordered (const aspen_hip_graph_t *g) { return g ? g->last_run_ordered : 0; }

extern "C" double aspen_hip_graph_parallelism (const aspen_hip_graph_t *g) { return g ? g->parallelism : 0.0; }

extern "C" int aspen_hip_profile_layers (aspen_hip_graph_t *g, uint32_t iters, float *ms_per_layer)
{
    if (!g || !ms_per_layer || iters == 0) return -1;
    for (uint32_t l = 0; l < g->num_layers; l++)
    {
        const aspen_hip_layer_t &L = g->h_layers[l];
        ms_per_layer[l] = 0.f;
        if (L.type == INPUT_LAYER || L.num_ninst == 0) continue;
        CHECK (hipEventRecord (g_events[NUM_EVENTS - 4], g_stream));
        for (uint32_t i = 0; i < iters; i++) launch_layer (g, l);
        CHECK (hipGetLastError ());
        CHECK (hipEventRecord (g_events[NUM_EVENTS - 3], g_stream));
        CHECK (hipEventSynchronize (g_events[NUM_EVENTS - 3]));
        float ms = 0.f;
        CHECK (hipEventElapsedTime (&ms, g_events[NUM_EVENTS - 4], g_events[NUM_EVENTS - 3]));
        ms_per_layer[l] = ms / (float)iters;
    }
    return 0;
}

extern "C" void aspen_hip_set_flags (uint32_t flags) { g_flags = flags; }

extern "C" int aspen_hip_sync (void)
{
    if (aspen_hip_init ()) return -1;
    CHECK (hipStreamSynchronize (g_stream));
    return 0;
}

extern "C" int aspen_hip_graph_sync (aspen_hip_graph_t *g)
{
    if (aspen_hip_init ()) return -1;
    CHECK (hipStreamSynchronize (g_stream));
    if (g && *(volatile uint32_t *)g->h_abort != 0)
    {
        *g->h_abort = 0;
        g->spread_armed = 0;
        snprintf (g_err, sizeof (g_err), "dataflow run stalled: a wait on the ready queue exceeded its spin limit and the run was aborted");
        fprintf (stderr, "aspen_hip: %s\n", g_err);
        return ASPEN_HIP_ERR_STALLED;
    }
    return 0;
}

extern "C" int aspen_hip_graph_group_done (aspen_hip_graph_t *g, uint32_t group)
{
    if (!g || group >= g->num_groups || !g->last_run_dataflow) return -1;
    return __atomic_load_n (&g->h_abort[HOST_DONE_WORD + group], __ATOMIC_ACQUIRE) == g->run_serial ? 1 : 0;
}

extern "C" int aspen_hip_graph_wait_group (aspen_hip_graph_t *g, uint32_t group)
{
    if (aspen_hip_init ()) return -1;
    if (!g || group >= g->num_groups || !g->last_run_dataflow) return -1;
    for (;;)
    {
        // the word is written by the device into pinned host memory: a few hundred polls between two looks at the stream
        for (int spin = 0; spin < 256; spin++)
        {
            if (__atomic_load_n (&g->h_abort[HOST_DONE_WORD + group], __ATOMIC_ACQUIRE) == g->run_serial) return 0;
            __builtin_ia32_pause ();
        }
        if (__atomic_load_n (&g->h_abort[0], __ATOMIC_ACQUIRE) != 0) return 0;      // given up: aspen_hip_graph_sync reports it
        if (hipStreamQuery (g_stream) == hipSuccess) return 0;                       // the run is over (a group without tiles never reports)
    }
}

extern "C" int aspen_hip_d2h_side (void *dst, const void *src, size_t bytes)
{
    if (aspen_hip_init ()) return -1;
    CHECK (hipMemcpyAsync (dst, src, bytes, hipMemcpyDeviceToHost, g_side_stream));
    CHECK (hipStreamSynchronize (g_side_stream));
    return 0;
}

extern "C" void aspen_hip_graph_debug_set_epoch (aspen_hip_graph_t *g, uint32_t epoch) { if (g) g->epoch = epoch % EPOCH_MAX; }

extern "C" int aspen_hip_idle (void)
{
    if (aspen_hip_init ()) return -1;
    return hipStreamQuery (g_stream) == hipSuccess ? 1 : 0;
}

extern "C" int aspen_hip_dataflow_stats (aspen_hip_graph_t *g, uint32_t *executed, uint32_t *double_runs, uint32_t *abort_flag)
{
    if (!g) return -1;
    uint32_t st[ST_WORDS];
    if (aspen_hip_d2h (st, g->d_state, sizeof (st))) return -1;
    if (executed) *executed = st[ST_DONE];
    if (abort_flag) *abort_flag = st[ST_ABORT];
    if (double_runs) *double_runs = st[ST_TWICE];
    return 0;
}

extern "C" int aspen_hip_dataflow_profile (aspen_hip_graph_t *g, uint64_t ticks[16], int reset)
{
    if (!g || !ticks) return -1;
    unsigned long long h[16];
    if (aspen_hip_d2h (h, g->d_prof, sizeof (h))) return -1;
    for (int i = 0; i < 16; i++) ticks[i] = h[i];
    if (reset) { CHECK (hipMemsetAsync (g->d_prof, 0, sizeof (h), g_stream)); }
    return 0;
}

extern "C" int aspen_hip_dataflow_trace (aspen_hip_graph_t *g, uint64_t *start_end, uint32_t num_ninst)
{
    if (!g || !start_end || !g->d_trace || num_ninst != g->num_ninst)
    { snprintf (g_err, sizeof (g_err), "dataflow_trace: no traced run, or wrong tile count"); return -1; }
    return aspen_hip_d2h (start_end, g->d_trace, sizeof (uint64_t) * 2 * (size_t)num_ninst);
}

extern "C" int aspen_hip_dataflow_trace_phases (aspen_hip_graph_t *g, uint64_t *kloop_epilogue, uint32_t num_ninst)
{
    if (!g || !kloop_epilogue || !g->d_trace || num_ninst != g->num_ninst)
    { snprintf (g_err, sizeof (g_err), "dataflow_trace_phases: no traced run, or wrong tile count"); return -1; }
    return aspen_hip_d2h (kloop_epilogue, g->d_trace + 2 * (size_t)num_ninst, sizeof (uint64_t) * 2 * (size_t)num_ninst);
}

extern "C" int aspen_hip_event_record (int slot)
{
    if (aspen_hip_init ()) return -1;
    if (slot < 0 || slot >= NUM_EVENTS) return -1;
    CHECK (hipEventRecord (g_events[slot], g_stream));
    return 0;
}

extern "C" int aspen_hip_event_elapsed_ms (int a, int b, float *ms)
{
    if (a < 0 || a >= NUM_EVENTS || b < 0 || b >= NUM_EVENTS || !ms) return -1;
    CHECK (hipEventSynchronize (g_events[b]));
    CHECK (hipEventElapsedTime (ms, g_events[a], g_events[b]));
    return 0;
}

extern "C" int aspen_hip_sgemm (uint32_t M, uint32_t N, uint32_t K, const float *A, uint32_t lda, const float *B,
    uint32_t ldb, float *C, uint32_t ldc, const float *bias, int act)
{
    if (aspen_hip_init ()) return -1;
    if (K == 0 || K % GEMM_BK || lda % 4 || ldb % 4 || ldc % 4 || lda < K || ldb < K || ldc < M)
    { snprintf (g_err, sizeof (g_err), "sgemm: K must be a multiple of 32, strides multiples of 4"); return -1; }
    // weight rows are read in blocks of 64 without a row clamp: stage A into a zero-padded copy
    const uint32_t Mp = (M + 127) / 128 * 128;
    float *Ap = (float *)aspen_hip_alloc ((size_t)Mp * K * sizeof (float));
    if (!Ap) return -1;
    CHECK (hipMemcpy2DAsync (Ap, (size_t)K * 4, A, (size_t)lda * 4, (size_t)K * 4, M, hipMemcpyDeviceToDevice, g_stream));
    aspen_hip_layer_t L;
    memset (&L, 0, sizeof (L));
    L.type = MATMUL_LAYER; L.act = act; L.variant = ASPEN_HIP_GEMM_SMALL; L.direct = 1;
    L.M = M; L.N = N; L.ld = ldc; L.tile_m = 64; L.tile_n = 64;
    L.tiles_m = (M + 63) / 64; L.tiles_n = (N + 63) / 64; L.num_ninst = L.tiles_m * L.tiles_n; L.splits = 1;
    L.K = K; L.Kp = K; L.ld0 = ldb; L.out = C; L.in0 = B; L.weight = Ap; L.bias = bias;
    fill_derived (L);
    aspen_hip_layer_t *dL = upload (&L, 1);
    if (!dL) { aspen_hip_free (Ap); return -1; }
    hipLaunchKernelGGL (layer_kernel, dim3 (L.num_ninst), dim3 (WG_THREADS), GEMM_SMEM_BYTES, g_stream, dL, 0u, 0u, (uint32_t *)nullptr);      // no split-K: the arrival counters are not touched
    hipError_t e = hipGetLastError ();
    if (e == hipSuccess) e = hipStreamSynchronize (g_stream);
    aspen_hip_free (dL); aspen_hip_free (Ap);
    if (e != hipSuccess) return fail (e, "sgemm launch");
    return 0;
}

// ------------------------------------------------------------------------------------------------
// SGEMM that allocates nothing (for callers that cannot call hipMalloc: tight serving loops, harnesses that
// forbid it).  It launches on the library's own stream, so it cannot join a caller's stream capture, and the first
// call on a device performs the library's one-time initialisation (stream and event creation, kernel attributes).  aspen_hip_sgemm stages A into a zero-padded copy it allocates and frees per call; here that
// staging copy lives in a file-scope device array, and the layer descriptor travels as a kernel argument.
// Each device holds its own copy of the array at its own address: the address is looked up once per device
// with hipGetSymbolAddress and only that pointer is ever handed to kernels.  Every call on a device shares the
// array (it keeps the previous call's contents, so the padding rows are rewritten each time): calls are ordered
// by the library's one stream; calls made concurrently from several host threads would race.
// ------------------------------------------------------------------------------------------------
#define SGEMM_SCRATCH_BYTES (8u << 20)
#define MAX_DEVICES 16
static __device__ __align__ (256) unsigned char scratch[SGEMM_SCRATCH_BYTES];
static float *g_scratch_ptr[MAX_DEVICES];           // device address of `scratch` per device, see scratch_for_current_device

static float *scratch_for_current_device (void)
{
    int dev = -1;
    if (hipGetDevice (&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES) { snprintf (g_err, sizeof (g_err), "sgemm_static: no current device"); return nullptr; }
    if (g_scratch_ptr[dev] == nullptr)
    {
        void *p = nullptr;
        const hipError_t e = hipGetSymbolAddress (&p, HIP_SYMBOL (scratch));
        if (e != hipSuccess || p == nullptr) { fail (e, "hipGetSymbolAddress (scratch)"); return nullptr; }
        g_scratch_ptr[dev] = (float *)p;
    }
    return g_scratch_ptr[dev];
}

// dst[r][0..K) = src[r][0..K) for r < M, zeros for M <= r < Mp; K % 4 == 0, lda % 4 == 0
__global__ void __launch_bounds__ (WG_THREADS) pad_rows_kernel (const float *__restrict__ src, uint32_t lda, float *__restrict__ dst, uint32_t M, uint32_t Mp, uint32_t K)
{
    const uint32_t k4 = K >> 2;
    const size_t n = (size_t)Mp * k4, step = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += step)
    {
        const uint32_t r = (uint32_t)(i / k4), c = (uint32_t)(i - (size_t)r * k4) * 4;
        const float4 v = r < M ? gld4 (src + (size_t)r * lda + c) : make_float4 (0.f, 0.f, 0.f, 0.f);
        st4 (dst + (size_t)r * K + c, v);
    }
}

// one contraction tile per workgroup, the descriptor in the kernel-argument segment
__global__ void __launch_bounds__ (WG_THREADS, WG_PER_CU) sgemm_kernel (const aspen_hip_layer_t L)
{
    extern __shared__ __align__ (16) float smem[];
    run_tile<0> ([&] () { return uniform_layer (L); }, blockIdx.x, false, smem, [] () { return (uint32_t *)nullptr; });
}

extern "C" size_t aspen_hip_sgemm_static_max_bytes (void) { return SGEMM_SCRATCH_BYTES; }

extern "C" int aspen_hip_sgemm_static (uint32_t M, uint32_t N, uint32_t K, const float *A, uint32_t lda, const float *B,
    uint32_t ldb, float *C, uint32_t ldc, const float *bias, int act)
{
    if (aspen_hip_init ()) return -1;
    if (M == 0 || N == 0 || !A || !B || !C) { snprintf (g_err, sizeof (g_err), "sgemm_static: empty problem or null pointer"); return -1; }
    if (K == 0 || K % GEMM_BK || lda % 4 || ldb % 4 || ldc % 4 || lda < K || ldb < K || ldc < M)
    { snprintf (g_err, sizeof (g_err), "sgemm_static: K must be a multiple of 32, strides multiples of 4"); return -1; }
    if (((uintptr_t)A | (uintptr_t)B | (uintptr_t)C) % 16 || (bias && (uintptr_t)bias % 4))
    { snprintf (g_err, sizeof (g_err), "sgemm_static: A, B and C must be 16-byte aligned"); return -1; }
    const uint64_t Mp = ((uint64_t)M + 127) / 128 * 128;
    if (Mp * K * sizeof (float) > SGEMM_SCRATCH_BYTES)
    {
        snprintf (g_err, sizeof (g_err), "sgemm_static: roundup (M, 128) * K * 4 = %llu bytes exceeds the static staging buffer of %u bytes; use aspen_hip_sgemm",
            (unsigned long long)(Mp * K * sizeof (float)), SGEMM_SCRATCH_BYTES);
        return -1;
    }
    if ((uint64_t)N * ldc * 4 >= 0xffffff00ull || (uint64_t)N * ldb * 4 >= 0xffffff00ull) { snprintf (g_err, sizeof (g_err), "sgemm_static: matrix larger than 4 GiB"); return -1; }
    float *Ap = scratch_for_current_device ();
    if (!Ap) return -1;
    hipLaunchKernelGGL (pad_rows_kernel, dim3 (stream_grid ((size_t)Mp * (K / 4))), dim3 (WG_THREADS), 0, g_stream, A, lda, Ap, M, (uint32_t)Mp, K);
    CHECK (hipGetLastError ());
    aspen_hip_layer_t L;
    memset (&L, 0, sizeof (L));
    L.type = MATMUL_LAYER; L.act = act; L.variant = ASPEN_HIP_GEMM_SMALL; L.direct = 1;
    L.M = M; L.N = N; L.ld = ldc; L.tile_m = VAR2_BM; L.tile_n = VAR2_BN;
    L.tiles_m = (M + VAR2_BM - 1) / VAR2_BM; L.tiles_n = (N + VAR2_BN - 1) / VAR2_BN; L.num_ninst = L.tiles_m * L.tiles_n; L.splits = 1;
    L.K = K; L.Kp = K; L.ld0 = ldb; L.out = C; L.in0 = B; L.weight = Ap; L.bias = bias;
    fill_derived (L);
    hipLaunchKernelGGL (sgemm_kernel, dim3 (L.num_ninst), dim3 (WG_THREADS), GEMM_SMEM_BYTES, g_stream, L);
    CHECK (hipGetLastError ());
    return 0;
}
