/*
 * sgl_hot.h -- C ABI of libsgl_hot.so: the temporal-GNN mini-batch hot path of
 * StarryGL for one GPU's graph partition, written for AMD gfx950 (MI355X).
 *
 * The four stages behind this boundary are
 *   (1) temporal neighbour sampling over a time-sorted CSR (T-CSR),
 *   (2) unique + compaction of sampled node ids to dense local ids,
 *   (3) feature / TGN-memory row gather through a cache index
 *       (HBM-resident hot rows, pinned-host cold rows),
 *   (4) the cos(w*dt + b) time encoding.
 *
 * Conventions
 *   - every pointer named in a "device" role must be dereferenceable from the
 *     GPU (hipMalloc memory, or hipHostMalloc'ed pinned memory where stated);
 *   - ids, timestamps and offsets are int64_t;
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream);
 *   - every entry point returns an int32_t status (SGL_OK or a negative SGL_E*);
 *     no C++ exception crosses the boundary, nothing calls exit();
 *   - the library allocates no device memory: outputs and workspace belong to
 *     the caller, `*_workspace_bytes` tells how much workspace a call needs;
 *   - entry points are asynchronous w.r.t. the host unless stated otherwise;
 *     two calls that share a workspace or a remap state must be ordered on one
 *     stream.
 *
 * The reference interface each entry point replaces is cited as
 * path:line relative to the StarryGL source tree.
 */
#ifndef SGL_HOT_H
#define SGL_HOT_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SGL_ABI_VERSION 8

/* ------------------------------------------------------------------ status */
#define SGL_OK        0
#define SGL_EINVAL  (-1) /* null pointer, negative size, bad enum value        */
#define SGL_ERANGE  (-2) /* node / chunk id outside [0,n), unsorted timestamps */
#define SGL_ENOTSUP (-3) /* unknown sampling strategy, unsupported fanout      */
#define SGL_EHIP    (-4) /* a HIP runtime call failed (see error string)       */
#define SGL_ENOMEM  (-5) /* caller-provided workspace / capacity too small     */

/* Thread-local, human readable description of the last non-OK status returned
 * to the calling thread.  Replaces the C++ exceptions / TORCH_CHECK messages of
 * csrc/srcs/starrygl/export.cu:237-244 and sample.cu.hpp:1001-1062. */
const char* sgl_last_error_string(void);
int32_t     sgl_abi_version(void);
/* sizeof of the ABI's structs as this library was compiled, so that a binding
 * which mirrors them field by field (ctypes, cgo, JNI) can check its layout at
 * load time: which = 0 sgl_tcsr, 1 sgl_sample_params, 2 sgl_hop_out,
 * 3 sgl_cache, 4 sgl_gather_seg, 5 sgl_seed_query, 6 sgl_window_params;
 * 0 for any other index. */
size_t      sgl_struct_bytes(int32_t which);

/* Kernels whose blocks exchange totals inside one launch (the 2-hop sampler of
 * small calls, the numbering pass of sgl_unique_compact on small universes)
 * poll for an earlier block's descriptor at most `polls` times before they give
 * up and poison the call's counts (see sgl_sample_khop, sgl_unique_compact).
 * polls <= 0 restores the default (2^20).  No counterpart in the reference;
 * meant for tests of that error path (a limit of 1 makes it reachable while
 * every kernel still exits normally).  Returns the previous limit. */
int32_t     sgl_set_wait_limit(int32_t polls);

/* ------------------------------------------------------------------- T-CSR */
/* Time-sorted CSR of one partition.  Row v occupies [row_ptr[v], row_ptr[v+1]);
 * inside a row edges ascend in (ts, eid).  Replaces the device arrays
 * row_ptr_/col_idx_/col_ts_/edge_id_ of `Graph` (sample.cu.hpp:960-1185). */
typedef struct sgl_tcsr {
    int64_t        n;       /* number of nodes                  */
    int64_t        m;       /* number of edges                  */
    const int64_t* row_ptr; /* [n+1] device                     */
    const int64_t* col;     /* [m]   device: destination node   */
    const int64_t* ts;      /* [m]   device: edge timestamp     */
    const int64_t* eid;     /* [m]   device: edge id            */
    /* Optional (NULL = absent) next-hop index of sgl_tcsr_hop_hint_build: for the
     * edge at position e, hop_hint[e] is the position in row col[e] of the first
     * edge whose timestamp is >= ts[e], i.e. where the window of the next hop's
     * slot (col[e], ts[e]) ends.  With it the sampler needs no search for the
     * slots of hops >= 1 (strictly-before windows, slot time = edge time). */
    const int64_t* hop_hint;/* [m]   device, or NULL            */
    /* Optional (NULL = absent) interleaved copy of the edge arrays, filled by
     * sgl_tcsr_records_build: rec[4*e .. 4*e+3] = {col[e], ts[e], eid[e],
     * x}, 32 bytes per edge; x = -1 without the index, else hop_hint[e] in bits
     * 0..39 and, in bits 40..62, the length of the window that entry ends
     * (hop_hint[e] - row_ptr[col[e]]) plus one, saturating at 2^23 - 1 (0 = not
     * recorded): a slot of the next hop then knows its whole window.  The uniform
     * strategy picks edges scattered over a window: from the separate arrays
     * every pick costs one memory sector per array, from the records one per
     * pick.  Searches always run on `ts`; results do not depend on it. */
    const int64_t* rec;     /* [4*m] device, 32-byte aligned, or NULL */
} sgl_tcsr;

/* Fill rec[0 .. 4*m) for the T-CSR `g` (whose own rec field is ignored; its
 * hop_hint field, when set, is copied into the records).  No counterpart in
 * the reference. */
int32_t sgl_tcsr_records_build(const sgl_tcsr* g, int64_t* rec, void* stream);

/* Fill hop_hint[0..m) for the T-CSR `g` (whose own hop_hint field is ignored):
 * one lower-bound search per edge, done once per graph.  -1 for an edge whose
 * destination lies outside [0,n).  No counterpart in the reference, which
 * searches the neighbour's row for every sampled edge of every batch
 * (find_time_range, sample.cu.hpp:264-295). */
int32_t sgl_tcsr_hop_hint_build(const sgl_tcsr* g, int64_t* hop_hint, void* stream);

/* out[i] = position in row node[i] of the first edge whose timestamp is >= t[i]
 * (row_ptr[node[i]+1] if there is none, -1 for a node outside [0,n)), i < N:
 * where the strictly-before window of the slot (node[i], t[i]) ends.  The same
 * search as find_time_range's upper end (sample.cu.hpp:264-295), as a batch:
 * a loader runs it once over the event stream it is going to train on -
 * (src, ts) and (dst, ts) of every event - and hands the values of a batch's
 * roots to the sampler (sgl_sample_params.root_hint), which then searches for
 * the negatives only. */
int32_t sgl_window_end(const sgl_tcsr* g, const int64_t* node, const int64_t* t,
                       int64_t N, int64_t* out, void* stream);

/* Build a T-CSR from a COO edge list (replaces from_edge_index / Graph::Graph,
 * export.cu:229-250, sample.cu.hpp:985-1185).  `eid` may be NULL (= 0..m-1).
 * Output order is the stable sort by (src, ts, eid).  Synchronous: returns
 * SGL_ERANGE if any src/dst is outside [0,n) (sample.cu.hpp:1043-1048). */
size_t  sgl_tcsr_build_workspace_bytes(int64_t n, int64_t m);
int32_t sgl_tcsr_build(int64_t n, int64_t m,
                       const int64_t* src, const int64_t* dst,
                       const int64_t* ts, const int64_t* eid,
                       int64_t* row_ptr, int64_t* col, int64_t* col_ts,
                       int64_t* col_eid,
                       void* workspace, size_t workspace_bytes, void* stream);

/* Check an adopted (already sorted) T-CSR: row_ptr monotone with
 * row_ptr[0]=0,row_ptr[n]=m, col in [0,n), ts ascending inside every row.
 * Synchronous.  `workspace` needs 8 bytes. */
int32_t sgl_tcsr_validate(const sgl_tcsr* g, void* workspace,
                          size_t workspace_bytes, void* stream);

/* ---------------------------------------------------------------- sampling */
#define SGL_SAMPLE_RECENT  0 /* "recent"  : the last min(k,cnt) window edges  */
#define SGL_SAMPLE_UNIFORM 1 /* "uniform" : k distinct window edges, uniform  */

/* Largest fanout the uniform strategy accepts (a slot's picks are kept in the
 * LDS of its block).  The most-recent strategy copies runs: its limit is what
 * the 32-bit edge offsets inside a block's chunk of 512 slots can hold.  The
 * reference has no limit for either (uniform_sample_single_hop_kernel,
 * sample.cu.hpp:783-827); SGL_ENOTSUP beyond. */
#define SGL_UNIFORM_MAX_FANOUT 1024
#define SGL_RECENT_MAX_FANOUT  (1 << 21)

/* Arguments of Graph::sample_src_in_chunks_khop (sample.cu.hpp:1532-1534,
 * export.cu:194-201).  Candidate window of a slot (v, t):
 *   t_lo <= ts[e] < t_hi,  t_hi = t + (equal_root_time ? 1 : 0),
 *   t_lo = allowed_offset < 0 ? -inf : t - allowed_offset. */
typedef struct sgl_sample_params {
    int32_t  type;            /* SGL_SAMPLE_*                                  */
    int32_t  fanout;          /* k                                             */
    int64_t  allowed_offset;  /* < 0: window is unbounded below                */
    int32_t  equal_root_time; /* 1: edges with ts == t are candidates          */
    int32_t  keep_root_time;  /* uniform only: neighbors_ts = root t           */
    int32_t  replace;         /* uniform only: 1 = k iid draws (may repeat)    */
    int32_t  hop;             /* RNG stream selector for sgl_sample_hop        */
    uint64_t seed;            /* Philox4x32-10 key                             */
    /* Optional fusion with the unique stage (no counterpart in the reference,
     * whose Remapper marks ids in a pass of its own, sample.cu.hpp:1719-1760):
     * when mark_state is a state of sgl_remap_init over mark_universe ids, the
     * sampler also records every id it emits - the hop-0 slot nodes of
     * sgl_sample_khop and the neighbours of every hop - as pending in that
     * state, which is the first pass of sgl_unique_compact.  The next
     * sgl_unique_compact on the state must then be the one over exactly those
     * arrays, with reset = 1 and mode SGL_UNIQUE_SORTED | SGL_UNIQUE_PREMARKED. */
    void*    mark_state;      /* NULL: off                                     */
    int64_t  mark_universe;
    /* Optional, sgl_sample_khop / sgl_sample_khop_multi only (no counterpart in
     * the reference): root_hint[s], s < S_pos, is where the window of positive
     * slot s ends - the value sgl_window_end gives for (root of s, root_ts[s]) -
     * or -1 (search).  Used when equal_root_time == 0; values are clamped to the
     * root's row, so a wrong hint gives a wrong sample, never a stray access.
     * Negative roots are always searched. */
    const int64_t* root_hint; /* device int64[S_pos], or NULL                  */
    /* SGL_SAMPLE_MULTI_LAUNCH: sgl_sample_khop / _multi take the launch-per-hop
     * route whatever the size of the call (no kernel of that route waits for
     * another block).  What a caller re-issues a query with after a result
     * whose counts[2] read INT64_MAX (see sgl_sample_khop). */
    int32_t  flags;
    int32_t  reserved;        /* 0 */
} sgl_sample_params;
#define SGL_SAMPLE_MULTI_LAUNCH 1

/* One hop's result, caller-allocated (replaces TemporalNeighbor,
 * sample.cu.hpp:882-915).  With S slots and E = sum_s c_s sampled edges:
 *   root_start_ptr[0..S] = exclusive prefix of c (root_start_ptr[S] = E),
 *   root_end_ptr[s] = root_start_ptr[s+1] for s < S, root_end_ptr[S] = E,
 *   neighbors*, [0..E): slot s owns [root_start_ptr[s], root_end_ptr[s]),
 *   neighbors_dt = ts[e] - t_root,
 *   counts[0] = S, counts[1] = E, counts[2] = slots with an out-of-range
 *   node (device scalars). */
typedef struct sgl_hop_out {
    int64_t  capacity_slots; /* root_*_ptr hold capacity_slots+1 entries       */
    int64_t  capacity_edges; /* neighbors* hold capacity_edges entries;        */
                             /* must be >= capacity_slots * fanout             */
    int64_t* root_start_ptr;
    int64_t* root_end_ptr;
    int64_t* neighbors;
    int64_t* neighbors_ts;
    int64_t* neighbors_eid;
    int64_t* neighbors_dt;
    int64_t* counts;         /* device int64[3]                                */
} sgl_hop_out;

/* One sampling hop over explicit slots (slot_node[s], slot_ts[s]), s < S.
 * S = *S_dev when S_dev != NULL (a device scalar, must be <= S_max), else
 * S_max.  Replaces static_recent_neighbor_num + recent_sample_single_hop_kernel
 * and static_neighbor_num + uniform_sample_single_hop_kernel plus the thrust
 * scans between them (sample.cu.hpp:706-827, 1569-1687).
 * A slot whose node lies outside [0,n) is sampled as empty and counted in
 * counts[2] (the caller turns a non-zero count into SGL_ERANGE). */
size_t  sgl_sample_hop_workspace_bytes(int64_t S_max);
int32_t sgl_sample_hop(const sgl_tcsr* g,
                       const int64_t* slot_node, const int64_t* slot_ts,
                       int64_t S_max, const int64_t* S_dev,
                       const sgl_sample_params* p, const sgl_hop_out* out,
                       void* workspace, size_t workspace_bytes, void* stream);

/* sgl_sample_hop for callers that cannot allocate device memory and have no
 * workspace to pass (code under HIP-graph capture, tight serving loops,
 * harnesses that forbid hipMalloc).  It has no counterpart in the reference.
 * Same arguments and results as sgl_sample_hop, without the workspace: the
 * hop's scratch (window starts / lengths per slot, per-block sums) is an array
 * of sgl_sample_hop_workspace_bytes(SGL_STATIC_HOP_MAX_SLOTS) bytes (about
 * 1.1 MB) inside the library image, one copy per GPU, held until the process
 * ends.  S_max > SGL_STATIC_HOP_MAX_SLOTS is refused with SGL_ENOMEM.  The
 * call allocates and frees nothing.  All calls on one GPU share that GPU's
 * array: calls that overlap on one GPU (different streams, or host threads on
 * different streams) race; order them on one stream or with events.  The
 * first call on a device looks the array's address up (no allocation); make
 * that call outside a stream capture. */
#define SGL_STATIC_HOP_MAX_SLOTS 65536
int32_t sgl_sample_hop_static(const sgl_tcsr* g,
                              const int64_t* slot_node, const int64_t* slot_ts,
                              int64_t S_max, const int64_t* S_dev,
                              const sgl_sample_params* p, const sgl_hop_out* out,
                              void* stream);

/* Whole-window sampling: every edge of a slot's time window, or the first k,
 * optionally only those carrying a given tag.  Replaces the 'full' and
 * 'cluster' layer types and the discrete-time branch of the offline sampler
 * (_jit_sample_kernel, prepare_sample.py:32-172; cut_idx / start_idx :50-55,
 * continuous cluster/full :62, :112-113, :131-132; discrete :65-76, :147-170).
 * Window of a slot (v, t): edges e of row v with
 *   (bounded_below ? t + lo_offset : -inf) <= ts[e] < t + hi_offset,
 * candidates: all of them, or those with edge_tag[e] == tag_value when
 * edge_tag != NULL ([m] device, in T-CSR order); taken: the first
 * min(first_k, candidates) in storage order (first_k < 0: all).
 * neighbors_ts = t when keep_slot_time (discrete snapshots) else ts[e];
 * neighbors_dt = ts[e] - t.  Result layout as sgl_hop_out.
 * The edge count is not bounded beforehand: called with out->neighbors ==
 * NULL the function only counts (root_start_ptr, root_end_ptr and counts are
 * written; counts[1] = E); the caller then allocates E edges and calls again.
 * Should capacity_edges of that second call be below E, counts[2] reads
 * INT64_MAX and the edge arrays are void. */
typedef struct sgl_window_params {
    int64_t        lo_offset, hi_offset;
    int32_t        bounded_below;
    int32_t        keep_slot_time;
    int64_t        first_k;
    const int64_t* edge_tag;   /* device [m] or NULL */
    int64_t        tag_value;
} sgl_window_params;
size_t  sgl_sample_window_workspace_bytes(int64_t S);
int32_t sgl_sample_window(const sgl_tcsr* g, const int64_t* slot_node,
                          const int64_t* slot_ts, int64_t S,
                          const sgl_window_params* p, const sgl_hop_out* out,
                          void* workspace, size_t workspace_bytes, void* stream);

/* k-hop driver (replaces Graph::sample_src_in_chunks_khop,
 * sample.cu.hpp:1532-1716).  Hop-0 slots are the positive roots expanded over
 * their timestamps (root r owns root_ts[ts_ptr[r]..ts_ptr[r+1])) followed by
 * the negative roots; they are written to slot_node0/slot_ts0
 * ([S_pos + N_neg] each).  Hop l+1 slots are hop l's (neighbors, neighbors_ts),
 * one slot per sampled edge, no dedup between hops.  p->hop is ignored; hop l
 * draws from RNG stream l.  outs[l].capacity_slots must be >= the worst-case
 * slot count of hop l ((S_pos+N_neg) * fanout^l).
 * Two-hop calls of up to 32768 root slots and fanout <= 16 run as one launch
 * whose blocks wait (bounded, sgl_set_wait_limit) for the edge totals of the
 * blocks before them; should a block ever give up, outs[0].counts[2] reads
 * INT64_MAX and the outputs of the call are void (a remap state named by
 * mark_state is then marked void as well: the next sgl_unique_compact on it
 * reports INT64_MAX until sgl_remap_init).  The same call with
 * SGL_SAMPLE_MULTI_LAUNCH in p->flags cannot give up. */
size_t  sgl_sample_khop_workspace_bytes(int64_t S0, int32_t layers,
                                        int32_t fanout);
int32_t sgl_sample_khop(const sgl_tcsr* g,
                        int64_t R, const int64_t* roots, const int64_t* ts_ptr,
                        int64_t S_pos, const int64_t* root_ts,
                        int64_t N_neg, const int64_t* neg_roots,
                        const int64_t* neg_ts,
                        int32_t layers, const sgl_sample_params* p,
                        int64_t* slot_node0, int64_t* slot_ts0,
                        const sgl_hop_out* outs,
                        void* workspace, size_t workspace_bytes, void* stream);

/* Q k-hop calls over the same roots in one library call: query q samples with
 * p[q] into outs[q * layers + l], l < layers; slot_node0/slot_ts0 are written
 * once (all queries expand the same roots).  This is what a loader issues when
 * one mini-batch is sampled under several policies - the reference submits them
 * one after the other (AsyncGraphBlob, graph.py:274-293; Graph::submit_query,
 * sample.cu.hpp:1903-1928).  Results equal those of Q sgl_sample_khop calls;
 * a most-recent and a uniform 2-hop query of at most 32768 root slots and
 * fanout <= 16 run side by side in one kernel launch.  The workspace is
 * sgl_sample_khop_multi_workspace_bytes(S0, layers, largest fanout, Q). */
size_t  sgl_sample_khop_multi_workspace_bytes(int64_t S0, int32_t layers,
                                              int32_t fanout, int32_t Q);
int32_t sgl_sample_khop_multi(const sgl_tcsr* g,
                              int64_t R, const int64_t* roots, const int64_t* ts_ptr,
                              int64_t S_pos, const int64_t* root_ts,
                              int64_t N_neg, const int64_t* neg_roots,
                              const int64_t* neg_ts,
                              int32_t layers, int32_t Q, const sgl_sample_params* p,
                              int64_t* slot_node0, int64_t* slot_ts0,
                              const sgl_hop_out* outs,
                              void* workspace, size_t workspace_bytes, void* stream);

/* B mini-batches sampled by ONE k-hop launch sequence, per-batch results
 * addressable on the device.  The reference keeps several windows in flight at
 * once - AsyncGraphBlob submits one query per window (graph.py:274-293),
 * AsyncTemporalSampler::submit_query queues them (sample.cu.hpp:1990-2020),
 * the loader prefetches (`prefetch_factor`, test/test.py:212-221) - but runs
 * them one after the other; a 12 000-root query is bound by launch floors and
 * by its chain of dependent loads, B of them in one call are bound by
 * throughput.
 *   slot_node/slot_ts [S_max]  the hop-0 slots of all batches, batch after
 *                              batch (per batch: its positive root timestamps,
 *                              then its negatives, as sgl_sample_khop lays
 *                              them out);
 *   batch_ptr  device int64[B+1], ascending: batch b owns the slots
 *              [batch_ptr[b], batch_ptr[b+1]); batch_ptr[B] <= S_max is the
 *              live slot count (trailing batches may be empty);
 *   slot_hint  optional device int64[S_max]: where slot s's window ends
 *              (sgl_window_end), -1 = search; used when equal_root_time == 0;
 *   p[q], outs[q * layers + l]  Q queries over the same slots, as
 *              sgl_sample_khop_multi (mark_state must be NULL: the batches
 *              have id spaces of their own, see sgl_unique_compact_batched).
 * The result equals ONE sgl_sample_khop call whose root slots are slot_node /
 * slot_ts (the generator of the uniform strategy is keyed by the slot's index
 * in the whole call); for the most-recent strategy that is the concatenation
 * of the batches' own results.
 *   seg  device int64[Q][layers+1][B+1]: seg[q][0][b] = batch_ptr[b];
 *        seg[q][l+1][b] = outs[q*layers+l].root_start_ptr[seg[q][l][b]], i.e.
 *        batch b owns the edges [seg[q][l+1][b], seg[q][l+1][b+1]) of hop l
 *        (which are the slots of hop l+1).
 * Always the launch-per-hop route (nothing waits for another block). */
size_t  sgl_sample_khop_batched_workspace_bytes(int64_t S_max, int32_t layers,
                                                int32_t fanout, int32_t Q);
int32_t sgl_sample_khop_batched(const sgl_tcsr* g, int32_t B,
                                const int64_t* batch_ptr, int64_t S_max,
                                const int64_t* slot_node, const int64_t* slot_ts,
                                const int64_t* slot_hint,
                                int32_t layers, int32_t Q,
                                const sgl_sample_params* p,
                                const sgl_hop_out* outs, int64_t* seg,
                                void* workspace, size_t workspace_bytes,
                                void* stream);

/* ------------------------------------------------------ unique / compaction */
#define SGL_UNIQUE_SORTED  0 /* all arrays form one group: == np.unique(return_inverse) */
#define SGL_UNIQUE_GROUPED 1 /* per array: ids new to the epoch, ascending, appended    */
#define SGL_UNIQUE_MULTI_LAUNCH 0x200 /* flag: the numbering pass of a dense state never exchanges counts
                                      * inside one launch (no bounded wait); for re-issuing a call whose
                                      * U_dev[0] read INT64_MAX, after sgl_remap_init                    */
#define SGL_UNIQUE_PREMARKED 0x100 /* flag, with SGL_UNIQUE_SORTED, reset = 1 and a dense state:
                                    * the sampler has already recorded the arrays' ids as
                                    * pending (sgl_sample_params.mark_state)              */

/* Persistent remap state over a dense id universe [0, universe): the
 * replacement of Remapper's id_mapper/global_mask tables and epoch counter
 * (sample.cu.hpp:1752-1763).  The caller allocates sgl_remap_state_bytes()
 * device bytes and calls sgl_remap_init once. */
size_t  sgl_remap_state_bytes(int64_t universe);
int32_t sgl_remap_init(void* state, size_t state_bytes, int64_t universe,
                       void* stream);

/* Rewrite G id arrays to dense local ids and emit the local->global table
 * (replaces Remapper::insert / remapper + mark_new_ids_kernel +
 * update_new_ids_kernel, sample.cu.hpp:1719-1854; np.unique /
 * _merge_and_map_nodes in prepare_sample.py:205-246).
 *   ids[g]       device array of len_max[g] ids; the live length is
 *                *len_dev[g] when len_dev != NULL && len_dev[g] != NULL.
 *   local_out[g] same shape as ids[g] (may alias ids[g]).
 *   reset        1: start a new local-id epoch (numbering restarts at 0);
 *                0: continue the epoch of the previous call on `state`.
 *   unique_out   local -> global; entries [U_before, U_total) are written.
 *   U_dev        device int64[2] = {U_total, U_before}.  U_total reads INT64_MAX
 *                when a numbering pass of this or an earlier call on the state
 *                gave up its bounded wait for another block: the result is void
 *                and the state must be initialised again.
 * `state` != NULL selects the dense-universe path: `universe` must be the value
 * given to sgl_remap_init, ids outside [0, universe) map to -1.  `state` ==
 * NULL (universe ignored) selects the one-shot hash-set path, which accepts
 * arbitrary non-negative ids but only reset = 1 (its table lives in the
 * workspace; sgl_unique_compact_hashed keeps one over several calls).
 * Negative ids always map to -1.  Both paths are asynchronous, fixed launch
 * sequences. */
size_t  sgl_unique_workspace_bytes(int64_t universe, int32_t G,
                                   const int64_t* len_max);
int32_t sgl_unique_compact(void* state, int64_t universe, int32_t reset,
                           int32_t mode, int32_t G, const int64_t* const* ids,
                           const int64_t* len_max,
                           const int64_t* const* len_dev,
                           int64_t* const* local_out,
                           int64_t* unique_out, int64_t unique_capacity,
                           int64_t* U_dev,
                           void* workspace, size_t workspace_bytes,
                           void* stream);

/* Persistent hash-set remap state for ids without a dense universe (arbitrary
 * non-negative 63-bit values, e.g. DistRouteIndex-encoded ids): the same role
 * as sgl_remap_init's state - Remapper's id_mapper and epoch counter
 * (sample.cu.hpp:1752-1763), which the reference keeps per graph so that the
 * queries of one AsyncGraphBlob share one numbering ('r' then 'f',
 * graph.py:291) - with memory proportional to `capacity`, the largest number
 * of distinct ids one epoch may hold (at most 2^31 - 256), instead of to the
 * id range.  The caller allocates sgl_remap_hashed_state_bytes(capacity)
 * device bytes (about 22 bytes per id) and calls sgl_remap_hashed_init once. */
size_t  sgl_remap_hashed_state_bytes(int64_t capacity);
int32_t sgl_remap_hashed_init(void* state, size_t state_bytes, int64_t capacity,
                              void* stream);

/* sgl_unique_compact over a hashed state: same arguments, modes and results
 * (Remapper::insert, sample.cu.hpp:1825-1852), with `capacity` - the value
 * given to sgl_remap_hashed_init - in place of the universe; reset = 0
 * continues the epoch of the previous call on the state.  No host
 * synchronisation.  When an epoch outgrows the capacity U_dev[0] reads
 * INT64_MAX from then on: the result is void and the state must be
 * initialised again (with a larger capacity). */
size_t  sgl_unique_hashed_workspace_bytes(int64_t capacity, int32_t G,
                                          const int64_t* len_max);
int32_t sgl_unique_compact_hashed(void* state, int64_t capacity, int32_t reset,
                                  int32_t mode, int32_t G,
                                  const int64_t* const* ids,
                                  const int64_t* len_max,
                                  const int64_t* const* len_dev,
                                  int64_t* const* local_out,
                                  int64_t* unique_out, int64_t unique_capacity,
                                  int64_t* U_dev,
                                  void* workspace, size_t workspace_bytes,
                                  void* stream);

/* Unique + compaction of B mini-batches, each with a local-id space of its
 * own, in one launch sequence (the loader's batches are independent: every one
 * starts a new epoch, Remapper with op 'r', sample.cu.hpp:1825-1852; np.unique
 * per batch in prepare_sample.py:205-213).  The state spans B copies of the
 * universe [0, universe) (B <= SGL_BATCH_MAX); every call starts a new epoch.
 * The caller allocates sgl_remap_batched_state_bytes(universe, B) device bytes,
 * 16-byte aligned (about 1.25 bytes per id of B x universe up to 2^26 ids in
 * all, 0.4 beyond), and calls sgl_remap_batched_init once.
 *   ids[g] / local_out[g]  G arrays of len_max[g] entries holding all batches;
 *   seg[g]     device int64[B+1]: elements [seg[g][b], seg[g][b+1]) of array g
 *              belong to batch b (seg[g][B] = live length <= len_max[g]) -
 *              what sgl_sample_khop_batched writes per hop;
 *   unique_out batch b's distinct ids, ascending, at [U_off[b], U_off[b+1]);
 *   U_off      device int64[B+1], U_off[B] = number of rows of unique_out;
 *   local_out  position of the id in its batch's list (-1 for ids outside
 *              [0, universe)).
 * Per batch this is sgl_unique_compact(..., reset = 1, SGL_UNIQUE_SORTED) over
 * the batch's slices. */
#define SGL_BATCH_MAX 64
size_t  sgl_remap_batched_state_bytes(int64_t universe, int32_t B);
int32_t sgl_remap_batched_init(void* state, size_t state_bytes, int64_t universe,
                               int32_t B, void* stream);
size_t  sgl_unique_batched_workspace_bytes(int64_t universe, int32_t B);
int32_t sgl_unique_compact_batched(void* state, int64_t universe, int32_t B,
                                   int32_t G, const int64_t* const* ids,
                                   const int64_t* len_max,
                                   const int64_t* const* seg,
                                   int64_t* const* local_out,
                                   int64_t* unique_out, int64_t unique_capacity,
                                   int64_t* U_off,
                                   void* workspace, size_t workspace_bytes,
                                   void* stream);

/* ------------------------------------------------------------ cache gather */
/* Two-tier row store (replaces IDMapper.to_local + DistNodeState.__getitem__,
 * starrygl/utils/partition_book.py:106-133, starrygl/cache/NodeState.py:36-44,
 * and tensor_gather / ShardTensor, csrc/include/starrygl/feature.cu.hpp:42-88,
 * 236-422).  Lookup of a requested id:
 *   key  = id & id_mask                      (id_mask = -1: use the id as is;
 *                                             0xFFFFFFFFFFFF: DistRouteIndex.loc)
 *   loc  = g2l ? g2l[key] : key              (-1 / out of range = not resident)
 *   slot = hot_slot ? hot_slot[loc] : loc    (>= 0: row `slot` of `hot`,
 *                                             < 0 : row `loc` of `cold`)
 * A non-resident id yields an all-zero row, out_ts = 0 and bumps stats[2].
 * The two strides let the cold tier keep a row and its time in one record
 * (cold = base, ts_cold = base + row_bytes, both strides = the record size, best
 * a multiple of 128): reads over PCIe are paid for in whole 128-byte lines, and
 * an 8-byte time in a table of its own costs as much as a third of a 400-byte row. */
typedef struct sgl_cache {
    int64_t        rows;      /* logical (local) rows                          */
    int64_t        row_bytes; /* multiple of 4                                 */
    int64_t        id_mask;
    const int64_t* g2l;       /* device [g2l_len] or NULL                      */
    int64_t        g2l_len;
    const int32_t* hot_slot;  /* device [rows] or NULL                         */
    const void*    hot;       /* device (HBM) [hot_rows, row_bytes]            */
    int64_t        hot_rows;
    const void*    cold;      /* device-visible pinned host [rows, row_bytes]  */
    const int64_t* ts_hot;    /* optional last-update time per hot row         */
    const int64_t* ts_cold;   /* optional last-update time per logical row     */
    int64_t        cold_stride;    /* bytes from one cold row to the next; 0 = row_bytes (a
                                    * multiple of 4, >= row_bytes)                       */
    int64_t        ts_cold_stride; /* bytes from one ts_cold entry to the next; 0 = 8 (a
                                    * multiple of 8)                                     */
    int64_t        hot_stride;     /* bytes from one hot row to the next; 0 = row_bytes (a
                                    * multiple of 4, >= row_bytes): a view of some columns of
                                    * wider HBM rows, e.g. the memory part of rows that hold a
                                    * node's memory and its features side by side          */
} sgl_cache;

/* out[i, :] = row(ids[i]); out_ts[i] = its last-update time when out_ts and the
 * tier's ts table are non-NULL.  N = *N_dev when N_dev != NULL (<= N_max).
 * stats (optional device int64[3]) += {hot hits, cold hits, absent}. */
int32_t sgl_gather(const sgl_cache* c, const int64_t* ids, int64_t N_max,
                   const int64_t* N_dev, void* out, int64_t* out_ts,
                   int64_t* stats, void* stream);

/* Several gathers in ONE launch (up to SGL_GATHER_MAX_SEGMENTS): each segment is
 * what one sgl_gather call takes.  A training step gathers node features, memory
 * rows and the edge features of every hop; on small batches each launch costs
 * more than its copy, and host-tier segments overlap their PCIe latency with the
 * HBM segments.  Every row size must be a multiple of 16 bytes and every table
 * and output 16-byte aligned (SGL_ENOTSUP otherwise: use sgl_gather). */
#define SGL_GATHER_MAX_SEGMENTS 8
typedef struct sgl_gather_seg {
    const sgl_cache* cache;
    const int64_t*   ids;
    int64_t          N_max;
    const int64_t*   N_dev;   /* optional device live count */
    void*            out;
    int64_t*         out_ts;  /* optional */
} sgl_gather_seg;
int32_t sgl_gather_multi(int32_t num_segments, const sgl_gather_seg* segs,
                         void* stream);

/* sgl_gather with every distinct cold row crossing PCIe once.  The requests of
 * a batch repeat rows (configs of 40 % duplicates and more); sgl_gather reads a
 * cold row from pinned host memory once per REQUEST.  Here the call first
 * numbers the distinct cold rows it asks for (the LDS-staged hash set of
 * sgl_unique_compact), fetches each of them once into `staging` (HBM,
 * [staging_rows, row_bytes]; and its time into staging_ts when the cache has
 * ts_cold and out_ts is wanted), overlapped with the gather of the hot rows,
 * and then serves every request of a cold row from there.  This is the plan of
 * the reference's per-shard selected-index lists (ShardTensor::operator[],
 * feature.cu.hpp:346-392) and of DistNodeState.prefetch (NodeState.py:77-82),
 * which index the host table once per request.  Results equal sgl_gather's.
 * Distinct cold rows beyond staging_rows are read in place, once per request.
 * stats (optional device int64[4]) += {hot requests, cold requests, absent,
 * distinct cold rows}.  Rows, tables, out and staging must be 16-byte aligned /
 * sized (SGL_ENOTSUP otherwise: use sgl_gather). */
size_t  sgl_gather_dedup_workspace_bytes(int64_t N_max);
int32_t sgl_gather_dedup(const sgl_cache* c, const int64_t* ids, int64_t N_max,
                         const int64_t* N_dev, void* out, int64_t* out_ts,
                         int64_t* stats, void* staging, int64_t* staging_ts,
                         int64_t staging_rows, void* workspace,
                         size_t workspace_bytes, void* stream);

/* Scatter rows back (replaces DistNodeState.update, NodeState.py:46-61):
 * ids that are not resident are skipped.  Duplicate ids: the highest i wins
 * is NOT guaranteed; callers pass unique ids (as the reference's callers do). */
int32_t sgl_scatter_update(const sgl_cache* c, void* hot_rw, void* cold_rw,
                           int64_t* ts_hot_rw, int64_t* ts_cold_rw,
                           const int64_t* ids, int64_t N,
                           const void* values, const int64_t* ts,
                           void* stream);

/* ------------------------------------------------------- chunks and seeds */
/* Nodes grouped by chunk: chunk c owns chunk_nodes[chunk_ptr[c] ..
 * chunk_ptr[c+1]), node ids ascending (replaces chunk_ptr_/row_idx_ of `Graph`,
 * sample.cu.hpp:1053-1065, 1135-1146).  Synchronous; SGL_ERANGE when a node's
 * chunk id is outside [0, num_chunks) (sample.cu.hpp:1059-1062). */
size_t  sgl_chunk_index_workspace_bytes(int64_t n);
int32_t sgl_chunk_index_build(int64_t n, int64_t num_chunks,
                              const int64_t* node_chunk, int64_t* chunk_ptr,
                              int64_t* chunk_nodes, void* workspace,
                              size_t workspace_bytes, void* stream);

/* Seed (root) extraction: every node of the selected chunks that has at least
 * one out-edge with t_begin <= ts < t_end becomes a root, in the order of
 * `chunks` and by ascending node id inside a chunk.  Per root: its distinct
 * event timestamps inside the window (ts, delimited by ts_ptr) and per
 * timestamp the ids of the events at that (node, timestamp) (q_eid, delimited
 * by q_ptr).  Replaces Graph::get_seeds_in_chunks with filter_seeds_kernel /
 * collect_seeds_kernel (sample.cu.hpp:517-705, 1303-1449).
 * cand_off is the exclusive prefix of the selected chunks' sizes
 * (cand_off[num_chunks] = n_cand).  Two calls sharing one workspace:
 *   sgl_seeds_count -> totals[0..2] = {R roots, S timestamps, Q events};
 *   (caller allocates roots[R], ts_ptr[R+1], ts[S], q_ptr[S+1], q_eid[Q])
 *   sgl_seeds_fill.
 * window_end (optional, [S] or NULL; no counterpart in the reference): per
 * (root, timestamp) the position of the root's first edge at that time, i.e.
 * what sgl_window_end gives for it - the extraction walks those edges anyway -
 * ready to be passed on as sgl_sample_params.root_hint. */
typedef struct sgl_seed_query {
    const int64_t* chunk_ptr;   /* device [total chunks + 1]          */
    const int64_t* chunk_nodes; /* device [n]                          */
    int64_t        num_chunks;  /* selected chunks                     */
    const int64_t* chunks;      /* device [num_chunks] chunk ids       */
    const int64_t* cand_off;    /* device [num_chunks + 1]             */
    int64_t        n_cand;
    int64_t        t_begin, t_end;
} sgl_seed_query;

size_t  sgl_seeds_workspace_bytes(int64_t n_cand);
int32_t sgl_seeds_count(const sgl_tcsr* g, const sgl_seed_query* q,
                        int64_t* totals, void* workspace,
                        size_t workspace_bytes, void* stream);
int32_t sgl_seeds_fill(const sgl_tcsr* g, const sgl_seed_query* q,
                       const int64_t* totals,
                       int64_t* roots, int64_t* ts_ptr, int64_t* ts,
                       int64_t* q_ptr, int64_t* q_eid, int64_t* window_end,
                       void* workspace, size_t workspace_bytes, void* stream);

/* ------------------------------------------- sub-graph slice ("cluster" mode) */
/* The sub-graph of a chunk set over a time window (replaces
 * count_edges_kernel / write_edges_kernel / mark_chunks_exists_kernel and
 * Graph::slice_by_chunk_ts, sample.cu.hpp:115-120, 299-515, 1189-1299; the
 * 'cluster' branch of the query worker, :1953-1961).  Candidates and window
 * as for the seeds: the nodes of the selected chunks in chunk-list order, edges
 * with t_begin <= ts < t_end.  A candidate with a non-empty window becomes a
 * node of the slice; of its window edges those whose destination lies in a
 * selected chunk (node_chunk[col[e]] selected) are kept, in storage order.
 *   nodes[R], ts_ptr[R+1] : slice nodes and their ranges in ts[]
 *   ts[T], edge_ptr[T+1]  : per node a list of timestamps; entry s owns the
 *                           kept edges [edge_ptr[s], edge_ptr[s+1]), exactly
 *                           those kept edges of the node with timestamp ts[s]
 *   col/col_ts/col_eid[E] : the kept edges
 * full_timestamps == 0: ts[] lists the distinct timestamps of the node's window
 * edges (kept or not).  full_timestamps == 1 (discrete-time snapshots, what the
 * query worker asks for): every node lists all integers t_begin .. t_end-1, so
 * T = R * (t_end - t_begin).
 *   sgl_slice_count -> totals[0..2] = {R, T, E};   (caller allocates)
 *   sgl_slice_fill.
 * node_chunk: device [g->n] chunk id of every node, in [0, total_chunks); NULL
 * keeps every window edge (no destination filter), which with
 * full_timestamps = 1 is get_seeds_in_chunks' using_full_timestamp mode
 * (filter_seeds_kernel, sample.cu.hpp:575-578): nodes/ts_ptr/ts are the roots,
 * edge_ptr/col_eid their q_ptr/q_eid. */
size_t  sgl_slice_workspace_bytes(int64_t n_cand, int64_t total_chunks);
int32_t sgl_slice_count(const sgl_tcsr* g, const sgl_seed_query* q,
                        const int64_t* node_chunk, int64_t total_chunks,
                        int32_t full_timestamps, int64_t* totals,
                        void* workspace, size_t workspace_bytes, void* stream);
int32_t sgl_slice_fill(const sgl_tcsr* g, const sgl_seed_query* q,
                       const int64_t* node_chunk, int64_t total_chunks,
                       int32_t full_timestamps, const int64_t* totals,
                       int64_t* nodes, int64_t* ts_ptr, int64_t* ts,
                       int64_t* edge_ptr, int64_t* col, int64_t* col_ts,
                       int64_t* col_eid, void* workspace,
                       size_t workspace_bytes, void* stream);

/* --------------------------------------------------------- block building */
/* Message-flow block of one layer in CSC form (replaces the tensor algebra of
 * AsyncBlock.to_block, starrygl/graph/graph.py:153-271, and
 * _build_csc_from_pairs, prepare_sample.py:215-229).  The layer has S slots
 * (= its destination nodes dst_offset .. dst_offset+S-1 of num_dst) and E
 * sampled edges; source node of edge e is src_offset + e.
 *   indptr[0 .. num_dst]   : 0 for dst < dst_offset, root_start_ptr beyond
 *   indices[e]             : src_offset + e
 *   edge_dst[e] (optional) : dst_offset + slot of e   (COO destination)
 * S, E are read from counts[0], counts[1] of the hop (device). */
int32_t sgl_block_build(const int64_t* root_start_ptr, const int64_t* counts,
                        int64_t S_max, int64_t E_max, int64_t dst_offset,
                        int64_t src_offset, int64_t* indptr, int64_t* indices,
                        int64_t* edge_dst, void* stream);

/* ------------------------------------------------ batch materialisation */
/* np.unique over (id, timestamp) records with return_inverse (replaces
 * _get_unique_pairs and, over the concatenation of two lists,
 * _merge_and_map_nodes, prepare_sample.py:205-213, 231-246): uniq_ids/uniq_ts
 * [U] ascend in (id, ts), signed order; inverse[i] is the place of pair i in
 * them; U_dev[0] = U.  Capacity of the three outputs: N_max.  N = *N_dev when
 * given. */
size_t  sgl_unique_pairs_workspace_bytes(int64_t N_max);
int32_t sgl_unique_pairs(const int64_t* ids, const int64_t* ts, int64_t N_max,
                         const int64_t* N_dev, int64_t* uniq_ids,
                         int64_t* uniq_ts, int64_t* inverse, int64_t* U_dev,
                         void* workspace, size_t workspace_bytes, void* stream);

/* Edge order and pointer array of a CSC block from (destination, timestamp)
 * pairs (replaces _build_csc_from_pairs, prepare_sample.py:215-229): perm is
 * the stable order np.lexsort((ts, dst_local)), indptr[d] the number of edges
 * with destination below d (d = 0 .. num_dst).  dst_local must lie in
 * [0, num_dst).  E = *E_dev when given. */
size_t  sgl_csc_from_pairs_workspace_bytes(int64_t E_max);
int32_t sgl_csc_from_pairs(const int64_t* dst_local, const int64_t* ts,
                           int64_t E_max, const int64_t* E_dev,
                           int64_t num_dst, int64_t* indptr, int64_t* perm,
                           void* workspace, size_t workspace_bytes,
                           void* stream);

/* -------------------------------------------------- latest event per node */
/* For N events with dense keys local[i] in [0, U) (local ids from
 * sgl_unique_compact) and timestamps ts[i]: max_ts[u] = max of ts over the
 * events of key u, arg[u] = the smallest event index attaining it (first
 * occurrence wins ties, as torch_scatter.scatter_max does on the CPU); keys
 * without events get max_ts = INT64_MIN, arg = -1.  Events with local[i]
 * outside [0, U) are ignored.  Replaces index.unique + scatter_max of
 * mailbox.get_update_mail / set_mailbox_local
 * (starrygl/nn/memory/mailbox.py:41-47, 78-83).  N = *N_dev, U = *U_dev when
 * given (<= N_max, U_max). */
int32_t sgl_segment_max_ts(const int64_t* local, const int64_t* ts,
                           int64_t N_max, const int64_t* N_dev,
                           int64_t U_max, const int64_t* U_dev,
                           int64_t* max_ts, int64_t* arg, void* stream);

/* ----------------------------------------------------------- time encoding */
#define SGL_DT_I64 0
#define SGL_DT_F32 1
/* out[i, j] = cos(fl32(fl32(w[j] * float(dt[i])) + b[j])), fp32, no FMA
 * contraction (replaces TimeEncoder.forward,
 * starrygl/nn/model/time_encoder.py:29-31). */
int32_t sgl_time_encode(const void* dt, int32_t dt_dtype, int64_t N_max,
                        const int64_t* N_dev, const float* w, const float* b,
                        int32_t dim, float* out, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* SGL_HOT_H */
