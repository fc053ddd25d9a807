/*
 * hira_hip.h -- C ABI of libhira_hip.so: the MI355X (gfx950) range-search sparse-attention
 * hot path: ball-tree index build / append, halfspace tree search, sparse attention.
 *
 * Conventions
 *   - Every pointer is a DEVICE pointer unless its name ends in _host.  The caller owns
 *     all memory; the library allocates nothing and keeps no state between calls
 *     (except the thread-local text returned by hira_last_error).
 *   - Every call only ENQUEUES work on `stream` (a hipStream_t passed as void*) and
 *     returns; calls that touch the same tree must be ordered by the caller (same stream).
 *   - Return value: 0 on success, a negative HIRA_E* code otherwise.
 *   - dtype: HIRA_F32 or HIRA_BF16; it is the storage type of keys, values, centers and
 *     queries.  All arithmetic accumulates in fp32.
 *
 * Tree layout (depth-generic, fixed fan-out; the layout of the reference's GPU indexer,
 * indexer/cuda.py:338-357, 439-446, generalised to any depth and to many trees):
 *   level 0 = keys; level l >= 1 = ball centers + radii.  The children of node p of
 *   level l+1 are the slots [p*bf, (p+1)*bf) of level l, filled from slot 0;
 *   counts[l+1][p] says how many are in use.  size[l] = slots of level l that may be in
 *   use (size[l] <= size[l+1]*bf), cap[l] = allocated slots per tree (row stride between
 *   trees).  A node without children has radius -inf.  perm maps a key slot to the
 *   position of that key in the order it was given to the index (-1 for an empty slot).
 */
#ifndef HIRA_HIP_H
#define HIRA_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define HIRA_ABI_VERSION 7
#define HIRA_MAX_LEVELS 8
#define HIRA_STATS_COLS (HIRA_MAX_LEVELS + 3) /* counters per tree a search can fill in */

enum { HIRA_F32 = 0, HIRA_BF16 = 1 };

/* How the keys and the centers of every level are stored inside one tree's (cap, D)
 * matrix.  HIRA_TILE16 (bf16 only, D a multiple of 32, every cap a multiple of 16): rows
 * are grouped in tiles of 16, columns in steps of 32; the 16-byte chunk holding columns
 * [32 s + 8 kb, +8) of row 16 tile + i sits at chunk index (tile*(D/32) + s)*64 + kb*16 + i,
 * i.e. one wave-wide 128-bit load fetches a complete 16x32 MFMA operand tile from 1 KiB of
 * contiguous memory.  Values, radii, counts and perm are never tiled. */
enum { HIRA_ROW_MAJOR = 0, HIRA_TILE16 = 1, HIRA_TILE16_Q8 = 2 };
/* HIRA_TILE16_Q8 (bf16 only, D = 64 or 128, every cap a multiple of 16): the centers of
 * every level are tiled as in HIRA_TILE16, the keys are ROW-MAJOR, and beside them sits an
 * 8-bit shadow copy `keys8` that the search scans first: k8 = round(k / kscale[channel]),
 * clipped to [-127, 127], with one step `kscale` per tree and channel, in tiles of 16 rows x
 * 64 columns -- the 16-byte chunk holding columns [64 s + 16 kb, +16) of row 16 tile + i sits
 * at chunk index (tile*(D/64) + s)*64 + kb*16 + i, one wave-wide 128-bit load per 16x64 tile.
 * keps[node] bounds |k/kscale - k8| over all channels of all keys of level-1 node `node`
 * (0.5 unless a key appended later clipped).  A key whose 8-bit score plus the error bound
 * these numbers give stays below the threshold cannot be selected; only the others have
 * their bf16 row fetched and tested exactly, so the selected set is that of the other
 * layouts bit for bit. */

enum {
    HIRA_OK = 0,
    HIRA_EINVAL = -1,   /* bad shape / dtype / null pointer: the message names it */
    HIRA_ELAUNCH = -2,  /* the HIP runtime refused a launch */
    HIRA_EWORKSPACE = -3 /* workspace too small */
};

typedef struct HiraTree {
    int32_t num_trees;  /* T = sequences x KV heads; one independent tree each */
    int32_t num_levels; /* L >= 1 (L = 1: keys only, every search is a flat scan) */
    int32_t bf;         /* fan-out, 1..64 */
    int32_t dim;        /* key / query / center dim D; D*elem_size a multiple of 16 B */
    int32_t vdim;       /* value dim Dv (0 if there are no values) */
    int32_t dtype;
    int32_t layout;     /* HIRA_ROW_MAJOR, HIRA_TILE16 or HIRA_TILE16_Q8 */
    int32_t reserved_;  /* keeps the arrays below 8-byte aligned; must be 0 */
    int32_t size[HIRA_MAX_LEVELS];
    int32_t cap[HIRA_MAX_LEVELS];
    void* keys;                      /* (T, cap[0], D), stored as `layout` says */
    void* values;                    /* (T, cap[0], Dv) or NULL */
    int32_t* perm;                   /* (T, cap[0]) */
    void* centers[HIRA_MAX_LEVELS];  /* [l >= 1] (T, cap[l], D), stored as `layout` says */
    float* radii[HIRA_MAX_LEVELS];   /* [l >= 1] (T, cap[l]) */
    int32_t* counts[HIRA_MAX_LEVELS];/* [l >= 1] (T, cap[l]) */
    /* HIRA_TILE16_Q8 only (NULL otherwise): */
    int8_t* keys8;                   /* (T, cap[0], D) 8-bit shadow of the keys, tiled 16 x 64 */
    float* kscale;                   /* (T, D) step of the shadow per tree and channel */
    float* keps;                     /* (T, cap[1]) largest rounding/clipping error, in steps,
                                        among the keys of each level-1 node */
} HiraTree;

/* One decode step's queries.  Query head h belongs to tree q2tree order given as CSR:
 * the heads of tree t are tree_q_heads[tree_q_off[t] .. tree_q_off[t+1]).  This carries
 * the reference's q_head_to_kv map (searcher/cpu.py:103-109, searcher/cuda.py:23-33),
 * including maps that are not monotone (tests/test_cpp_kernels.py:529-565). */
typedef struct HiraQuery {
    int32_t num_q_heads;         /* H_q (all sequences) */
    const void* q;               /* (H_q, D), tree dtype */
    const float* tau;            /* (H_q) threshold on the raw score q.k */
    const float* scaling;        /* (H_q) factor applied to returned scores / softmax logits */
    const int32_t* tree_q_off;   /* (T+1) */
    const int32_t* tree_q_heads; /* (H_q) */
    int32_t max_group;           /* max heads of one tree (host knows it) */
    int32_t group_size;          /* > 0: the default map, head h belongs to tree
                                    h / group_size (H_q = T * group_size); the kernels then
                                    skip the CSR lookup.  0: use the CSR above. */
} HiraQuery;

/* Keys/values that are cached but not yet in the index (the reference's decode queue,
 * cache/hira_cache.py:121-140): attention always attends to all of them. */
typedef struct HiraQueue {
    const void* keys;   /* (T, cap, D) or NULL */
    const void* values; /* (T, cap, Dv) */
    int32_t len;        /* rows in use per tree */
    int32_t cap;
} HiraQueue;

/* What a search writes.  Any of the three groups may be absent (NULL pointers). */
typedef struct HiraSearchOut {
    /* (1) dense scores, the reference's return value (searcher/cpu.py:44-101,
     *     searcher/cuda.py:56-143): dense[h*dense_stride + i] = (q_h.k_i)*scaling[h] for
     *     every selected key, untouched elsewhere (caller pre-fills).  dense_by_position
     *     != 0: i = position of the key in insertion order (CPU searcher's index space);
     *     0: i = key slot (GPU searcher's index space).  dense_fill != 0 (slots only): the
     *     search writes dense_fill_value to every other element dense[h*dense_stride + i],
     *     i < size[0], itself -- no pre-fill, one launch less (the reference fills its output
     *     buffer before every search, searcher/cuda.py:35-54). */
    float* dense;
    int64_t dense_stride;
    int32_t dense_by_position;
    int32_t dense_fill;
    /* (2) compact lists: for head h, sel_count[h] entries (unordered) of
     *     sel_index[h*sel_cap + j] (slot or position, as above) and sel_score (raw q.k).
     *     sel_count must be zeroed by the caller; entries beyond sel_cap are counted but
     *     not stored. */
    int32_t* sel_index;
    float* sel_score;
    int32_t* sel_count;
    int32_t sel_cap;
    float dense_fill_value;
    /* (3) attention over the selected keys (+ the queue): out (H_q, Dv) fp32.
     *     Heads with an empty selection get zeros. */
    float* attn_out;
    /* optional counters, zeroed by the caller: (T, HIRA_STATS_COLS) uint64:
     *     [l] nodes of level l evaluated by at least one head of the tree's group
     *     (l = 0: candidate keys), [HIRA_MAX_LEVELS] keys selected by at least one head,
     *     [HIRA_MAX_LEVELS+1] (key, head) selections, [HIRA_MAX_LEVELS+2] keys whose bf16 row
     *     was fetched for the exact test after the 8-bit scan (HIRA_TILE16_Q8; else 0). */
    unsigned long long* stats;
} HiraSearchOut;

typedef struct HiraLaunch {
    int32_t block_threads;  /* vector-ALU kernel: 64, 128 or 256; MFMA kernel: a multiple of 64
                               up to 512; 0 = default */
    int32_t nodes_per_wave; /* vector-ALU kernel: level-1 nodes one wavefront walks; MFMA kernel:
                               tiles of 16 level-1 nodes one workgroup walks (at most 16);
                               0 = chosen from the tree and the device */
    int32_t kernel;         /* 0 = auto, 1 = vector-ALU kernel, 2 = MFMA kernel (bf16) */
    int32_t separate_merge; /* != 0: fold the attention partials in a second launch even
                               where the search kernel could do it itself */
} HiraLaunch;

int hira_abi_version(void);
const char* hira_last_error(void);

/* Bytes of workspace hira_search needs for this tree/query (arrival counters, one per tree
 * and head pass, at the start; attention partials after them).  The workspace must be ZERO
 * before its first use; every completed call leaves the counters zero again, and they sit
 * at an offset that depends only on the number of trees and head passes, so a workspace can
 * be reused without clearing by any later call with the same trees and heads that needs no
 * more bytes (a tree that grew, a queue that came or went).  Two calls that may run
 * concurrently need separate workspaces. */
size_t hira_search_workspace_bytes(const HiraTree* tree, const HiraQuery* query,
                                   const HiraQueue* queue, const HiraLaunch* launch);

/*
 * Halfspace range search (+ optional fused sparse attention).
 * Replaces: fused_tree_search_v3 (kernels/cpp/torch_ext_v3.cpp:36-247),
 * triton_two_level_filter / triton_three_level_filter (kernels/triton_search_wrappers.py:
 * 113-211, 214-358; kernels/triton_search_kernels.py:6-148) and the attention function
 * the reference leaves unwritten (attention/hira_attention.py:1-3).
 * Semantics: a node is pruned when q.c + ||q||*r < tau; a key is selected when
 * q.k >= tau (the CPU kernels' comparisons, torch_ext_v3.cpp:182, 212, 238).
 * queue may be NULL.  workspace is needed only when out->attn_out != NULL.
 */
int hira_search(const HiraTree* tree, const HiraQuery* query, const HiraQueue* queue,
                const HiraSearchOut* out, const HiraLaunch* launch, void* workspace,
                size_t workspace_bytes, void* stream);

/*
 * hira_search for callers that cannot allocate device memory and have no workspace to pass:
 * code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  It has
 * no counterpart in the reference.  Same arguments and results as hira_search; the arrival
 * counters and attention partials live in a buffer inside the library's own device image
 * (8 MiB per GPU the library runs on, held until the process ends), so the call allocates
 * nothing and asks the caller for nothing.  Limits: at most 16384 trees x head passes, and
 * H_q * P * (Dv + 2) * 4 bytes of partials (P = workgroups per tree, as
 * hira_search_workspace_bytes counts them) must fit in 8 MiB - 64 KiB; larger searches are
 * refused with HIRA_EWORKSPACE and a message naming both sizes.  The device that `stream`
 * belongs to must be the current device.  Every call on a GPU shares that GPU's buffer: calls
 * that may overlap on one GPU (different streams) race -- order them, or give the others a
 * workspace of their own through hira_search.  The counters are left at zero by every
 * completed call; the partials keep the last call's contents and are overwritten before they
 * are read.  The first call on a device looks the buffer's address up (a symbol lookup that may
 * load the library's code object -- not a stream operation): make one call on the device, at
 * set-up, before a stream capture begins; every later call, under capture too, records nothing
 * but the kernel launch.
 */
int hira_search_noalloc(const HiraTree* tree, const HiraQuery* query, const HiraQueue* queue,
                        const HiraSearchOut* out, const HiraLaunch* launch, void* stream);

/*
 * Index build.  Replaces CUDAIndexer.build and its helpers (indexer/cuda.py:56-108,
 * 200-336, 338-538: centroid choice, nearest-centroid assignment, closest-first packing into
 * blocks of bf, layout of the levels, radii from the layout, indexer/cuda.py:114-198) and,
 * for the Lloyd rounds, CPUIndexer._sample_centroids_faiss (indexer/cpu.py:223-261).
 *   tree       buffers for the result; tree->size[] must be the padded layout of n keys:
 *              size[L-1] = K_{L-1}, size[l] = size[l+1]*bf with K_0 = n,
 *              K_l = ceil(K_{l-1}/bf); cap[l] >= size[l].  Slots beyond size[] are not
 *              touched.
 *   keys_in    (T, n, D), values_in (T, n, Dv) or NULL, in insertion order, tree dtype.
 *   niter      Lloyd rounds per level (the reference's max_iterations); 0 = sampled points
 *              as centroids, as the reference's GPU build does.
 *   pack_rounds rounds of "propose to the nearest centroid with room" before leftovers
 *              are placed in order; >= 1.
 *   seed       picks the initial centroids.
 */
size_t hira_build_workspace_bytes(const HiraTree* tree, int32_t n);
int hira_build(const HiraTree* tree, const void* keys_in, const void* values_in, int32_t n,
               int32_t niter, int32_t pack_rounds, uint64_t seed, void* workspace,
               size_t workspace_bytes, void* stream);

/*
 * hira_build for trees that hold different numbers of keys: tree t's keys are the first
 * n_live[t] (device array of T counts, each <= n) rows of its (n, D) block of keys_in; the
 * other rows are never read.  Every tree gets the layout of n keys (tree->size[] as for
 * hira_build); a tree with fewer keys has emptier or empty nodes (count 0, radius -inf) and
 * empty key slots (perm < 0).  Two levels only.  It is what re-clusters one subtree of every
 * tree of an index in a single build (the subtrees hold different numbers of keys); the
 * reference has no counterpart (its update never re-clusters, indexer/cuda.py:544-701).
 * n_live == NULL: hira_build.
 */
int hira_build_ragged(const HiraTree* tree, const void* keys_in, const void* values_in, int32_t n,
                      const int32_t* n_live, int32_t niter, int32_t pack_rounds, uint64_t seed,
                      void* workspace, size_t workspace_bytes, void* stream);

/*
 * Nearest centre of every row, the distance step of the build (every Lloyd round and every
 * packing round of hira_build runs these kernels) as a call of its own:
 *   idx[t][i] = argmin_k ||x[t][i] - centers[t][k]||^2 over the centres with valid[t][k] != 0,
 * the lowest k on ties, -1 (and dist2 = +inf) when no centre is valid.
 * Replaces nearest_l2_triton_batched (kernels/triton_update_kernels.py:6-123, 329-418:
 * argmin of ||c||^2 - 2 x.c over valid centres in blocks of 128, then across the blocks) and
 * the cdist + argmin of the reference's GPU build (indexer/cuda.py:244-264).
 *   x        (T, n, D) rows in `dtype`; centers (T, m, D) fp32 (k-means centroids are fp32
 *            means); valid (T, m) int32 or NULL (all valid)
 *   idx      (T, n) int32; dist2 (T, n) fp32 squared distance to the chosen centre
 * bf16 rows of 64, 128 or 256 columns run on the matrix cores (centres split into two bf16
 * halves so that the choice is as good as with fp32 products), everything else on the vector
 * ALUs with fp32 differences.
 */
size_t hira_nearest_workspace_bytes(int32_t dtype, int32_t num_trees, int32_t m, int32_t dim);
int hira_nearest(const void* x, int32_t dtype, int32_t num_trees, int32_t n,
                 const float* centers, int32_t m, int32_t dim, const int32_t* valid,
                 int32_t* idx, float* dist2, void* workspace, size_t workspace_bytes,
                 void* stream);

/*
 * Append m new keys (and values) per tree to an existing index, in insertion order.
 * Replaces CUDAIndexer.update (indexer/cuda.py:544-701) and its kernels nearest_l2 (kernels/
 * triton_update_kernels.py:6-123, 329-418), fill_existing_children_atomic (:126-235) and
 * update_parent_radii_atomic (:238-326): a key joins the nearest level-1 node with a free
 * slot (radius and ancestors' radii grow, centres never move); when none has room it opens
 * a new level-1 node centred on itself, attached upwards by the same rule.
 *   tree       the index; cap[] must leave room: per call at most ceil(m/bf)+1 new nodes
 *              appear at level 1, ceil(that/bf)+1 at level 2, ... (tree->size[] is not read)
 *   new_keys   (T, m, D), new_values (T, m, Dv) or NULL, tree dtype, row-major
 *   state      (T, HIRA_MAX_LEVELS+2) int32, kept by the caller across calls:
 *              [l] = slots of level l in use (initially size[l]; [0] is only kept for
 *              one-level indexes), [HIRA_MAX_LEVELS] = keys inserted so far (initially n),
 *              [HIRA_MAX_LEVELS+1] = set to 1 if a key was dropped for lack of capacity.
 * After the call the caller sets size[l] = max over trees of state[.][l] (level 0:
 * size[0] = size[1]*bf) before the next search.
 */
int hira_update(const HiraTree* tree, const void* new_keys, const void* new_values, int32_t m,
                int32_t* state, void* stream);

/*
 * (Re)compute the 8-bit shadow of a HIRA_TILE16_Q8 index from its bf16 keys, for the key slots
 * [slot_first, slot_first + slot_count) of every tree (whole level-1 nodes: both multiples of
 * bf): keys8 for those slots and keps for their nodes.  recompute_scale != 0 first derives
 * kscale from ALL key slots [0, size[0]) (largest magnitude per channel / 127) and then needs
 * the whole range.  hira_build calls this itself; callers that move keys around afterwards
 * (grafting a sub-tree, re-clustering a subtree, restoring a file) call it for what they
 * touched.  Empty slots (perm < 0) hold zeros and do not count.  No counterpart in the
 * reference, which keeps fp32 keys only (indexer/cuda.py:365-368).
 */
int hira_quantize(const HiraTree* tree, int32_t slot_first, int32_t slot_count,
                  int32_t recompute_scale, void* stream);

/*
 * Per-head thresholds from a sample of each tree's keys, in one launch ahead of hira_search
 * on the same stream.  The reference names the two rules and leaves them unwritten
 * (cache/threshold_finder.py:1-14: sample_max and sample_mean_topk raise NotImplementedError;
 * cache/hira_config.py:20-22 holds their settings threshold_method and sample_size):
 *   HIRA_TAU_SAMPLE_MAX        tau[h] = max over the samples x of head h's tree of q_h.x
 *   HIRA_TAU_SAMPLE_MEAN_TOPK  tau[h] = mean of the k largest q_h.x  (1 <= k <= num_samples)
 *   samples    (num_trees, num_samples, dim) row-major in `dtype`, num_samples <= 4096
 *   query      q, num_q_heads and the head map are read (tau and scaling are not)
 *   tau_out    (H_q) fp32; scores are accumulated in fp32
 */
enum { HIRA_TAU_SAMPLE_MAX = 0, HIRA_TAU_SAMPLE_MEAN_TOPK = 1 };
int hira_threshold(const void* samples, int32_t dtype, int32_t num_trees, int32_t num_samples,
                   int32_t dim, const HiraQuery* query, int32_t method, int32_t k,
                   float* tau_out, void* stream);

/*
 * hira_update and hira_threshold of one decode step as ONE launch, for a step that appends a key
 * per tree and takes its thresholds from a key sample: the reference does the two from Python
 * one after the other (cache/hira_cache.py:121-153 appends, cache/threshold_finder.py:1-14 names
 * the rules), and the two share no data, so one launch's workgroups can do both (a launch less
 * per token: some 6 us).  Arguments and results are those of the two calls, bit for bit; the
 * samples have the tree's dtype, dim and tree count.  A window that hira_update places with its
 * window kernel (m >= 4 on two or more levels) and m = 0 are served by the two launches.
 */
int hira_update_threshold(const HiraTree* tree, const void* new_keys, const void* new_values,
                          int32_t m, int32_t* state, const void* samples, int32_t num_samples,
                          const HiraQuery* query, int32_t method, int32_t k, float* tau_out,
                          void* stream);

/*
 * Softmax attention over given lists of selected keys, for callers that edit the selection
 * between search and attention (hira_search with attn_out does both in one launch):
 *   out[h] = sum_j softmax_j(scaling[h] * sel_score[h][j]) * values[tree(h)][sel_index[h][j]]
 * This is the attention the reference leaves unwritten (attention/hira_attention.py:1-3) over
 * the result of its searchers (searcher/cuda.py:56-143).
 *   tree       values, vdim, dtype, cap[0] and num_trees are read
 *   query      num_q_heads, scaling and the head map are read
 *   sel_*      the lists as hira_search writes them: sel_index key SLOTS (dense_by_position
 *              = 0), sel_score raw q.k, sel_count entries per head (more than sel_cap: the
 *              first sel_cap count); an index outside [0, cap[0]) is clamped
 *   attn_out   (H_q, Dv) fp32; zeros for a head with an empty list
 */
int hira_sparse_attention(const HiraTree* tree, const HiraQuery* query, const int32_t* sel_index,
                          const float* sel_score, const int32_t* sel_count, int32_t sel_cap,
                          float* attn_out, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* HIRA_HIP_H */
