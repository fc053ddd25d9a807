// Host side of the halfspace range search: the launch plan, the entry points, and the fold of
// the partials as a launch of its own.  The kernel is in search_vec_kernel.h, instantiated per
// element type in search_vec_f32.hip and search_vec_bf16.hip.
#include "search_vec_kernel.h"

namespace hira {

// The fold as a launch of its own: one workgroup per head.
__global__ __launch_bounds__(256) void merge_kernel(const float* __restrict__ part_m,
                                                    const float* __restrict__ part_l,
                                                    const float* __restrict__ part_acc, int P,
                                                    int Dv, int dvl, float* __restrict__ out) {
    __shared__ float red[4];
    extern __shared__ float smem[];  // (NG, Dv + 1)
    const int head = blockIdx.x;
    fold_partials(part_m + (size_t)head * P, part_l + (size_t)head * P,
                  part_acc + (size_t)head * P * Dv, P, Dv, dvl, out + (size_t)head * Dv, smem, red);
}

// ---- host side ------------------------------------------------------------------------
static int round_pow2(int v) {
    int r = 1;
    while (r < v) r <<= 1;
    return r;
}

// compute units of the current device (asked once per device: the launch plan depends on it)
static int compute_units() {
    constexpr int kMaxDev = 64;
    static int cus[kMaxDev];  // 0: not asked yet (written once per entry, the same value from any thread)
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDev) return 256;
    int n = __atomic_load_n(&cus[dev], __ATOMIC_RELAXED);
    if (n == 0) {
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
            n = 256;
        __atomic_store_n(&cus[dev], n, __ATOMIC_RELAXED);
    }
    return n;
}

// attn: the launch writes attention partials (the plan then also weighs what folding them costs)
static int make_plan(const HiraTree* t, const HiraQuery* q, const HiraQueue* queue,
                     const HiraLaunch* launch, bool attn, SearchPlan* plan) {
    HIRA_CHECK_ARG(t && q, "tree and query must not be NULL");
    HIRA_CHECK_ARG(t->dtype == HIRA_F32 || t->dtype == HIRA_BF16, "dtype %d", t->dtype);
    const int esize = t->dtype == HIRA_F32 ? 4 : 2;
    const int epl = 16 / esize;
    HIRA_CHECK_ARG(t->num_trees >= 1, "num_trees %d", t->num_trees);
    HIRA_CHECK_ARG(t->num_levels >= 1 && t->num_levels <= HIRA_MAX_LEVELS, "num_levels %d",
                   t->num_levels);
    HIRA_CHECK_ARG(t->bf >= 1 && t->bf <= 64, "branching factor %d not in 1..64", t->bf);
    HIRA_CHECK_ARG(t->dim >= epl && t->dim % epl == 0,
                   "dim %d: rows must be a multiple of 16 bytes", t->dim);
    HIRA_CHECK_ARG(t->vdim >= 0 && t->vdim % epl == 0,
                   "vdim %d: rows must be a multiple of 16 bytes", t->vdim);
    const int widest = t->dim > t->vdim ? t->dim : t->vdim;
    int lpr = round_pow2((widest + epl - 1) / epl);
    if (lpr < 2) lpr = 2;
    HIRA_CHECK_ARG(lpr <= 64, "dim %d / vdim %d too wide (max %d)", t->dim, t->vdim, 64 * epl);
    HIRA_CHECK_ARG(t->keys != nullptr, "keys is NULL");
    for (int l = 0; l < t->num_levels; ++l) {
        HIRA_CHECK_ARG(t->size[l] >= 0 && t->size[l] <= t->cap[l], "size[%d]=%d cap=%d", l,
                       t->size[l], t->cap[l]);
        if (l >= 1) {
            HIRA_CHECK_ARG(t->centers[l] && t->radii[l] && t->counts[l],
                           "level %d arrays missing", l);
            HIRA_CHECK_ARG((int64_t)t->size[l] * t->bf >= t->size[l - 1],
                           "size[%d]=%d exceeds size[%d]*bf", l - 1, t->size[l - 1], l);
        }
    }
    HIRA_CHECK_ARG(q->num_q_heads >= 1 && q->q && q->tau && q->scaling && q->tree_q_off &&
                       q->tree_q_heads,
                   "query arrays missing");
    HIRA_CHECK_ARG(q->max_group >= 1, "max_group %d", q->max_group);
    HIRA_CHECK_ARG(t->layout == HIRA_ROW_MAJOR || t->layout == HIRA_TILE16 ||
                       t->layout == HIRA_TILE16_Q8, "layout %d", t->layout);
    if (t->layout == HIRA_TILE16_Q8)
        HIRA_CHECK_ARG((t->dim == 64 || t->dim == 128) && t->num_levels >= 2 && t->keys8 &&
                           t->kscale && t->keps,
                       "the layout with an 8-bit shadow needs rows of 64 or 128 columns, at least "
                       "two levels, and the keys8 / kscale / keps arrays");
    if (t->layout != HIRA_ROW_MAJOR) {
        HIRA_CHECK_ARG(t->dtype == HIRA_BF16 && t->dim % 32 == 0,
                       "the tiled layout needs bf16 rows of a multiple of 32 columns");
        for (int l = 0; l < t->num_levels; ++l)
            HIRA_CHECK_ARG(t->cap[l] % 16 == 0, "tiled layout: cap[%d]=%d not a multiple of 16",
                           l, t->cap[l]);
    }
    plan->gate_steps = 1;
    plan->num_queue_blocks = 0;
    if (queue && queue->keys && queue->len > 0) {
        HIRA_CHECK_ARG(queue->len <= queue->cap, "queue len %d > cap %d", queue->len,
                       queue->cap);
        plan->num_queue_blocks = (queue->len + kPseudoBlock - 1) / kPseudoBlock;
    }
    const int want = launch ? launch->kernel : 0;
    HIRA_CHECK_ARG(want >= 0 && want <= 2, "kernel %d", want);
    const bool mfma_ok = mfma_search_supported(t, queue);
    HIRA_CHECK_ARG(want != 2 || mfma_ok,
                   "the MFMA kernel needs bf16, tiled layout, >= 2 levels, fan-out 16/32/48/64, "
                   "dim = vdim in {64,128,256}, under 4 GiB of key slots per tree");
    plan->kernel = (want == 2 || (want == 0 && mfma_ok)) ? 2 : 1;
    plan->lpr = lpr;
    if (plan->kernel == 2) {
        // one workgroup per tile of 16 level-1 nodes; heads in passes of 16
        plan->gmax = q->max_group < 16 ? q->max_group : 16;
        plan->head_chunks = (q->max_group + 15) / 16;
        int threads = launch && launch->block_threads ? launch->block_threads : kMfmaThreads;
        HIRA_CHECK_ARG(threads >= 64 && threads <= kMfmaThreads && threads % 64 == 0,
                       "block_threads %d must be a multiple of 64 up to %d", threads, kMfmaThreads);
        plan->threads = threads;
        // a workgroup walks `tpw` tiles of 16 level-1 nodes (a stride apart): as few as keep
        // one workgroup per CU in the launch (the kernel runs one at a time on a CU) and no
        // more partials per head than the fold can list in LDS, 128 at most: a tree alone on
        // the chip is scanned by up to 128 workgroups (131072 keys: 20.5 us; with 64 workgroups
        // of four tiles 23.9 us, with 256 of one tile 24.1 us)
        const int tiles = (t->size[1] + 15) / 16;
        int max_parts = 16 * t->dim / plan->gmax;
        max_parts = max_parts < 64 ? 64 : (max_parts > 128 ? 128 : max_parts);
        int tpw = launch ? launch->nodes_per_wave : 0;
        HIRA_CHECK_ARG(tpw >= 0 && tpw <= kMfmaMaxTilesPerWg,
                       "MFMA kernel: %d tiles per workgroup (at most %d)", tpw, kMfmaMaxTilesPerWg);
        if (tpw == 0) {
            const int64_t all = (int64_t)tiles * t->num_trees * plan->head_chunks;
            const int cus = compute_units();
            tpw = (int)((all + cus - 1) / cus);
            if (tpw * max_parts < tiles) tpw = (tiles + max_parts - 1) / max_parts;
            if (tpw < 1) tpw = 1;
            // more work than one workgroup per CU can take: several rounds of workgroups of 8 to 16
            // tiles, of the size whose rounds add up to the least (a workgroup costs some two
            // tiles' time before and after its scan; measured at 128 trees x 64 tiles: 16 tiles a
            // workgroup 178 us, 8 tiles 182 us, 4 tiles 206 us)
            if (tpw > kMfmaMaxTilesPerWg) {
                int64_t best = 0;
                for (int c = kMfmaMaxTilesPerWg; c >= kMfmaMaxTilesPerWg / 2; --c) {
                    const int64_t wgs = (int64_t)((tiles + c - 1) / c) * t->num_trees * plan->head_chunks;
                    const int64_t cost = ((wgs + cus - 1) / cus) * (c + 2);
                    if (best == 0 || cost < best) best = cost, tpw = c;
                }
            }
        }
        plan->nodes_per_wave = tpw;
        plan->num_nodes = t->size[1];
        plan->tree_blocks = (tiles + tpw - 1) / tpw;
        if (!(launch && launch->nodes_per_wave)) {
            // a launch that fits one round: as many workgroups a tree as there are compute units
            // for it, each with `tpw` tiles or one less (the tiles are dealt out a stride apart),
            // rather than fewer workgroups that all hold `tpw` (66 tiles a tree on 32 compute units
            // a tree: 32 workgroups of 2 or 3 tiles, not 22 of 3 -- what an index that grew by a
            // few nodes since the last rebuild looks like: 24.6 -> 21 us per step)
            const int64_t per_tree = compute_units() / ((int64_t)t->num_trees * plan->head_chunks);
            int64_t blocks = per_tree < tiles ? per_tree : tiles;
            if (blocks > max_parts) blocks = max_parts;
            if (blocks > plan->tree_blocks) plan->tree_blocks = (int)blocks;
        }
        plan->queue_blocks = plan->num_queue_blocks > 0 ? 1 : 0;  // one workgroup takes the whole queue
        plan->smem = 0;
        // every workgroup that walks the tree must own at least one tile: one without a tile
        // leaves the kernel before it draws its ticket, and the fold would never run
        if (plan->tree_blocks > tiles)
            return fail(HIRA_EINVAL, "launch plan: %d workgroups for %d tiles", plan->tree_blocks, tiles);
        return HIRA_OK;
    }
    plan->gmax = q->max_group <= 1 ? 1 : (q->max_group <= 4 ? 4 : 8);
    plan->head_chunks = (q->max_group + plan->gmax - 1) / plan->gmax;
    int threads = launch && launch->block_threads ? launch->block_threads : 256;
    HIRA_CHECK_ARG(threads == 64 || threads == 128 || threads == 256,
                   "block_threads %d must be 64, 128 or 256", threads);
    plan->threads = threads;
    const int rpw = 64 / lpr;
    // nodes that hold very few keys (a step of gates leads to at most 8 rows): a wave batches
    // two or four steps of gates and scans the batch's keys as one block -- as long as that
    // leaves the chip's 256 compute units eight waves each (below that the longer chain of a
    // wave costs more than its trips save)
    if (t->num_levels >= 2 && t->bf * rpw <= 8) {
        const long long steps = (long long)t->num_trees * plan->head_chunks *
                                ((t->size[1] + rpw - 1) / rpw);
        plan->gate_steps = steps >= 4 * 2048 ? 4 : (steps >= 2 * 2048 ? 2 : 1);
        if (launch && launch->nodes_per_wave)
            plan->gate_steps = launch->nodes_per_wave > rpw ? 4 : 1;
    }
    int npw = launch && launch->nodes_per_wave ? launch->nodes_per_wave : rpw * plan->gate_steps;
    HIRA_CHECK_ARG(npw >= 1, "nodes_per_wave %d", npw);
    plan->num_nodes = t->num_levels >= 2 ? t->size[1]
                                         : (t->size[0] + kPseudoBlock - 1) / kPseudoBlock;
    // large trees under attention: a wave takes more steps of nodes, towards 64 partials a head to
    // fold, as long as the launch keeps two workgroups per compute unit (8 trees x 65536 fp32
    // keys, fan-out 32, 4 heads a tree: 256 partials 127 us, 128: 103, 64: 94, 32: 158; one such
    // tree alone: 256 partials 47 us, 128: 55, 64: 82)
    if (attn && !(launch && launch->nodes_per_wave) && plan->gate_steps == 1) {
        const int wpb = threads / 64;
        auto parts = [&](int n) { return (plan->num_nodes + wpb * n - 1) / (wpb * n); };
        while (parts(npw) > 64 &&
               (int64_t)t->num_trees * plan->head_chunks * parts(2 * npw) >= 2 * compute_units())
            npw *= 2;
    }
    plan->nodes_per_wave = npw;
    const int per_block = (threads / 64) * npw;
    plan->tree_blocks = (plan->num_nodes + per_block - 1) / per_block;
    plan->queue_blocks = (plan->num_queue_blocks + per_block - 1) / per_block;
    plan->smem = (size_t)(threads / 64) * plan->gmax * (lpr * epl + 2) * sizeof(float);
    {   // the fold of the last workgroup reuses the same LDS: (ng, vdim + 1) floats
        const int dvl = round_pow2((t->vdim + 3) / 4);
        if (dvl > 0 && dvl <= threads) {
            const size_t fold = (size_t)(threads / dvl) * (t->vdim + 1) * sizeof(float);
            if (fold > plan->smem) plan->smem = fold;
        }
    }
    return HIRA_OK;
}

}  // namespace hira

using namespace hira;

// partials (acc, m, l) followed by the arrival counters of the fused fold
// bytes of the arrival counters, which come first: their place does not depend on the
// number of partials, so a workspace stays usable when the tree grows or a queue comes and goes
static size_t counter_bytes(int trees, int passes) {
    return (((size_t)trees * passes * sizeof(int32_t)) + 255) & ~(size_t)255;
}

static size_t workspace_need(int h_q, size_t P, int vdim, int trees, int passes) {
    return counter_bytes(trees, passes) + (size_t)h_q * P * (size_t)(vdim + 2) * sizeof(float);
}

extern "C" size_t hira_search_workspace_bytes(const HiraTree* tree, const HiraQuery* query,
                                              const HiraQueue* queue,
                                              const HiraLaunch* launch) {
    SearchPlan plan;
    if (make_plan(tree, query, queue, launch, true, &plan) != HIRA_OK) return 0;
    const size_t P = (size_t)plan.tree_blocks + plan.queue_blocks;
    return workspace_need(query->num_q_heads, P, tree->vdim, tree->num_trees, plan.head_chunks);
}

// The search behind both entry points.  Attention needs arrival counters (one int32 per tree
// and head pass, zero between calls) and room for the partials; `fixed_counters` > 0: the
// counters live in a region of that many entries of their own (the entry point that allocates
// nothing), else at the start of the caller's workspace, the partials right after them.
static int search_impl(const HiraTree* tree, const HiraQuery* query, const HiraQueue* queue,
                       const HiraSearchOut* out, const HiraLaunch* launch, void* workspace,
                       size_t workspace_bytes, size_t fixed_counters, void* stream) {
    SearchPlan plan;
    HIRA_CHECK_ARG(out != nullptr, "out is NULL");
    const bool attn = out->attn_out != nullptr;
    int rc = make_plan(tree, query, queue, launch, attn, &plan);
    if (rc != HIRA_OK) return rc;
    if (attn) {
        HIRA_CHECK_ARG(tree->values != nullptr && tree->vdim > 0,
                       "attention needs values in the tree");
        HIRA_CHECK_ARG(tree->vdim % 4 == 0, "vdim %d must be a multiple of 4", tree->vdim);
        HIRA_CHECK_ARG(plan.num_queue_blocks == 0 || queue->values != nullptr,
                       "queue values missing");
    }
    // by position the row length is the number of keys inserted so far, which only the
    // caller knows; by slot it must cover every slot in use
    if (out->dense && !out->dense_by_position)
        HIRA_CHECK_ARG(out->dense_stride >= tree->size[0], "dense_stride %lld < %d slots",
                       (long long)out->dense_stride, tree->size[0]);
    HIRA_CHECK_ARG(!(out->dense && out->dense_fill && out->dense_by_position),
                   "dense_fill goes with key slots, not with positions");
    if (out->dense_by_position && (out->dense || out->sel_count))
        HIRA_CHECK_ARG(tree->perm != nullptr, "perm missing");
    if (out->sel_count)
        HIRA_CHECK_ARG(out->sel_index && out->sel_score && out->sel_cap > 0,
                       "selection list arrays missing");

    SearchParams p;
    memset(&p, 0, sizeof(p));
    p.keys = tree->keys;
    p.values = tree->values;
    p.perm = tree->perm;
    for (int l = 0; l < HIRA_MAX_LEVELS; ++l) {
        p.centers[l] = tree->centers[l];
        p.radii[l] = tree->radii[l];
        p.counts[l] = tree->counts[l];
        p.size[l] = tree->size[l];
        p.cap[l] = tree->cap[l];
    }
    p.num_levels = tree->num_levels;
    p.bf = tree->bf;
    p.dim = tree->dim;
    p.vdim = tree->vdim;
    p.layout = center_layout_of(tree->layout);
    p.key_layout = key_layout_of(tree->layout);
    if (tree->layout == HIRA_TILE16_Q8) {
        p.keys8 = tree->keys8;
        p.kscale = tree->kscale;
        p.keps = tree->keps;
    }
    p.q = query->q;
    p.tau = query->tau;
    p.scaling = query->scaling;
    p.tree_q_off = query->tree_q_off;
    p.tree_q_heads = query->tree_q_heads;
    const bool use_queue = attn && plan.num_queue_blocks > 0;
    if (use_queue) {
        p.queue_keys = queue->keys;
        p.queue_values = queue->values;
        p.queue_len = queue->len;
        p.queue_cap = queue->cap;
    }
    p.nodes_per_wave = plan.nodes_per_wave;
    p.tree_blocks = plan.tree_blocks;
    {   // up to what the eight L2s hold together (32 MiB) the default policy; up to 512 MiB the
        // key tiles and the value rows non-temporal; beyond, the key tiles only
        const size_t key_bytes = (size_t)tree->num_trees * (size_t)tree->size[0] * (size_t)tree->dim * 2;
        p.key_policy = key_bytes <= ((size_t)32 << 20) ? 0 : (key_bytes <= ((size_t)512 << 20) ? 2 : 1);
    }
    p.num_nodes = plan.num_nodes;
    p.num_queue_blocks = use_queue ? plan.num_queue_blocks : 0;
    p.dense = out->dense;
    p.dense_stride = out->dense_stride;
    p.dense_by_position = out->dense_by_position;
    p.dense_fill = out->dense != nullptr ? out->dense_fill : 0;
    p.dense_fill_value = out->dense_fill_value;
    p.sel_index = out->sel_index;
    p.sel_score = out->sel_score;
    p.sel_count = out->sel_count;
    p.sel_cap = out->sel_cap;
    p.stats = out->stats;

    const int P = plan.tree_blocks + (use_queue ? plan.queue_blocks : 0);
    if (P == 0) return HIRA_OK;
    p.num_parts = P;
    if (attn) {
        size_t ctr_bytes = counter_bytes(tree->num_trees, plan.head_chunks);
        if (fixed_counters > 0) {
            if ((size_t)tree->num_trees * plan.head_chunks > fixed_counters)
                return fail(HIRA_EWORKSPACE, "%d trees x %d head passes: more than the %zu arrival "
                            "counters of the built-in scratch buffer", tree->num_trees,
                            plan.head_chunks, fixed_counters);
            ctr_bytes = fixed_counters * sizeof(int32_t);
        }
        const size_t need = ctr_bytes + workspace_need(query->num_q_heads, (size_t)P, tree->vdim, 0, 0);
        if (workspace == nullptr || workspace_bytes < need)
            return fail(HIRA_EWORKSPACE, fixed_counters > 0
                            ? "the built-in scratch buffer holds %zu bytes, this search needs %zu"
                            : "workspace %zu bytes, need %zu", workspace_bytes, need);
        float* w = reinterpret_cast<float*>(reinterpret_cast<char*>(workspace) + ctr_bytes);
        p.part_acc = w;
        p.part_m = w + (size_t)query->num_q_heads * P * tree->vdim;
        p.part_l = p.part_m + (size_t)query->num_q_heads * P;
        p.attn_out = out->attn_out;
        // the search kernel folds the partials itself (the last workgroup of a tree to arrive
        // does it) unless the caller asks for the second launch
        p.fold_dvl = round_pow2((tree->vdim + 3) / 4);
        // (vector-ALU kernel: its last workgroup folds the heads of its pass one after the
        // other, which only pays for a single head with few partials; the second launch has
        // a workgroup per head)
        const bool can_fold = plan.kernel == 2 ||
                              (p.fold_dvl <= plan.threads && plan.gmax == 1 && P <= 64);
        if (can_fold && !(launch && launch->separate_merge))
            p.done = reinterpret_cast<int32_t*>(workspace);
    }
    p.group_size = query->group_size > 0 ? query->group_size : 0;
    if (p.group_size > 0)
        HIRA_CHECK_ARG((int64_t)p.group_size * tree->num_trees == query->num_q_heads,
                       "group_size %d x %d trees != %d heads", p.group_size, tree->num_trees,
                       query->num_q_heads);

    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    dim3 grid(P, tree->num_trees, plan.head_chunks);
    p.gmax_state = plan.gmax;
    if (plan.kernel == 2)
        rc = launch_search_mfma(plan, p, dim3(tree->num_trees, P, plan.head_chunks), s);
    else
        rc = tree->dtype == HIRA_F32 ? launch_vec_f32(plan, p, grid, s)
                                     : launch_vec_bf16(plan, p, grid, s);
    if (rc != HIRA_OK) return rc;
    HIRA_CHECK_LAUNCH("search kernel");

    if (attn && p.done == nullptr) {
        int dvl = round_pow2((tree->vdim + 3) / 4);
        if (dvl > 256) return fail(HIRA_EINVAL, "vdim %d too wide", tree->vdim);
        const int ng = 256 / dvl;
        const size_t smem = (size_t)ng * (tree->vdim + 1) * sizeof(float);
        hipLaunchKernelGGL(merge_kernel, dim3(query->num_q_heads), dim3(256), smem, s, p.part_m,
                           p.part_l, p.part_acc, P, tree->vdim, dvl, out->attn_out);
        HIRA_CHECK_LAUNCH("merge kernel");
    }
    return HIRA_OK;
}

extern "C" int hira_search(const HiraTree* tree, const HiraQuery* query, const HiraQueue* queue,
                           const HiraSearchOut* out, const HiraLaunch* launch, void* workspace,
                           size_t workspace_bytes, void* stream) {
    return search_impl(tree, query, queue, out, launch, workspace, workspace_bytes, 0, stream);
}

// ---- the same search for callers that cannot allocate ----------------------------------------
// Its scratch (arrival counters, then attention partials) is this array in the library's own
// device image: every GPU the library runs on holds a copy until the process ends.  Host code
// never touches `scratch` by name (the name is a host-side stand-in, not a device address): the
// device address is asked for once per device, with that device current, and kept.
namespace hira {
constexpr size_t kScratchBytes = (size_t)8 << 20;
constexpr size_t kScratchCounters = 16384;  // int32 arrival counters at the start (64 KiB)
constexpr int kMaxDevices = 64;
}  // namespace hira
static __device__ __align__(256) unsigned char scratch[hira::kScratchBytes];
static void* g_scratch_ptr[hira::kMaxDevices];  // per device; written once (same value from any thread)

static int scratch_for_current_device(void** out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return fail(HIRA_ELAUNCH, "hipGetDevice: %s", hipGetErrorString(e));
    HIRA_CHECK_ARG(dev >= 0 && dev < kMaxDevices, "device %d: at most %d devices", dev, kMaxDevices);
    void* ptr = __atomic_load_n(&g_scratch_ptr[dev], __ATOMIC_ACQUIRE);
    if (ptr == nullptr) {
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || ptr == nullptr)
            return fail(HIRA_ELAUNCH, "hipGetSymbolAddress(scratch) on device %d: %s", dev,
                        hipGetErrorString(e));
        __atomic_store_n(&g_scratch_ptr[dev], ptr, __ATOMIC_RELEASE);
    }
    *out = ptr;
    return HIRA_OK;
}

extern "C" int hira_search_noalloc(const HiraTree* tree, const HiraQuery* query,
                                   const HiraQueue* queue, const HiraSearchOut* out,
                                   const HiraLaunch* launch, void* stream) {
    void* ptr = nullptr;
    const int rc = scratch_for_current_device(&ptr);
    if (rc != HIRA_OK) return rc;
    return search_impl(tree, query, queue, out, launch, ptr, kScratchBytes, kScratchCounters, stream);
}
