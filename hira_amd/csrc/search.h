// Kernel arguments and launch plan shared by the two search kernels (vector-ALU: any
// dtype/row width/fan-out, row-major or tiled keys; MFMA: bf16, tiled keys).
#pragma once

#include "common.hip.h"

namespace hira {

constexpr int kPseudoBlock = 32;  // rows per block when there is no level-1 node (flat scan, queue)

struct SearchParams {
    // tree
    const void* keys;
    const void* values;
    const int32_t* perm;
    const void* centers[HIRA_MAX_LEVELS];
    const float* radii[HIRA_MAX_LEVELS];
    const int32_t* counts[HIRA_MAX_LEVELS];
    int32_t size[HIRA_MAX_LEVELS];
    int32_t cap[HIRA_MAX_LEVELS];
    int32_t num_levels, bf, dim, vdim;
    int32_t layout;  // of the centers: HIRA_ROW_MAJOR or HIRA_TILE16
    int32_t key_layout;  // of the keys
    const int8_t* keys8;  // HIRA_TILE16_Q8: the 8-bit shadow, its steps and error bounds
    const float* kscale;
    const float* keps;
    // queries
    const void* q;
    const float* tau;
    const float* scaling;
    const int32_t* tree_q_off;
    const int32_t* tree_q_heads;
    int32_t group_size;  // > 0: head h belongs to tree h / group_size (the CSR is not read)
    // queue (always row-major)
    const void* queue_keys;
    const void* queue_values;
    int32_t queue_len, queue_cap;
    // work split
    int32_t nodes_per_wave;  // level-1 nodes (or pseudo blocks) per wave; MFMA kernel: tiles per workgroup
    int32_t tree_blocks;     // workgroups that walk the tree; the rest scan the queue
    int32_t key_policy;      // MFMA kernel: which cache policy the scan's loads use (0: default,
                             // 1: key tiles non-temporal, 2: value rows too), by the launch's size
    int32_t num_nodes;       // level-1 nodes (or pseudo blocks over the keys when L == 1)
    int32_t num_queue_blocks;
    // outputs
    float* dense;
    int64_t dense_stride;
    int32_t dense_by_position;
    int32_t dense_fill;       // the kernels write dense_fill_value wherever no score goes
    float dense_fill_value;
    int32_t* sel_index;
    float* sel_score;
    int32_t* sel_count;
    int32_t sel_cap;
    float* part_m;    // (H_q, P)
    float* part_l;    // (H_q, P)
    float* part_acc;  // (H_q, P, Dv)
    int32_t num_parts;  // P = gridDim.x
    int32_t gmax_state; // MFMA kernel: heads per pass its LDS state rows are sized for
    float* attn_out;    // (H_q, Dv): written by the kernel itself when `done` is set
    int32_t* done;      // (T, passes) arrival counters, zero between launches; NULL: no fold
    int32_t fold_dvl;   // vector-ALU kernel's fold: threads per partial (four columns each)
    unsigned long long* stats;
};

struct SearchPlan {
    int kernel;       // 1 = vector-ALU, 2 = MFMA
    int lpr;          // lanes per row (vector-ALU kernel)
    int gmax;         // heads per pass
    int threads;      // workgroup size
    int nodes_per_wave;
    int num_nodes, num_queue_blocks;
    int tree_blocks, queue_blocks, head_chunks;
    int gate_steps;   // vector-ALU kernel: steps of gates a wave batches (1 or 4)
    size_t smem;
};

// search_vec_f32.hip, search_vec_bf16.hip: the vector-ALU kernel for rows of one element type
int launch_vec_f32(const SearchPlan& plan, const SearchParams& p, dim3 grid, hipStream_t s);
int launch_vec_bf16(const SearchPlan& plan, const SearchParams& p, dim3 grid, hipStream_t s);

// search_mfma.hip
bool mfma_search_supported(const HiraTree* t, const HiraQueue* queue);
constexpr int kMfmaThreads = 512;       // workgroup size of the MFMA kernel (8 waves), at most
constexpr int kMfmaMaxTilesPerWg = 16;  // tiles of 16 level-1 nodes one workgroup walks, at most
int launch_search_mfma(const SearchPlan& plan, const SearchParams& p, dim3 grid, hipStream_t s);

// Hand-off of the attention partials from the workgroups of a tree to the one that folds them
// (maybe behind another L2).  The partials are written with device-scope atomic stores: they
// are written through to the level at which every compute unit of the device sees them, and
// such a store only counts as complete (leaves the wave's count of outstanding memory
// operations) once it is visible at that level.  Every thread therefore waits here for its own
// stores to complete; the caller's barrier follows, then ONE thread takes a ticket with a
// device-scope atomic add, so every ticket is drawn after all partials of its workgroup are
// visible.  The workgroup that draws the last ticket reads the partials with device-scope
// atomic loads (which do not take a stale copy from its own L2) after a barrier that depends
// on the ticket.  A release fence at device scope would also order the stores but writes the
// whole L2 back first (measured: the decode step takes 36 instead of 20 microseconds);
// nothing but these atomic stores has to be handed over, so the wait is enough.
__device__ __forceinline__ void hand_off_release() {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
}

// The kernel's arguments lie in nine 64-byte lines of memory, and compiled code asks for each
// argument where it is first needed: line after line, each a trip to memory that the next one
// waits for (measured: the gates began 1.5 us after the workgroup).  Asking for a word of every
// line here, at once, makes them one trip; the reads of the arguments that follow are served from
// the scalar cache.  (The wait is inside the statement: its destination registers are free again
// when it ends.)
__device__ __forceinline__ void touch_kernel_arguments() {
    static_assert(sizeof(SearchParams) <= 9 * 64, "one load per 64-byte line of the arguments");
    auto ka = __builtin_amdgcn_kernarg_segment_ptr();
    uint32_t d0, d1, d2, d3, d4, d5, d6, d7, d8;
    asm volatile(
        "s_load_dword %0, %9, 0x0\n\t"
        "s_load_dword %1, %9, 0x40\n\t"
        "s_load_dword %2, %9, 0x80\n\t"
        "s_load_dword %3, %9, 0xc0\n\t"
        "s_load_dword %4, %9, 0x100\n\t"
        "s_load_dword %5, %9, 0x140\n\t"
        "s_load_dword %6, %9, 0x180\n\t"
        "s_load_dword %7, %9, 0x1c0\n\t"
        "s_load_dword %8, %9, 0x200\n\t"
        "s_waitcnt lgkmcnt(0)"
        : "=&s"(d0), "=&s"(d1), "=&s"(d2), "=&s"(d3), "=&s"(d4), "=&s"(d5), "=&s"(d6), "=&s"(d7), "=&s"(d8)
        : "s"(ka)
        : "memory");
}

// Where the keys / the centers of a tree layout sit (HIRA_TILE16_Q8: tiled centers, row-major
// keys beside their 8-bit shadow).
__device__ __host__ __forceinline__ int key_layout_of(int layout) {
    return layout == HIRA_TILE16 ? HIRA_TILE16 : HIRA_ROW_MAJOR;
}
__device__ __host__ __forceinline__ int center_layout_of(int layout) {
    return layout == HIRA_ROW_MAJOR ? HIRA_ROW_MAJOR : HIRA_TILE16;
}
// Byte index of column j of row `row` inside one tree's 8-bit shadow (tiles of 16 x 64).
__device__ __host__ __forceinline__ size_t shadow_index(int D, size_t row, int j) {
    const size_t chunk = ((row / 16) * (size_t)(D / 64) + (size_t)(j / 64)) * 64 + (size_t)((j % 64) / 16) * 16 + row % 16;
    return chunk * 16 + (size_t)(j % 16);
}

// Element index of (row, column j) inside one tree's (cap, D) matrix.
//   row-major: row*D + j
//   tiled (16 rows x 32 columns per tile, 16-byte chunks stored lane-major so that one
//   wave-wide 128-bit load fetches a whole MFMA A-operand tile):
//     chunk (tile = row/16, s = j/32, kb = (j%32)/8, i = row%16) at ((tile*KS + s)*64 + kb*16 + i)
__device__ __host__ __forceinline__ size_t elem_index(int layout, int D, size_t row, int j) {
    if (layout == HIRA_ROW_MAJOR) return row * (size_t)D + j;
    const size_t ks = (size_t)D / 32;
    const size_t chunk = ((row / 16) * ks + (size_t)(j / 32)) * 64 + (size_t)((j % 32) / 8) * 16 + row % 16;
    return chunk * 8 + (size_t)(j % 8);
}

// 16-byte load of chunk `c` (8 bf16 or 4 fp32) of row `row` of one tree's matrix.
template <typename T>
__device__ __forceinline__ uint4 load_row_chunk(const void* base, int layout, int D,
                                                size_t tree_row0, size_t row, int c) {
    constexpr int EPL = Elem<T>::kPerChunk;
    const T* p = reinterpret_cast<const T*>(base) + tree_row0 * (size_t)D;
    if (layout == HIRA_ROW_MAJOR) return *reinterpret_cast<const uint4*>(p + row * (size_t)D + c * EPL);
    return *reinterpret_cast<const uint4*>(p + elem_index(layout, D, row, c * EPL));
}

}  // namespace hira
