// Time stamps inside the MFMA search kernel, for looking at where a decode step spends its time.
// Compiled in only with -DHIRA_TIMELINE (the Makefile's `timeline` target builds
// libhira_hip_timeline.so that way); in the library that serves, every call below is empty and
// the kernel carries no trace of it.  With the stamps on, the buffer the caller passes as
// HiraSearchOut.stats receives kTlCols 64-bit words per workgroup instead of the statistics
// (which are then not counted): the constant-rate clock (100 MHz) at the points named below.
#pragma once

#include "search.h"

namespace hira {

// columns of a workgroup's row
enum TlStamp {
    kTlStart = 0,     // first instruction of thread 0
    kTlArgs,          // kernel arguments in registers, the heads of the pass known
    kTlGateIssued,    // queries and the first gate's operands asked for
    kTlGated,         // wave 0 has gated its tiles (its loads arrived, products, verdicts in LDS)
    kTlBarrier,       // every wave has: the barrier behind the gates passed
    kTlFetched,       // survivors listed, the first round's key tiles asked for
    kTlTiles,         // wave 0: the first round's products done (its tiles have arrived)
    kTlListed,        // wave 0: the first round's rows listed
    kTlGathered,      // wave 0: the first round's value rows in the sums
    kTlWave0Done,     // wave 0 at the merge
    kTlMerged,        // every wave at the merge: first barrier of the merge passed
    kTlStoresIssued,  // the workgroup's partial is on its way to memory
    kTlStored,        // ... and has arrived there (the wait ahead of the ticket)
    kTlTicket,        // ticket drawn, the workgroup knows whether it folds
    kTlFoldListed,    // fold: maxima and sums of the partials read, the non-empty ones listed
    kTlFoldDone,      // fold: output written
    kTlRows,          // (a count, not a time) rows wave 0 listed in the first round
    kTlRounds,        // (a count) rounds of the workgroup
    kTlAlive,         // (a count) nodes of the workgroup's tiles that survived the gates
    kTlWaveEnd = 24,       // + wave: the wave arrives at the merge
    kTlWaveRows = 32,      // + wave: (a count) rows the wave listed over all rounds
    kTlWaveScanned = 40,   // + wave: the wave's first round is scanned
    kTlWaveIssued = 48,    // + wave: its first batch of value rows is asked for
    kTlWaveConsumed = 56,  // + wave: ... and in the sums
    kTlCols = 64
};

#ifdef HIRA_TIMELINE
struct Timeline {
    static constexpr bool kOn = true;
    unsigned long long* row;
    unsigned long long rows = 0;
    // (a launch without a statistics buffer records nothing)
    __device__ __forceinline__ explicit Timeline(const SearchParams& p)
        : row(p.stats == nullptr ? nullptr
                                 : p.stats + (((size_t)blockIdx.z * gridDim.y + blockIdx.y) * gridDim.x +
                                              blockIdx.x) * kTlCols) {}
    __device__ __forceinline__ void stamp(int k) const {
        if (threadIdx.x == 0 && row) row[k] = (unsigned long long)wall_clock64();
    }
    __device__ __forceinline__ void stamp_wave(int k) const {
        if ((threadIdx.x & 63) == 0 && row) row[k + (threadIdx.x >> 6)] = (unsigned long long)wall_clock64();
    }
    __device__ __forceinline__ void set(int k, unsigned long long v) const {
        if (threadIdx.x == 0 && row) row[k] = v;
    }
    __device__ __forceinline__ void set_wave(int k, unsigned long long v) const {
        if ((threadIdx.x & 63) == 0 && row) row[k + (threadIdx.x >> 6)] = v;
    }
    __device__ __forceinline__ void add_rows(int n) { rows += (unsigned long long)n; }
};
#else
struct Timeline {
    static constexpr bool kOn = false;
    static constexpr unsigned long long rows = 0;
    __device__ __forceinline__ explicit Timeline(const SearchParams&) {}
    __device__ __forceinline__ void stamp(int) const {}
    __device__ __forceinline__ void stamp_wave(int) const {}
    __device__ __forceinline__ void set(int, unsigned long long) const {}
    __device__ __forceinline__ void set_wave(int, unsigned long long) const {}
    __device__ __forceinline__ void add_rows(int) const {}
};
#endif

}  // namespace hira
