// Hand-over protocol of the one-launch ("paired") transforms: the sixteen workgroups of a limb run the limb's sixteen first-pass
// tiles, then its sixteen second-pass tiles, and a second-pass tile may only start when all first-pass tiles are complete.
//
// The protocol makes no assumption about which workgroups are resident or in which order they start, and no wait in it is
// unbounded, so a launch completes all its work wherever at least one of its workgroups runs:
//   claim   a workgroup claims its own first-pass tile (bit in the claim mask) before it runs it;
//   steal   a workgroup whose wait for the limb's sixteen first-pass tiles runs past `spin_steal` polls claims a tile that
//           nobody has claimed yet (its workgroup has not started) and runs that too - the workgroup that starts late finds
//           its tile taken and has nothing left to do;
//   defer   when every tile is claimed and the count still does not complete within `spin_max` polls (the claimers are
//           running, only slowly), the workgroup records its second-pass tiles in the todo mask instead of waiting on;
//   finish  every workgroup counts itself out once it knows whether it goes on or defers (before its own second pass: nothing
//           below depends on that); the last of the sixteen to count out - by then every first-pass tile is complete, because a
//           claimer completes its tiles before it counts out - runs the second-pass tiles of the todo mask and returns the
//           four words to zero, so a launch leaves them as it found them (it can be replayed from a HIP graph).
// The decisions are taken by one lane per workgroup with atomic operations on the limb's four words; this file holds exactly
// that logic, as functions that compile for the device (relaxed atomics at agent scope) and for the host (the model test runs
// it with one thread per workgroup).
#pragma once
#include <hip/hip_runtime.h>

namespace ckks {
namespace pair {

constexpr unsigned TILES = 16;
constexpr unsigned ALL = (1u << TILES) - 1;
// what the deciding lane tells its workgroup
constexpr unsigned GO = 16;        // all first-pass tiles are complete: run the second pass of the tiles this workgroup ran
constexpr unsigned DEFER = 17;     // the wait ran out: leave the second-pass tiles to the last workgroup out
constexpr unsigned LEAVE = 18;     // nothing to do (the own tile was taken by another workgroup)
// Words of a limb.  The three words that every workgroup of a launch touches lie in 128-byte lines of their own: atomics on one
// line are carried out one after the other, and the polls of the count should not queue behind the claims and the counting out.
constexpr int WORDS = 128;         // per limb (four lines)
constexpr int CLAIM = 0, DONE = 32, LEFT = 64, TODO = 96, DEFERRED_TOTAL = 97, STOLEN_TOTAL = 98;      // the totals only ever grow (statistics)

// atomics: on the device relaxed operations at agent scope (carried out in the cache all compute units share); on the host the
// compiler's sequentially consistent builtins
struct Atomics {
    static __host__ __device__ __forceinline__ unsigned load(unsigned* p) {
#if defined(__HIP_DEVICE_COMPILE__)
        return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#else
        return __atomic_load_n(p, __ATOMIC_SEQ_CST);
#endif
    }
    static __host__ __device__ __forceinline__ void store(unsigned* p, unsigned v) {
#if defined(__HIP_DEVICE_COMPILE__)
        __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#else
        __atomic_store_n(p, v, __ATOMIC_SEQ_CST);
#endif
    }
    static __host__ __device__ __forceinline__ unsigned fetch_add(unsigned* p, unsigned v) {
#if defined(__HIP_DEVICE_COMPILE__)
        return __hip_atomic_fetch_add(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#else
        return __atomic_fetch_add(p, v, __ATOMIC_SEQ_CST);
#endif
    }
    static __host__ __device__ __forceinline__ unsigned fetch_or(unsigned* p, unsigned v) {
#if defined(__HIP_DEVICE_COMPILE__)
        return __hip_atomic_fetch_or(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#else
        return __atomic_fetch_or(p, v, __ATOMIC_SEQ_CST);
#endif
    }
    static __host__ __device__ __forceinline__ void pause() {
#if defined(__HIP_DEVICE_COMPILE__)
        __builtin_amdgcn_s_sleep(4);
#endif
    }
};

// First decision of a workgroup: its own tile, or LEAVE when another workgroup has taken it.
__host__ __device__ __forceinline__ unsigned claim_own(unsigned* w, unsigned tile, bool stealing) {
    if (!stealing) return tile;                      // tiles are never taken over in this form: no claim needed
    const unsigned old = Atomics::fetch_or(w + CLAIM, 1u << tile);
    return (old >> tile) & 1u ? LEAVE : tile;
}
// After a first-pass tile of this workgroup is complete (its stores acknowledged): count it, then decide what comes next -
// another first-pass tile to run (0..15), GO, or DEFER.
__host__ __device__ __forceinline__ unsigned tile_done_then_decide(unsigned* w, bool stealing, unsigned spin_steal, unsigned spin_max) {
    (void)Atomics::fetch_add(w + DONE, 1u);
    for (;;) {
        for (unsigned n = 0; n <= spin_steal; n++) {
            if (Atomics::load(w + DONE) == TILES) return GO;
            Atomics::pause();
        }
        if (stealing) {
            const unsigned claimed = Atomics::load(w + CLAIM) & ALL;
            if (claimed != ALL) {
                const unsigned s = (unsigned)__builtin_ctz(~claimed & ALL);
                const unsigned old = Atomics::fetch_or(w + CLAIM, 1u << s);
                if (!((old >> s) & 1u)) { (void)Atomics::fetch_add(w + STOLEN_TOTAL, 1u); return s; }      // taken over: run it
                continue;                                    // its own workgroup (or another waiter) was quicker: wait on
            }
        }
        // every tile is in somebody's hands: they are running
        for (unsigned n = 0; n < spin_max; n++) {
            if (Atomics::load(w + DONE) == TILES) return GO;
            Atomics::pause();
        }
        return DEFER;
    }
}
// A workgroup that defers records the tiles whose second pass it leaves undone.
__host__ __device__ __forceinline__ void defer(unsigned* w, unsigned mine) {
    if (mine) (void)Atomics::fetch_or(w + TODO, mine);
}
// Counting out.  Returns the todo mask with bit 31 set if this workgroup is the last of the limb's sixteen to leave (it then runs
// the second pass of those tiles and calls reset), 0 otherwise.
__host__ __device__ __forceinline__ unsigned leave(unsigned* w) {
    const unsigned before = Atomics::fetch_add(w + LEFT, 1u);
    if (before + 1u != TILES) return 0u;
    return 0x80000000u | (Atomics::load(w + TODO) & ALL);
}
__host__ __device__ __forceinline__ void reset(unsigned* w, unsigned finished_here) {
    if (finished_here) (void)Atomics::fetch_add(w + DEFERRED_TOTAL, (unsigned)__builtin_popcount(finished_here));
    Atomics::store(w + CLAIM, 0u);
    Atomics::store(w + DONE, 0u);
    Atomics::store(w + TODO, 0u);
    Atomics::store(w + LEFT, 0u);
}

}  // namespace pair
}  // namespace ckks
