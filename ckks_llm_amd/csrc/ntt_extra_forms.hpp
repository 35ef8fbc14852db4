// Two more launch forms of the transform, built only with CKKS_NTT_EXTRA_FORMS (the default library leaves them out: both lose
// to two launches at every batch size on this hardware and exist for experiments): mode 3, one workgroup per limb, and mode 2,
// the chained transform with its finishing launch.  Included by ntt.hip inside namespace ckks, behind the tile functions.
// ------------------------------------------------------------------------------------------------------------
// Whole-limb transform: one workgroup carries one limb through both passes in one launch.
//
// The workgroup is GROUPS groups of 256 lanes; each group takes every GROUPS-th tile of the first pass, the workgroup waits
// until all its stores have left the compute unit, then the groups take the tiles of the second pass.  Nothing is exchanged
// between workgroups, so there is no synchronisation beyond the workgroup barrier.  Between the passes the limb is not
// read back from HBM: its lines are still in the XCD's L2 or, once displaced from there, in the memory-side cache, because
// only (resident workgroups) x N x 8 bytes are in that state at any time.  The second-pass loads bypass the L1, which may
// still hold pre-transform copies of the same lines from the first pass of this very workgroup.
// ------------------------------------------------------------------------------------------------------------
template <class AR, int SA, int SB, bool INVERSE, int GROUPS>
__global__ __launch_bounds__(256 * GROUPS) void ntt_limb_kernel(NttArgs a) {
    typedef StridedCfg<SA, SB> CS;
    typedef RowCfg<SA, SB> CR;
    static_assert(CS::THREADS == 256 && CR::THREADS == 256 && CS::TILES == CR::TILES, "whole-limb kernel: tile shapes must agree");
    static_assert(CS::TILES % GROUPS == 0, "whole-limb kernel: tiles must divide among the groups");
    constexpr int TILES = CS::TILES;
    constexpr long N = 1l << (SA + SB);
    constexpr int LDS_WORDS = CS::LDS_WORDS > CR::LDS_WORDS ? CS::LDS_WORDS : CR::LDS_WORDS;
    typedef typename AR::TW TW;
    __shared__ typename AR::V lds_all[GROUPS][LDS_WORDS];
    const unsigned grp = threadIdx.x / 256, tid = threadIdx.x % 256;
    typename AR::V* lds = lds_all[grp];
    int prime;
    u64* limb = limb_ptr(a, blockIdx.x, N, prime);
    const AR ar(a.primes[prime]);
    const TW* __restrict__ tw = (const TW*)a.tw + (long)prime * N;
#pragma unroll 1
    for (int t = grp; t < TILES; t += GROUPS) {
        if (!INVERSE) strided_tile<AR, SA, SB, false, false>(limb, t, tw, ar, lds, tid);
        else row_tile<AR, SA, SB, true, false>(limb, t, tw, ar, lds, tid);
        __syncthreads();
    }
    // every store of the first pass has been acknowledged by the L2 before any lane starts the second pass
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
#pragma unroll 1
    for (int t = grp; t < TILES; t += GROUPS) {
        if (!INVERSE) row_tile<AR, SA, SB, false, true>(limb, t, tw, ar, lds, tid);
        else strided_tile<AR, SA, SB, true, true>(limb, t, tw, ar, lds, tid);
        __syncthreads();
    }
}

// ------------------------------------------------------------------------------------------------------------
// Chained transform: both passes in ONE launch, the data between them held in the XCD's L2.
//
// A two-launch transform moves every limb through HBM twice.  Here the second pass of a limb runs on the same XCD as its first
// pass, a few microseconds later, while the limb's lines (512 KiB at N = 2^16, written in place by the first pass) are still
// dirty in that XCD's 4 MiB L2: HBM sees one read and one write per limb.
//
// Order of work.  The grid is one-dimensional and not persistent.  Workgroup b belongs to chain x = b mod 8 and takes slot
// s = b / 8 of that chain; the hardware hands consecutive workgroups of a grid to the XCDs in turn, so a chain's workgroups all
// run on one XCD.  A chain works through the limbs x, x + 8, x + 16, .. in entries of TILES workgroups (one pass of one limb):
//     P1(k=0) .. P1(k=skew-1) | P1(k=skew) P2(k=0) | P1(k=skew+1) P2(k=1) | ...
// so that the second pass of a limb is dispatched while later limbs' first passes keep the compute units busy.
//
// Synchronisation.  A first-pass workgroup waits for nothing; when its stores have reached the L2 it adds 1 to the limb's
// completion word.  A second-pass workgroup waits until that word reads TILES.  Workgroups of a grid start in the order of their
// index, so what it waits for has started before it; the wait is bounded by a poll count all the same.
// Nothing depends on the placement or on the wait for correctness: every workgroup reads the XCD it really runs on from the
// hardware register; a first-pass workgroup that finds itself on another XCD than its chain's adds a mark to the completion word
// instead of the plain 1, and a second-pass workgroup that is on the wrong XCD, sees a mark, or runs out of polls does not touch
// the data: it records its tile in the limb's `todo` word and leaves.  A second launch (ntt_chain_finish_kernel, one workgroup
// per limb) runs the recorded tiles - after the kernel boundary every store is visible everywhere - and returns both words to
// zero for the next transform.  Every workgroup of both launches ends after a bounded number of steps.
// ------------------------------------------------------------------------------------------------------------
constexpr unsigned CHAIN_XCDS = 8;
constexpr unsigned CHAIN_MARK = 0x10000u;          // added by a first-pass workgroup that ran on an unexpected XCD
struct ChainArgs {
    unsigned* done;            // [limb] completion word of the first pass
    unsigned* todo;            // [limb] bit t: second-pass tile t was left to the finishing launch
    unsigned* stats;           // [0]: tiles left to the finishing launch since the context was created
    unsigned limbs, kmax, skew, spin_max;
    unsigned zero;             // 0, but not known to the compiler: "add zero" stays a read-modify-write executed at the L2
    unsigned long long xcc_of; // nibble x: the XCD that runs chain x
};


template <class AR, int SA, int SB, bool INVERSE>
__global__ __launch_bounds__(256) void ntt_chain_kernel(NttArgs a, ChainArgs ch) {
    typedef StridedCfg<SA, SB> CS;
    typedef RowCfg<SA, SB> CR;
    static_assert(CS::THREADS == 256 && CR::THREADS == 256 && CS::TILES == CR::TILES && CS::TILES <= 16, "chained kernel: tile shapes");
    constexpr unsigned TILES = CS::TILES;
    constexpr long N = 1l << (SA + SB);
    constexpr int LDS_WORDS = CS::LDS_WORDS > CR::LDS_WORDS ? CS::LDS_WORDS : CR::LDS_WORDS;
    typedef typename AR::TW TW;
    __shared__ typename AR::V lds[LDS_WORDS];
    __shared__ unsigned go;
    const unsigned x = blockIdx.x % CHAIN_XCDS;
    unsigned second, k, tile;
    chain_slot(blockIdx.x / CHAIN_XCDS, TILES, ch.skew, second, k, tile);
    const unsigned limb_id = x + CHAIN_XCDS * k;
    if (k >= ch.kmax || limb_id >= ch.limbs) return;                            // uniform over the workgroup
    const unsigned xcc = __builtin_amdgcn_s_getreg((3 << 11) | 20) & 15u;       // XCC_ID[3:0]
    const bool placed = xcc == (unsigned)((ch.xcc_of >> (4 * x)) & 15u);
    int prime;
    u64* limb = limb_ptr(a, limb_id, N, prime);
    const AR ar(a.primes[prime]);
    const TW* __restrict__ tw = (const TW*)a.tw + (long)prime * N;
    if (!second) {
        if (!INVERSE) strided_tile<AR, SA, SB, false, false>(limb, tile, tw, ar, lds, threadIdx.x);
        else row_tile<AR, SA, SB, true, false>(limb, tile, tw, ar, lds, threadIdx.x);
        // every store of this tile has been acknowledged by the L2 before the completion word moves
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        __builtin_amdgcn_s_waitcnt(0);
        __syncthreads();
        if (threadIdx.x == 0) atomicAdd(&ch.done[limb_id], placed ? 1u : CHAIN_MARK + 1u);
        return;
    }
    if (threadIdx.x == 0) {
        unsigned ok = placed ? 1u : 0u;
        if (ok) {
            unsigned v = 0;
            for (unsigned n = 0; n < ch.spin_max; n++) {
                v = atomicAdd(&ch.done[limb_id], ch.zero);
                if (v >= TILES) break;
                __builtin_amdgcn_s_sleep(8);
            }
            ok = v == TILES ? 1u : 0u;
        }
        if (!ok) atomicOr(&ch.todo[limb_id], 1u << tile);
        go = ok;
    }
    __syncthreads();
    if (!go) return;
    // second-pass loads bypass this compute unit's L1 (which may hold pre-transform copies of the same lines) and are served by the L2
    if (!INVERSE) row_tile<AR, SA, SB, false, true>(limb, tile, tw, ar, lds, threadIdx.x);
    else strided_tile<AR, SA, SB, true, true>(limb, tile, tw, ar, lds, threadIdx.x);
}

// One workgroup per limb: runs the second-pass tiles that the chained launch left behind, then clears the limb's words.
template <class AR, int SA, int SB, bool INVERSE>
__global__ __launch_bounds__(256) void ntt_chain_finish_kernel(NttArgs a, ChainArgs ch) {
    typedef StridedCfg<SA, SB> CS;
    typedef RowCfg<SA, SB> CR;
    constexpr long N = 1l << (SA + SB);
    constexpr int LDS_WORDS = CS::LDS_WORDS > CR::LDS_WORDS ? CS::LDS_WORDS : CR::LDS_WORDS;
    typedef typename AR::TW TW;
    __shared__ typename AR::V lds[LDS_WORDS];
    __shared__ unsigned mask_s;
    const unsigned limb_id = blockIdx.x;
    if (limb_id >= ch.limbs) return;
    if (threadIdx.x == 0) mask_s = ch.todo[limb_id];
    __syncthreads();
    const unsigned mask = mask_s;
    if (mask) {
        int prime;
        u64* limb = limb_ptr(a, limb_id, N, prime);
        const AR ar(a.primes[prime]);
        const TW* __restrict__ tw = (const TW*)a.tw + (long)prime * N;
#pragma unroll 1
        for (unsigned tile = 0; tile < (unsigned)CS::TILES; tile++) {
            if (!((mask >> tile) & 1u)) continue;
            if (!INVERSE) row_tile<AR, SA, SB, false, false>(limb, tile, tw, ar, lds, threadIdx.x);
            else strided_tile<AR, SA, SB, true, false>(limb, tile, tw, ar, lds, threadIdx.x);
            __syncthreads();
        }
    }
    if (threadIdx.x == 0) {
        ch.done[limb_id] = 0;
        ch.todo[limb_id] = 0;
        if (mask) atomicAdd(ch.stats, (unsigned)__builtin_popcount(mask));
    }
}


constexpr unsigned CHAIN_MAX_LIMBS = 65536;
static int ensure_chain(ckks_ctx* c) {
    if (c->d_ntt_chain) return CKKS_OK;
    const size_t bytes = (2 * (size_t)CHAIN_MAX_LIMBS + 16) * sizeof(unsigned);
    if (hipMalloc(&c->d_ntt_chain, bytes) != hipSuccess) { set_error("NTT: cannot allocate the completion words of the chained transform"); return CKKS_E_NOMEM; }
    CKKS_HIP_TRY(hipMemsetAsync(c->d_ntt_chain, 0, bytes, c->stream));
    return CKKS_OK;
}

template <class AR, int SA, int SB>
static int launch_chain(ckks_ctx* c, NttArgs args, int limbs, bool inverse) {
    int rc = ensure_chain(c);
    if (rc) return rc;
    args.limb_base = 0;
    args.limbs_total = (unsigned)limbs;
    args.mid = nullptr;
    ChainArgs ch;
    ch.done = (unsigned*)c->d_ntt_chain;
    ch.todo = ch.done + CHAIN_MAX_LIMBS;
    ch.stats = ch.todo + CHAIN_MAX_LIMBS;
    ch.limbs = (unsigned)limbs;
    ch.kmax = ((unsigned)limbs + CHAIN_XCDS - 1) / CHAIN_XCDS;
    ch.skew = c->chain_skew > 0 ? (unsigned)c->chain_skew : 1u;
    if (ch.skew > ch.kmax) ch.skew = ch.kmax;
    // about 5 ms of polls by default, far beyond any wait of a healthy launch; 0 polls (a test setting) leaves every second-pass
    // tile to the finishing launch
    ch.spin_max = c->chain_spin >= 0 ? (unsigned)c->chain_spin : 20000u;
    ch.zero = 0;
    ch.xcc_of = 0x76543210ull;
    const unsigned blocks = chain_slots(ch.kmax, StridedCfg<SA, SB>::TILES, ch.skew) * CHAIN_XCDS;
    if (!inverse) {
        hipLaunchKernelGGL((ntt_chain_kernel<AR, SA, SB, false>), dim3(blocks), dim3(256), 0, c->stream, args, ch);
        hipLaunchKernelGGL((ntt_chain_finish_kernel<AR, SA, SB, false>), dim3((unsigned)limbs), dim3(256), 0, c->stream, args, ch);
    } else {
        hipLaunchKernelGGL((ntt_chain_kernel<AR, SA, SB, true>), dim3(blocks), dim3(256), 0, c->stream, args, ch);
        hipLaunchKernelGGL((ntt_chain_finish_kernel<AR, SA, SB, true>), dim3((unsigned)limbs), dim3(256), 0, c->stream, args, ch);
    }
    CKKS_HIP_TRY(hipGetLastError());
    return CKKS_OK;
}
// tiles that second-pass workgroups of chained transforms have left to the finishing launch so far (synchronises the stream)
int ntt_chain_deferred(ckks_ctx* c, long* tiles) {
    *tiles = 0;
    if (!c->d_ntt_chain) return CKKS_OK;
    CKKS_HIP_TRY(hipStreamSynchronize(c->stream));
    unsigned v = 0;
    CKKS_HIP_TRY(hipMemcpy(&v, (unsigned*)c->d_ntt_chain + 2 * (size_t)CHAIN_MAX_LIMBS, sizeof(v), hipMemcpyDeviceToHost));
    *tiles = v;
    return CKKS_OK;
}

template <class AR, int SA, int SB>
static int launch_whole_limb(ckks_ctx* c, NttArgs args, int limbs, bool inverse) {
    const int groups_env = 0;                          // 2: workgroups of 512 lanes instead of 1024 (an experiment's setting)
    args.limb_base = 0;
    args.limbs_total = (unsigned)limbs;
    args.mid = nullptr;
    if (groups_env == 2) {
        if (!inverse) hipLaunchKernelGGL((ntt_limb_kernel<AR, SA, SB, false, 2>), dim3(limbs), dim3(512), 0, c->stream, args);
        else hipLaunchKernelGGL((ntt_limb_kernel<AR, SA, SB, true, 2>), dim3(limbs), dim3(512), 0, c->stream, args);
    } else {
        if (!inverse) hipLaunchKernelGGL((ntt_limb_kernel<AR, SA, SB, false, 4>), dim3(limbs), dim3(1024), 0, c->stream, args);
        else hipLaunchKernelGGL((ntt_limb_kernel<AR, SA, SB, true, 4>), dim3(limbs), dim3(1024), 0, c->stream, args);
    }
    CKKS_HIP_TRY(hipGetLastError());
    return CKKS_OK;
}

