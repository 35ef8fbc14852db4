// Batched RNS negacyclic NTT / iNTT for gfx950.
//
// Replaces Context_23::ToNTTInplace / FromNTTInplace (+ _for_externalProduct) and their eight kernels
// (Context_23.cuh:847-930, ntt_60bit.cuh:421-1318).  Same transform: forward = Cooley-Tukey, natural ->
// bit-reversed order, twiddle of stage m / group i is psi_table[m + i]; inverse = Gentleman-Sande with
// psiinv_table[h + i], scaled by N^-1; outputs fully reduced.
//
// Decomposition (N = N1 * N2, N1 = 2^SA >= N2 = 2^SB):
//   forward : "strided" pass = first SA stages on columns (elements N2 apart), a workgroup owns all N1 rows of
//             CW adjacent columns (CW*8 B = one 128 B line per row); then the "row" pass = last SB stages on
//             rows of N2 contiguous words.  Inverse runs the mirror image (row pass first).
//   Each pass keeps R = 2^ceil(S/2) values per lane in registers and does its S stages in two register rounds
//   with one LDS exchange in between; every HBM access of both passes is a full 128 B line per 16 lanes.
//   All columns of the strided pass share the same 2^SA - 1 twiddles; the row pass reads each of the other
//   N - N1 twiddles exactly once per limb.
//
// Arithmetic back ends (modarith.hpp): IntArith (any q < 2^62) and F64Arith (q < 2^41): values are exact signed
// integers in doubles, a*w mod q = fma(-rint(a*w/q), q, a*w) evaluated with the two-product trick, no
// conditional corrections inside the butterflies.  Range analysis for F64Arith (|w| <= q/2):
//   forward: each stage adds at most 0.51 q to |x|, so after 16 stages |x| < 9.2 q < 2^45; the quotient
//            estimate rint(h * qinv) is off by < 2^-8, so |a*w - c*q| < 0.51 q.
//   inverse: the sum branch doubles |x| per stage; values are reduced to (-q/2, q/2] between the two passes, so
//            |x| < 2^8 * q < 2^49 inside a pass and every integer involved stays below 2^53.
// Between the two passes of one transform the buffer holds back-end specific words (lazy residues in [0,4q) /
// [0,2q) for IntArith, raw double bit patterns for F64Arith); after the second pass it holds canonical residues.
#include <cstddef>
#include <cstdlib>
#include <mutex>
#include <string>
#include <type_traits>

#include "context.hpp"
#include "ntt_core.hpp"
#include "pair_protocol.hpp"

namespace ckks {


// ------------------------------------------------------------------------------------------------------------
// strided pass (first SA forward stages / last SA inverse stages): one tile = CW adjacent columns, all N1 rows
// ------------------------------------------------------------------------------------------------------------

// The two questions that a workgroup of a paired launch asks of its limb's protocol words (pair_protocol.hpp) with atomics that
// return an answer - the claim of its own first-pass tile and its counting out - ride inside a tile: lane 0 asks behind the
// tile's own loads (memory operations return in the order of their issue, so an answer that queues behind the other workgroups'
// atomics on the same words does not hold the loads up) and publishes the answer in LDS, the claim just ahead of the tile's
// first barrier, the count at the tile's end.  Behind that barrier every lane knows whether a claimed tile is this workgroup's;
// up to there a tile only reads global memory and writes LDS, so a tile that turns out to be another's leaves no trace.
// Default: nothing to ask.
struct TileClaim {
    unsigned* lds = nullptr;       // where the answer is published (nullptr: nothing to ask)
    unsigned* words = nullptr;     // the limb's protocol words
    unsigned tile = 0;
    bool counting_out = false;     // false: the claim of a first-pass tile; true: the counting out, inside a second-pass tile
    // start() only issues the atomic and returns what it will bring, untouched: anything computed from it here would make the
    // wave wait for it at this point; publish() is where it is first looked at
    __device__ __forceinline__ unsigned start(unsigned tid) const {
        unsigned v = 0;
        if (lds && tid == 0) {
            asm volatile("" ::: "memory");
            v = counting_out ? pair::Atomics::fetch_add(words + pair::LEFT, 1u) : pair::Atomics::fetch_or(words + pair::CLAIM, 1u << tile);
        }
        return v;
    }
    // claim: the tile, or LEAVE if it was taken; counting out: how many had left before (the last one out sees TILES - 1)
    __device__ __forceinline__ void publish(unsigned tid, unsigned raw) const {
        if (lds && tid == 0) *lds = counting_out ? raw : ((raw >> tile) & 1u ? pair::LEAVE : tile);
    }
    __device__ __forceinline__ bool lost() const { return lds && !counting_out && *lds == pair::LEAVE; }
};

// PAIRED: the tile is one half of a paired transform - what it hands to or takes from the other pass moves as shared accesses
template <class AR, int SA, int SB, bool INVERSE, bool COHERENT, bool COMPACT = false, bool EMBED = false, bool PAIRED = false>
__device__ __forceinline__ void strided_tile(u64* limb, unsigned tile, const typename AR::TW* __restrict__ tw, const AR& ar,
                                             typename AR::V* lds, unsigned tid, char* mid_limb = nullptr, const NttArgs* ea = nullptr,
                                             unsigned poly = 0, bool lift = false, const TileClaim& claim = TileClaim()) {
    typedef StridedCfg<SA, SB> C;
    constexpr int S1 = C::S1, R = C::R, N2 = C::N2, G = C::G, CW = C::CW;
    typedef typename AR::V V;
    const unsigned cl = tid % CW, g = tid / CW;
    u64* col = limb + tile * CW + cl;
    V v[R];
    if (!INVERSE) {
        if constexpr (EMBED) {
            const unsigned kmask = (1u << ea->embed_logk) - 1, gmask = (1u << ea->embed_loggap) - 1;
            if (SA == 8 && SB == 8 && ea->embed_logk == 9) {
                // N = 2^16, rank 512 (the BERT layer's ring): the tile's 16 columns x 256 rows are 128 coefficients of each of 32 sample
                // rows.  Staged through LDS so that a wave reads 512 contiguous bytes of one sample row; the 16-byte k index is
                // xor-swizzled with the column so that neither the staging writes nor the register reads conflict on the banks.
                // all sample pointers first, then all coefficients, unconditionally (a coefficient that the embedding leaves zero is
                // read and dropped): sixteen independent loads in flight per lane instead of sixteen pointer-then-data round trips
                const u64* row[16];
                u64 x[16];
#pragma unroll
                for (int it = 0; it < 16; it++) {
                    const unsigned sidx = (it * 256 + tid) >> 7;
                    const unsigned off = (sidx >> 4) * 256 + tile * CW + (sidx & 15);
                    row[it] = ea->embed_mlwe[off >> ea->embed_loggap] + (long)poly * ea->embed_n1 + (tid & 127);
                }
#pragma unroll
                for (int it = 0; it < 16; it++) x[it] = *row[it];
#pragma unroll
                for (int it = 0; it < 16; it++) {
                    const unsigned sidx = (it * 256 + tid) >> 7, n = tid & 127, clx = sidx & 15;
                    const unsigned off = (sidx >> 4) * 256 + tile * CW + clx;
                    u64 y = (off & gmask) == 0 ? x[it] : 0;
                    if (lift) y = embed_lift(y, *ea);
                    lds[sidx * 128 + (n ^ (clx << 1))] = ar.from_canonical(y);
                }
                __syncthreads();
#pragma unroll
                for (int j = 0; j < R; j++) v[j] = lds[((g & 1) * 16 + cl) * 128 + (((g >> 1) + 8 * j) ^ (cl << 1))];
                __syncthreads();
            } else
#pragma unroll
            for (int j = 0; j < R; j++) {
                const unsigned pos = (g + j * G) * N2 + tile * CW + cl;
                const unsigned n = pos >> ea->embed_logk, off = pos & kmask;
                const u64 raw = ea->embed_mlwe[off >> ea->embed_loggap][(long)poly * ea->embed_n1 + n];     // unconditional: loads overlap
                u64 x = (off & gmask) == 0 ? raw : 0;
                if (lift) x = embed_lift(x, *ea);
                v[j] = ar.from_canonical(x);
            }
        } else {
#pragma unroll
            for (int j = 0; j < R; j++) v[j] = ar.from_canonical(load_word<COHERENT>(col + (long)(g + j * G) * N2));
        }
        const unsigned claimed = claim.start(tid);
        fwd_spread<AR, SA, S1>(v, tw, 1u, ar);
        ar.round_end(v);
#pragma unroll
        for (int j = 0; j < R; j++) lds[(g + j * G) * CW + cl] = v[j];
        claim.publish(tid, claimed);
        __syncthreads();
        if (claim.lost()) return;                       // uniform: another workgroup has taken this tile; nothing was stored yet
#pragma unroll
        for (int j = 0; j < R; j++) v[j] = lds[(g * R + j) * CW + cl];
        fwd_packed<AR, SA, S1>(v, tw, 1u, g, ar);
        if constexpr (COMPACT) {
            if constexpr (R == 16) mid_store_columns<AR, PAIRED>(mid_limb, tile, g, cl, v, ar);      // the 5-byte form exists for 256 x 256 only
        } else {
#pragma unroll
            for (int j = 0; j < R; j++) put<PAIRED>(col + (long)(g * R + j) * N2, ar.to_mid_fwd(v[j]));
        }
    } else {
        if constexpr (COMPACT) {
            const char* piece = mid_piece(mid_limb, tile, g);
#pragma unroll
            for (int j = 0; j < R; j++)
                v[j] = ar.dec40(get<PAIRED>(reinterpret_cast<const unsigned*>(piece + (j * 16 + cl) * 4)),
                                get<PAIRED>(reinterpret_cast<const unsigned char*>(piece + 1024 + j * 16 + cl)));
        } else {
#pragma unroll
            for (int j = 0; j < R; j++) v[j] = ar.from_mid(PAIRED ? get<true>(col + (long)(g * R + j) * N2) : load_word<COHERENT>(col + (long)(g * R + j) * N2));
        }
        const unsigned counted = claim.start(tid);
        inv_packed<AR, SA, S1>(v, tw, 1u, g, ar);
        ar.round_end(v);
#pragma unroll
        for (int j = 0; j < R; j++) lds[(g * R + j) * CW + cl] = v[j];
        __syncthreads();
#pragma unroll
        for (int j = 0; j < R; j++) v[j] = lds[(g + j * G) * CW + cl];
        inv_spread<AR, SA, S1, 1>(v, tw, 1u, ar);
        // stage 0 (h = 1): pairs (j, j + R/2), N^-1 folded in
#pragma unroll
        for (int j = 0; j < R / 2; j++) {
            u64 ox, oy;
            ar.gs_last(v[j], v[j + R / 2], ox, oy);
            store_word<COHERENT>(col + (long)(g + j * G) * N2, ox);
            store_word<COHERENT>(col + (long)(g + (j + R / 2) * G) * N2, oy);
        }
        claim.publish(tid, counted);
    }
}

template <class AR, int SA, int SB, bool INVERSE, bool COMPACT = false, bool EMBED = false>
__global__ __launch_bounds__((StridedCfg<SA, SB>::THREADS)) void ntt_strided_pass(NttArgs a) {
    constexpr long N = 1l << (SA + SB);
    __shared__ typename AR::V lds[StridedCfg<SA, SB>::LDS_WORDS];
    int prime;
    const unsigned l = a.reverse ? gridDim.y - 1 - blockIdx.y : blockIdx.y;
    u64* limb = limb_ptr(a, l, N, prime);
    const AR ar(a.primes[prime]);
    strided_tile<AR, SA, SB, INVERSE, false, COMPACT, EMBED>(limb, blockIdx.x, (const typename AR::TW*)a.tw + (long)prime * N, ar, lds, threadIdx.x,
                                                             COMPACT ? a.mid + l * MID_LIMB_BYTES : nullptr, &a,
                                                             EMBED ? limb_poly(a, l) : 0u, EMBED && prime == a.start_mod_idx);
}

// ------------------------------------------------------------------------------------------------------------
// row pass (last SB forward stages / first SB inverse stages): one tile = ROWS rows of N2 contiguous words
// ------------------------------------------------------------------------------------------------------------

template <class AR, int SA, int SB, bool INVERSE, bool COHERENT, bool COMPACT = false, bool PAIRED = false>
__device__ __forceinline__ void row_tile(u64* limb, unsigned tile, const typename AR::TW* __restrict__ tw, const AR& ar,
                                         typename AR::V* lds, unsigned tid, char* mid_limb = nullptr, const TileClaim& claim = TileClaim(),
                                         const u64* addend = nullptr, u64 addend_q = 0) {
    typedef RowCfg<SA, SB> C;
    constexpr int S1 = C::S1, R = C::R, N2 = C::N2, U = C::U, N1 = C::N1, ROWS = C::ROWS;
    typedef typename AR::V V;
    const unsigned u = tid % U, rl = tid / U;
    const unsigned row = tile * ROWS + rl;
    u64* rp = limb + (long)row * N2;
    V* lrow = lds + rl * C::PITCH;
    const unsigned tw_off = N1 + row;
    V v[R];
    if (!INVERSE) {
        if constexpr (COMPACT) {
            if constexpr (R == 16) {
                unsigned lo[16], hi[16];
                mid_load_row_raw<PAIRED>(mid_limb, tile, rl, u, lo, hi);
#pragma unroll
                for (int j = 0; j < R; j++) v[j] = mid_decode_row(ar, lo[j], hi[j], rl);
            }
        } else {
#pragma unroll
            for (int j = 0; j < R; j++) v[j] = ar.from_mid(PAIRED ? get<true>(rp + u + j * U) : load_word<COHERENT>(rp + u + j * U));
        }
        const unsigned counted = claim.start(tid);
        fwd_spread<AR, SB, S1>(v, tw, tw_off, ar);
        ar.round_end(v);
#pragma unroll
        for (int j = 0; j < R; j++) lrow[padded(u + j * U)] = v[j];
        __syncthreads();
#pragma unroll
        for (int j = 0; j < R; j++) v[j] = lrow[padded(u * R + j)];
        fwd_packed<AR, SB, S1>(v, tw, tw_off, u, ar);
        __syncthreads();
        // transpose back through LDS so the global stores are coalesced
#pragma unroll
        for (int j = 0; j < R; j++) lrow[padded(u * R + j)] = v[j];
        __syncthreads();
#pragma unroll
        for (int j = 0; j < R; j++) {
            u64 w = ar.to_canonical_fwd(lrow[padded(u + j * U)]);
            // a forward transform whose result is added to a limb in the NTT domain (null for every plain transform: folded away)
            if (addend) w = csub(w + addend[(long)row * N2 + u + j * U], addend_q);
            store_word<COHERENT>(rp + u + j * U, w);
        }
        claim.publish(tid, counted);
    } else {
        u64 raw[R];
#pragma unroll
        for (int j = 0; j < R; j++) raw[j] = load_word<COHERENT>(rp + u + j * U);
        const unsigned claimed = claim.start(tid);
#pragma unroll
        for (int j = 0; j < R; j++) lrow[padded(u + j * U)] = ar.from_canonical(raw[j]);
        claim.publish(tid, claimed);
        __syncthreads();
        if (claim.lost()) return;                       // uniform: another workgroup has taken this tile; nothing was stored yet
#pragma unroll
        for (int j = 0; j < R; j++) v[j] = lrow[padded(u * R + j)];
        inv_packed<AR, SB, S1>(v, tw, tw_off, u, ar);
        ar.round_end(v);
        __syncthreads();
#pragma unroll
        for (int j = 0; j < R; j++) lrow[padded(u * R + j)] = v[j];
        __syncthreads();
#pragma unroll
        for (int j = 0; j < R; j++) v[j] = lrow[padded(u + j * U)];
        inv_spread<AR, SB, S1, 0>(v, tw, tw_off, ar);
        if constexpr (COMPACT) {
            // inverse transforms keep the hi bytes as bytes [r_local][c_local]: a wave (16 columns x 4 rows of a piece) stores
            // 64 contiguous bytes per instruction and needs no cross-lane packing
            if constexpr (R == 16) mid_store_row_inverse<AR, PAIRED>(mid_limb, tile, rl, u, v, ar);
        } else {
#pragma unroll
            for (int j = 0; j < R; j++) put<PAIRED>(rp + u + j * U, ar.to_mid_inv(v[j]));
        }
    }
}

template <class AR, int SA, int SB, bool INVERSE, bool COMPACT = false>
__global__ __launch_bounds__((RowCfg<SA, SB>::THREADS)) void ntt_row_pass(NttArgs a) {
    constexpr long N = 1l << (SA + SB);
    __shared__ typename AR::V lds[RowCfg<SA, SB>::LDS_WORDS];
    int prime;
    const unsigned l = a.reverse ? gridDim.y - 1 - blockIdx.y : blockIdx.y;
    u64* limb = limb_ptr(a, l, N, prime);
    const AR ar(a.primes[prime]);
    row_tile<AR, SA, SB, INVERSE, false, COMPACT>(limb, blockIdx.x, (const typename AR::TW*)a.tw + (long)prime * N, ar, lds, threadIdx.x,
                                                  COMPACT ? a.mid + l * MID_LIMB_BYTES : nullptr);
}

// The row pass of a forward transform that adds its result to a second operand in the NTT domain: limb (polynomial y, modulus j)
// of the launch receives addend[(y * addend_poly_stride + j) * N ...] (the closing additions of a multiplication,
// KeySwitch_23.cuh:233-234, without a launch, a read and a write of their own).
template <class AR, int SA, int SB, bool COMPACT>
__global__ __launch_bounds__((RowCfg<SA, SB>::THREADS)) void ntt_row_pass_add(NttArgs a, const u64* addend, long addend_poly_stride) {
    constexpr long N = 1l << (SA + SB);
    __shared__ typename AR::V lds[RowCfg<SA, SB>::LDS_WORDS];
    int prime;
    const unsigned l = blockIdx.y;
    u64* limb = limb_ptr(a, l, N, prime);
    const AR ar(a.primes[prime]);
    const u64* add = addend + ((long)limb_poly(a, l) * addend_poly_stride + (prime - a.start_mod_idx)) * N;
    row_tile<AR, SA, SB, false, false, COMPACT>(limb, blockIdx.x, (const typename AR::TW*)a.tw + (long)prime * N, ar, lds, threadIdx.x,
                                                COMPACT ? a.mid + l * MID_LIMB_BYTES : nullptr, TileClaim(), add, a.primes[prime].q);
}

// order of work of the chained transform (mode 2, ntt_extra_forms.hpp); pure arithmetic, also exported for its host-side test
// slot s of a chain -> pass (0 / 1), index k of the limb within the chain, tile.  k >= kmax: an empty slot.
__host__ __device__ inline void chain_slot(unsigned s, unsigned tiles, unsigned skew, unsigned& second, unsigned& k, unsigned& tile) {
    const unsigned e = s / tiles;
    tile = s % tiles;
    if (e < skew) { second = 0; k = e; }
    else { const unsigned r = e - skew; second = r & 1u; k = second ? r / 2 : skew + r / 2; }
}
__host__ __device__ inline unsigned chain_slots(unsigned kmax, unsigned tiles, unsigned skew) { return (skew + 2 * kmax) * tiles; }

#ifdef CKKS_NTT_EXTRA_FORMS
#include "ntt_extra_forms.hpp"
#else
int ntt_chain_deferred(ckks_ctx*, long* tiles) { *tiles = 0; return CKKS_OK; }
#endif
// host view of the slot order, for tests
void ntt_chain_slot(unsigned s, unsigned tiles, unsigned skew, unsigned* second, unsigned* k, unsigned* tile) { chain_slot(s, tiles, skew, *second, *k, *tile); }
unsigned ntt_chain_slots(unsigned kmax, unsigned tiles, unsigned skew) { return chain_slots(kmax, tiles, skew); }

// ------------------------------------------------------------------------------------------------------------
// Paired transform for small batches: both passes in one launch, one workgroup per (limb, tile) that runs the tile of the
// first pass, waits until the limb's other first-pass tiles are done, and runs the same-numbered tile of the second pass.
// A launch of a few hundred workgroups is over before the chip has ramped up, so for one ciphertext the second launch's
// ramp and the drain between the launches cost as much as the work; here they fall away.
//
// Synchronisation (pair_protocol.hpp has the protocol and its reasoning): what the first pass hands to the second moves as
// relaxed atomic accesses at agent scope - on this hardware ordinary stores that are written through to, and loads that are
// served from, the level of the memory system that all compute units share.  Every wave waits until its stores have been
// acknowledged (s_waitcnt 0 behind a workgroup-scope release fence), the workgroup meets at a barrier, and one lane then counts
// the tile done with a relaxed atomic at agent scope.  A reader has seen the full count, by an access of the same kind, before
// it issues its loads.  This rests on the hardware's behaviour for these access kinds, which is what the programming model's
// agent-scope release/acquire pair would also compile to for them; no cache maintenance is asked for beyond it.
// Progress does not depend on which workgroups are resident or in what order they start: a workgroup whose wait outlasts a few
// tens of polls takes over first-pass tiles whose workgroups have not started, every wait is bounded, and what a workgroup
// leaves undone the last workgroup of the limb to leave completes; the launch returns its words to zero.
// Blocks are numbered so that the tiles of a limb go to one XCD (workgroup b of a grid goes to XCD b mod 8): the inter-pass
// data then stays in that XCD's L2.  Placement only matters for speed.
// ------------------------------------------------------------------------------------------------------------
constexpr unsigned PAIR_XCDS = 8;
constexpr int PAIR_MAX_LIMBS = 4096;               // protocol words per context
constexpr int PAIR_GROUPED_LIMBS = 40;             // ... and up to this many with a limb's tiles on one XCD, above it spread over all
constexpr int PAIR_WORD_STRIDE = pair::WORDS;      // protocol words per limb (pair_protocol.hpp)
constexpr int PAIR_AUTO_LIMBS = 128;               // automatic mode: batches up to this many limbs take the paired kernel (while the grid fits the chip)
struct PairArgs {
    unsigned* done;            // [limb * PAIR_WORD_STRIDE] the limb's protocol words (pair_protocol.hpp), zero between launches
    unsigned* fail;            // host-visible word: nonzero once a wait of the key switch's last launch has run out
    unsigned limbs;
    unsigned spin_steal;       // polls after which a waiting workgroup takes over tiles whose workgroups have not started
    unsigned spin_max;         // polls after which it leaves its second-pass tiles to the last workgroup out
    unsigned steal;            // 0: no workgroup takes over another's tile (a test setting)
    unsigned spread;           // the tiles of a limb go to consecutive workgroups, i.e. to all XCDs (larger batches, and a test setting)
};
// (limb, tile) of workgroup b of a paired launch
__device__ __forceinline__ void pair_block(const PairArgs& p, unsigned b, unsigned tiles, unsigned& limb_id, unsigned& tile) {
    const unsigned idx = b / PAIR_XCDS;
    limb_id = p.spread ? b / tiles : b % PAIR_XCDS + PAIR_XCDS * (idx / tiles);
    tile = p.spread ? b % tiles : idx % tiles;
}
// The two passes of (limb_id, tile) under the protocol.  pass1(t) and pass2(t) run tile t on the whole workgroup (t is the
// workgroup's own tile unless it has taken over others; uniform over the workgroup).  stealing = false: a workgroup only ever
// runs its own tile (the first pass is work that only this workgroup can do, already under way when this is called).
template <class P1, class P2>
__device__ __forceinline__ void pair_run(const PairArgs& p, unsigned limb_id, unsigned tile, unsigned* sh, bool stealing, P1 pass1, P2 pass2) {
    static_assert(pair::TILES == 16, "sixteen tiles per limb");
    unsigned* w = p.done + (size_t)limb_id * PAIR_WORD_STRIDE;
    // The claim of the own tile travels while the tile's loads do (see TileClaim); a tile taken over later is claimed before it starts.
    TileClaim own;
    own.lds = stealing ? sh : nullptr;
    own.words = w;
    own.tile = tile;
    unsigned mine = 0, act = tile;
    for (bool first = true;; first = false) {
        pass1(act, first ? own : TileClaim());
        if (first && own.lost()) { act = pair::LEAVE; break; }                  // uniform: behind the tile's first barrier every lane reads the same word
        mine |= 1u << act;
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        __builtin_amdgcn_s_waitcnt(0);                                          // every shared store of this wave has been acknowledged
        __syncthreads();
        if (threadIdx.x == 0) *sh = pair::tile_done_then_decide(w, stealing, p.spin_steal, p.spin_max);
        // The deciding lane's LDS write is complete before its wave reaches the barrier: said explicitly, because a barrier in a
        // loop has been seen compiled with no wait for a write that reaches it over the loop's back edge.
        __builtin_amdgcn_s_waitcnt(0);
        __syncthreads();
        act = *sh;
        __syncthreads();
        if (act >= pair::TILES) break;
    }
    // Counting out does not wait for the own second pass: nothing that the last workgroup out does (the second pass of tiles that
    // others have left, the reset of the words) depends on it.  It rides inside the first second-pass tile (see TileClaim); a
    // workgroup with no second pass to run counts out here.
    unsigned todo = act == pair::GO ? mine : 0u;
    TileClaim out;
    out.lds = sh;
    out.words = w;
    out.counting_out = true;
    if (todo == 0u && threadIdx.x == 0) {
        if (act == pair::DEFER) pair::defer(w, mine);
        *sh = pair::Atomics::fetch_add(w + pair::LEFT, 1u);
    }
    for (bool first = true; todo; first = false) {
        const unsigned t = (unsigned)__builtin_ctz(todo);
        todo &= todo - 1u;
        __syncthreads();                                                        // the tile before is done with the LDS
        pass2(t, first ? out : TileClaim());
    }
    __builtin_amdgcn_s_waitcnt(0xc07f);                                         // lgkmcnt(0) only: the LDS write above, not the tile's last stores
    __syncthreads();
    if (*sh + 1u != pair::TILES) return;                                        // how many had counted out before this workgroup
    // last out: every first-pass tile of the limb is complete; what the others left undone, then the words back to zero
    __syncthreads();
    if (threadIdx.x == 0) *sh = pair::Atomics::load(w + pair::TODO) & pair::ALL;
    __builtin_amdgcn_s_waitcnt(0xc07f);
    __syncthreads();
    const unsigned finished = *sh;
    todo = finished;
    while (todo) {
        const unsigned t = (unsigned)__builtin_ctz(todo);
        todo &= todo - 1u;
        __syncthreads();
        pass2(t, TileClaim());
    }
    if (threadIdx.x == 0) pair::reset(w, finished);
}
template <class AR, int SA, int SB, bool INVERSE, bool COMPACT>
__global__ __launch_bounds__(256, 4) void ntt_pair_kernel(NttArgs a, PairArgs p) {
    typedef StridedCfg<SA, SB> CS;
    typedef RowCfg<SA, SB> CR;
    static_assert(CS::THREADS == 256 && CR::THREADS == 256 && CS::TILES == CR::TILES && CS::TILES == 16, "paired kernel: tile shapes");
    constexpr unsigned TILES = CS::TILES;
    constexpr long N = 1l << (SA + SB);
    constexpr int LDS_WORDS = CS::LDS_WORDS > CR::LDS_WORDS ? CS::LDS_WORDS : CR::LDS_WORDS;
    typedef typename AR::TW TW;
    __shared__ typename AR::V lds[LDS_WORDS];
    __shared__ unsigned go;
    unsigned limb_id, tile;
    pair_block(p, blockIdx.x, TILES, limb_id, tile);
    if (limb_id >= p.limbs) return;                                             // uniform over the workgroup
    int prime;
    u64* limb = limb_ptr(a, limb_id, N, prime);
    const AR ar(a.primes[prime]);
    const TW* __restrict__ tw = (const TW*)a.tw + (long)prime * N;
    char* mid_limb = COMPACT ? a.mid + (long)limb_id * MID_LIMB_BYTES : nullptr;
    u64* out_limb = COMPACT ? limb + a.out_delta : limb;
    pair_run(p, limb_id, tile, &go, p.steal != 0,
             [&](unsigned t, const TileClaim& claim) {
                 if (!INVERSE) strided_tile<AR, SA, SB, false, false, COMPACT, false, true>(limb, t, tw, ar, lds, threadIdx.x, mid_limb, nullptr, 0, false, claim);
                 else row_tile<AR, SA, SB, true, false, COMPACT, true>(limb, t, tw, ar, lds, threadIdx.x, mid_limb, claim);
             },
             [&](unsigned t, const TileClaim& out) {
                 if (!INVERSE) row_tile<AR, SA, SB, false, false, COMPACT, true>(out_limb, t, tw, ar, lds, threadIdx.x, mid_limb, out);
                 else strided_tile<AR, SA, SB, true, false, COMPACT, false, true>(out_limb, t, tw, ar, lds, threadIdx.x, mid_limb, nullptr, 0, false, out);
             });
}

static int ensure_mid(ckks_ctx* c, size_t need);

static void pair_resident_blocks(ckks_ctx* c);      // defined behind the kernels it asks about

// Protocol words and failure word of the paired transform, once per context (at its creation, so that no transform allocates).
int ntt_pair_init(ckks_ctx* c) {
    if (c->d_ntt_pair) return CKKS_OK;
    if (hipHostMalloc((void**)&c->h_pair_fail, sizeof(unsigned), hipHostMallocMapped) != hipSuccess) { set_error("NTT: cannot allocate the failure word of the paired transform"); return CKKS_E_NOMEM; }
    *c->h_pair_fail = 0;
    const size_t bytes = ((size_t)PAIR_MAX_LIMBS + 64) * PAIR_WORD_STRIDE * sizeof(unsigned);      // the last 64: counters of ks_back_kernel
    if (hipMalloc(&c->d_ntt_pair, bytes) != hipSuccess) { set_error("NTT: cannot allocate the completion words of the paired transform"); return CKKS_E_NOMEM; }
    CKKS_HIP_TRY(hipMemset(c->d_ntt_pair, 0, bytes));          // complete before the caller can launch anything on any stream
    pair_resident_blocks(c);
    return CKKS_OK;
}
int ntt_pair_failed(const ckks_ctx* c) { return c->h_pair_fail && *(volatile unsigned*)c->h_pair_fail ? 1 : 0; }
int ntt_pair_deferred(ckks_ctx* c, long* tiles, bool stolen) {
    *tiles = 0;
    if (!c->d_ntt_pair) return CKKS_OK;
    CKKS_HIP_TRY(hipStreamSynchronize(c->stream));
    std::vector<unsigned> w((size_t)PAIR_MAX_LIMBS * PAIR_WORD_STRIDE);
    CKKS_HIP_TRY(hipMemcpy(w.data(), c->d_ntt_pair, w.size() * sizeof(unsigned), hipMemcpyDeviceToHost));
    for (int i = 0; i < PAIR_MAX_LIMBS; i++) *tiles += w[(size_t)i * PAIR_WORD_STRIDE + (stolen ? pair::STOLEN_TOTAL : pair::DEFERRED_TOTAL)];
    return CKKS_OK;
}
int ntt_extra_forms() {
#ifdef CKKS_NTT_EXTRA_FORMS
    return 1;
#else
    return 0;
#endif
}

static PairArgs pair_args(const ckks_ctx* c, int limbs) {
    PairArgs p;
    p.done = (unsigned*)c->d_ntt_pair; p.fail = c->h_pair_fail; p.limbs = (unsigned)limbs;
    p.spin_max = c->chain_spin >= 0 ? (unsigned)c->chain_spin : 4000000u;
    p.spin_steal = c->chain_spin >= 0 && c->chain_spin < 32 ? (unsigned)c->chain_spin : 32u;
    p.steal = c->pair_no_steal ? 0u : 1u;
    p.spread = c->ntt_mode == 5 || (c->ntt_mode == 0 && limbs > PAIR_GROUPED_LIMBS) ? 1u : 0u;
    return p;
}
static unsigned pair_blocks(int limbs, unsigned tiles) { return ((unsigned)limbs + PAIR_XCDS - 1) / PAIR_XCDS * PAIR_XCDS * tiles; }

template <class AR, int SA, int SB>
static int launch_pair(ckks_ctx* c, NttArgs args, int limbs, bool inverse, bool compact_ok, char* mid = nullptr) {
    constexpr bool CAN_COMPACT = std::is_same<AR, F64Arith>::value && SA == 8 && SB == 8;
    int rc = ntt_pair_init(c);
    if (rc) return rc;
    const bool compact = CAN_COMPACT && compact_ok;
    args.limb_base = 0;
    args.limbs_total = (unsigned)limbs;
    args.mid = nullptr;
    if (compact && mid) {
        args.mid = mid;                                   // the caller's inter-pass area
    } else if (compact) {
        if ((rc = ensure_mid(c, (size_t)limbs * MID_LIMB_BYTES))) return rc;
        args.mid = (char*)c->d_ntt_mid;
    }
    const PairArgs p = pair_args(c, limbs);
    const unsigned blocks = pair_blocks(limbs, StridedCfg<SA, SB>::TILES);
    const dim3 g(blocks), b(256);
    if constexpr (CAN_COMPACT) {
        if (compact) {
            if (!inverse) hipLaunchKernelGGL((ntt_pair_kernel<AR, SA, SB, false, true>), g, b, 0, c->stream, args, p);
            else hipLaunchKernelGGL((ntt_pair_kernel<AR, SA, SB, true, true>), g, b, 0, c->stream, args, p);
            CKKS_HIP_TRY(hipGetLastError());
            return CKKS_OK;
        }
    }
    if (!inverse) hipLaunchKernelGGL((ntt_pair_kernel<AR, SA, SB, false, false>), g, b, 0, c->stream, args, p);
    else hipLaunchKernelGGL((ntt_pair_kernel<AR, SA, SB, true, false>), g, b, 0, c->stream, args, p);
    CKKS_HIP_TRY(hipGetLastError());
    return CKKS_OK;
}

// inter-pass area that a call brings with it (the entry point that allocates nothing) instead of the context's buffer
struct NttFixedArea { char* mid; size_t cap; };

// launches of one chunk of limbs; COMPACT selects the 5-byte inter-pass buffer
template <class AR, int SA, int SB, bool COMPACT>
static void launch_passes(ckks_ctx* c, const NttArgs& args_in, int n, bool inverse) {
    typedef StridedCfg<SA, SB> CS;
    typedef RowCfg<SA, SB> CR;
    // The second launch walks the limbs backwards: what the first launch wrote last is still in the memory-side cache (256 MiB)
    // when the second starts, and what the second writes last is what a following transform of the same data reads first.
    NttArgs args = args_in, args2 = args_in;
    args2.reverse = c->ntt_no_reverse ? 0 : 1;
    dim3 gs(CS::TILES, n), bs(CS::THREADS);
    dim3 gr(CR::TILES, n), br(CR::THREADS);
    if (!inverse) {
        if (args.embed_mlwe) hipLaunchKernelGGL((ntt_strided_pass<AR, SA, SB, false, COMPACT, true>), gs, bs, 0, c->stream, args);
        else hipLaunchKernelGGL((ntt_strided_pass<AR, SA, SB, false, COMPACT>), gs, bs, 0, c->stream, args);
        if (c->ev_mid_armed) (void)hipEventRecord(c->ev_mid, c->stream);
        hipLaunchKernelGGL((ntt_row_pass<AR, SA, SB, false, COMPACT>), gr, br, 0, c->stream, args2);
    } else {
        hipLaunchKernelGGL((ntt_row_pass<AR, SA, SB, true, COMPACT>), gr, br, 0, c->stream, args);
        if (c->ev_mid_armed) (void)hipEventRecord(c->ev_mid, c->stream);
        hipLaunchKernelGGL((ntt_strided_pass<AR, SA, SB, true, COMPACT>), gs, bs, 0, c->stream, args2);
    }
}

template <class AR, int SA, int SB>
static int launch_two_pass(ckks_ctx* c, NttArgs args, int limbs, bool inverse, bool compact_ok, int first = 0, const NttFixedArea* fixed = nullptr) {
    // first: the limbs before it have been taken by another launch form (the resident transform takes whole rounds of a batch)
    constexpr bool CAN_COMPACT = std::is_same<AR, F64Arith>::value && SA == 8 && SB == 8;
    int chunk = (c->ntt_chunk > 0 && !c->ev_mid_armed) ? c->ntt_chunk : limbs - first;
    const bool compact = CAN_COMPACT && compact_ok && (fixed || c->ntt_mode != 1);
    if (compact) {
        // the inter-pass buffer is kept at or below 1 GiB; larger batches go through it in chunks (stream order keeps them apart)
        if (fixed) {
            // inter-pass area given with the call (the entry point that allocates nothing): the batch must fit it whole
            if ((size_t)(limbs - first) * MID_LIMB_BYTES > fixed->cap) { set_error("NTT: batch larger than the fixed inter-pass area"); return CKKS_E_INVALID; }
            chunk = limbs - first;
            args.mid = fixed->mid;
        } else {
            const int max_limbs = (int)((1l << 30) / MID_LIMB_BYTES);
            if (chunk > max_limbs) chunk = max_limbs;
            const int rc_mid = ensure_mid(c, (size_t)chunk * MID_LIMB_BYTES);
            if (rc_mid) return rc_mid;
            args.mid = (char*)c->d_ntt_mid;
        }
    } else {
        args.mid = nullptr;
    }
    args.limbs_total = (unsigned)limbs;
    for (int base = first; base < limbs; base += chunk) {
        const int n = limbs - base < chunk ? limbs - base : chunk;
        args.limb_base = (unsigned)base;
        if constexpr (CAN_COMPACT) {
            if (compact) { launch_passes<AR, SA, SB, true>(c, args, n, inverse); continue; }
        }
        launch_passes<AR, SA, SB, false>(c, args, n, inverse);
    }
    CKKS_HIP_TRY(hipGetLastError());
    return CKKS_OK;
}

// Whether a transform of `limbs` limbs runs as the paired kernel: always in modes 4 and 5 while its protocol words suffice, in
// the automatic mode up to the batch at which two launches are as fast and only while every workgroup of the launch fits the chip
// at once (the protocol completes without that, but workgroups that wait for ones that cannot start yet gain nothing).  Measured
// against two launches: with a limb's tiles on one XCD 9.5 us against 15.7 us at 16 limbs, 15 against 22.5 at 32, level at 48 and
// behind above; with the tiles spread over the XCDs 14.4 us at 16 limbs, 20.5 against 22.5 at 48, 34.8 against 36 at 96,
// 49.5 against 48 at 144.  Hence: one XCD per limb up to 40 limbs, spread from there to 128.
// kind: which kernel would run (PAIR_KIND_*): its own occupancy decides what fits the chip
static bool pair_applies(const ckks_ctx* c, int limbs, int kind) {
    if (limbs > PAIR_MAX_LIMBS) return false;
    if (c->ntt_mode == 4 || c->ntt_mode == 5) return true;
    return c->ntt_mode == 0 && limbs <= PAIR_AUTO_LIMBS && pair_blocks(limbs, 16u) <= c->pair_resident_blocks[kind];
}
template <class AR> constexpr int pair_kind_of() { return std::is_same<AR, F64Arith>::value ? PAIR_KIND_F64 : std::is_same<AR, F64WideArith>::value ? PAIR_KIND_WIDE : PAIR_KIND_INT; }

template <class AR>
static int dispatch_logn(ckks_ctx* c, const NttArgs& args, int limbs, bool inverse, bool compact_ok, bool res36_ok = false,
                         const NttFixedArea* fixed = nullptr) {
    // A call that brings its inter-pass area runs as two launches whatever the context's mode (nothing of the context is
    // changed for it: other threads' calls on the same context see the mode they set).
    const int mode = fixed ? 1 : c->ntt_mode;
    // mode 2: both passes in one launch, the limb held in the XCD's L2 between them (N >= 2^15)
#ifdef CKKS_NTT_EXTRA_FORMS
    if (!c->ev_mid_armed && mode == 2 && !args.embed_mlwe) {
        if (c->logN == 16) return launch_chain<AR, 8, 8>(c, args, limbs, inverse);
        if (c->logN == 15) return launch_chain<AR, 8, 7>(c, args, limbs, inverse);
    }
#endif
    // The resident transform - one persistent workgroup per compute unit carries whole limbs through both passes in its registers
    // (N = 2^16, primes below 2^36) - takes the whole rounds of a batch (one limb per compute unit and round) and a last round that is
    // at least three quarters full; what is left goes out as two launches behind it.  Mode 6 asks for it wherever it applies, the
    // automatic mode takes it too, mode 1 never.
    if (std::is_same<AR, F64Arith>::value && !c->ev_mid_armed && !args.embed_mlwe && (mode == 0 || mode == 6) && res36_ok &&
        ntt_resident_applies(c, limbs)) {
        const int per_round = ntt_resident_round(c);
        int whole = limbs / per_round * per_round;
        if (limbs - whole >= per_round * 3 / 4) whole = limbs;
        int rc = launch_ntt_resident(c, args, limbs, whole, inverse);
        if (rc || whole == limbs) return rc;
        return launch_two_pass<AR, 8, 8>(c, args, limbs, inverse, compact_ok, whole);
    }
    // mode 4, and the automatic mode for small batches: both passes in one launch of one workgroup per (limb, tile)
    if (!c->ev_mid_armed && !fixed && !args.embed_mlwe && c->logN == 16 && pair_applies(c, limbs, pair_kind_of<AR>())) return launch_pair<AR, 8, 8>(c, args, limbs, inverse, compact_ok);
    // mode 3: one workgroup per limb, both passes in one launch.  Measured slower than two launches at the full batch size
    // (the limbs in flight, 0.5 MiB per resident workgroup, exceed the L2 by far), so the automatic mode does not pick it.
#ifdef CKKS_NTT_EXTRA_FORMS
    if (!c->ev_mid_armed && mode == 3) {
        if (c->logN == 16) return launch_whole_limb<AR, 8, 8>(c, args, limbs, inverse);
        if (c->logN == 15) return launch_whole_limb<AR, 8, 7>(c, args, limbs, inverse);
    }
#endif
    switch (c->logN) {
        case 8:  return launch_two_pass<AR, 4, 4>(c, args, limbs, inverse, compact_ok, 0, fixed);
        case 9:  return launch_two_pass<AR, 5, 4>(c, args, limbs, inverse, compact_ok, 0, fixed);
        case 10: return launch_two_pass<AR, 5, 5>(c, args, limbs, inverse, compact_ok, 0, fixed);
        case 11: return launch_two_pass<AR, 6, 5>(c, args, limbs, inverse, compact_ok, 0, fixed);
        case 12: return launch_two_pass<AR, 6, 6>(c, args, limbs, inverse, compact_ok, 0, fixed);
        case 13: return launch_two_pass<AR, 7, 6>(c, args, limbs, inverse, compact_ok, 0, fixed);
        case 14: return launch_two_pass<AR, 7, 7>(c, args, limbs, inverse, compact_ok, 0, fixed);
        case 15: return launch_two_pass<AR, 8, 7>(c, args, limbs, inverse, compact_ok, 0, fixed);
        case 16: return launch_two_pass<AR, 8, 8>(c, args, limbs, inverse, compact_ok, 0, fixed);
        default: set_error("NTT: logN must be in [8, 16]"); return CKKS_E_INVALID;
    }
}


// ------------------------------------------------------------------------------------------------------------
// Middle of the hybrid key switch in one launch: the row pass of the forward transform of every digit, the inner product with
// the key over the digits, and the row pass of the inverse transform of both sums, on one tile of 16 rows of one limb.
// Between the two row passes the data of a tile never leaves the workgroup: the digits' transforms are multiplied in
// registers (in the lane layout in which the row pass stores, so the key is read in full lines), the sums go straight into
// the inverse row pass.  Against the three launches it replaces this saves one write and one read of every digit limb and
// of both sums.  Same integers as the separate launches: every step is exact modulo the prime.
// N = 2^16, FP64 back end, 5-byte inter-pass form on both sides.
// ------------------------------------------------------------------------------------------------------------
struct KsRowArgs {
    const char* mid_in;          // inter-pass buffer of the digits' forward transform, limb index o * ndigits + d
    char* mid_out;               // inter-pass buffer of the sums' inverse transform, limb index o * 2 + z
    const u64* key;              // limb (z * key_z_stride + d * key_digit_stride + o), canonical residues in the NTT domain
    const PrimeConst* primes;
    const double* tw_fwd;
    const double* tw_inv;
    int ndigits;
    long key_digit_stride, key_z_stride;
    // Limb o >= p_num of digit (o - p_num) / p_num is the input itself: the digit's own residues pass through the conversion and
    // the forward transform of a coefficient form gives the NTT-domain input back.  With in_ntt set (limb o - p_num of the input,
    // canonical, NTT domain) that digit's term is taken from there and its transform is never computed.
    const u64* in_ntt;
    int p_num;
};
__global__ __launch_bounds__(256, 2) void ks_row_fused_kernel(KsRowArgs a) {
    typedef RowCfg<8, 8> C;
    constexpr int S1 = C::S1, R = C::R, N2 = C::N2, U = C::U, N1 = C::N1, ROWS = C::ROWS;
    constexpr long N = 1l << 16;
    static_assert(R == 16 && U == 16 && ROWS == 16, "tile shape");
    __shared__ double lds[C::LDS_WORDS];
    const unsigned tile = blockIdx.x, o = blockIdx.y, tid = threadIdx.x;
    const F64Arith ar(a.primes[o]);
    const double* twf = a.tw_fwd + (long)o * N;
    const double* twi = a.tw_inv + (long)o * N;
    const unsigned u = tid % U, rl = tid / U;
    const unsigned row = tile * ROWS + rl;
    double* lrow = lds + rl * C::PITCH;
    const unsigned tw_off = N1 + row;
    double acc[2][R];
#pragma unroll
    for (int j = 0; j < R; j++) acc[0][j] = acc[1][j] = 0.0;
    // raw 5-byte values of the digit in work, requested one digit ahead
    unsigned raw_lo[R], raw_hi[R];
    auto request = [&](int d) { mid_load_row_raw(a.mid_in + ((long)o * a.ndigits + d) * MID_LIMB_BYTES, tile, rl, u, raw_lo, raw_hi); };
    const int own = a.in_ntt && (int)o >= a.p_num ? ((int)o - a.p_num) / a.p_num : -1;
    if (own != 0) request(0);
    else if (a.ndigits > 1) request(1);
    for (int d = 0; d < a.ndigits; d++) {
        const u64* ka = a.key + ((long)d * a.key_digit_stride + o) * N + (long)row * N2 + u;
        const u64* kb = ka + a.key_z_stride * N;
        if (d == own) {
            const u64* xp = a.in_ntt + (long)((int)o - a.p_num) * N + (long)row * N2 + u;
            u64 xi[R], k0[R], k1[R];
#pragma unroll
            for (int j = 0; j < R; j++) { xi[j] = xp[j * U]; k0[j] = ka[j * U]; k1[j] = kb[j * U]; }
#pragma unroll
            for (int j = 0; j < R; j++) {
                const double x = ar.balance((double)(long long)xi[j]);
                acc[0][j] += ar.mulmod(x, (double)(long long)k0[j]);
                acc[1][j] += ar.mulmod(x, (double)(long long)k1[j]);
            }
            continue;
        }
        const int nxt = d + 1 == own ? d + 2 : d + 1;
        double v[R];
        unsigned two = tw_off;                              // opaque per digit: the twiddle loads stay inside the loop (they hit the
        asm volatile("" : "+v"(two));                       // cache) instead of occupying registers across it
#pragma unroll
        for (int j = 0; j < R; j++) v[j] = mid_decode_row(ar, raw_lo[j], raw_hi[j], rl);
        fwd_spread<F64Arith, 8, S1>(v, twf, two, ar);
        // the first writes of a digit go to the words this lane read last in the digit before: no barrier needed in between
#pragma unroll
        for (int j = 0; j < R; j++) lrow[padded(u + j * U)] = v[j];
        __syncthreads();
#pragma unroll
        for (int j = 0; j < R; j++) v[j] = lrow[padded(u * R + j)];
        fwd_packed<F64Arith, 8, S1>(v, twf, two, u, ar);
        __syncthreads();
#pragma unroll
        for (int j = 0; j < R; j++) lrow[padded(u * R + j)] = v[j];
        u64 k0[R], k1[R];                                   // requested once the butterflies' registers are free
#pragma unroll
        for (int j = 0; j < R; j++) { k0[j] = ka[j * U]; k1[j] = kb[j * U]; }
        if (nxt < a.ndigits) request(nxt);
        __syncthreads();
#pragma unroll
        for (int j = 0; j < R; j++) {
            const double x = ar.balance(lrow[padded(u + j * U)]);                 // column u + 16 j of the row, |x| <= q/2
            acc[0][j] += ar.mulmod(x, (double)(long long)k0[j]);                  // each term in (-0.51 q, 0.51 q)
            acc[1][j] += ar.mulmod(x, (double)(long long)k1[j]);
        }
    }
#pragma unroll
    for (int z = 0; z < 2; z++) {
        char* mid_limb = a.mid_out + ((long)o * 2 + z) * MID_LIMB_BYTES;
        double v[R];
#pragma unroll
        for (int j = 0; j < R; j++) lrow[padded(u + j * U)] = ar.balance(acc[z][j]);
        __syncthreads();
#pragma unroll
        for (int j = 0; j < R; j++) v[j] = lrow[padded(u * R + j)];
        inv_packed<F64Arith, 8, S1>(v, twi, tw_off, u, ar);
        __syncthreads();
#pragma unroll
        for (int j = 0; j < R; j++) lrow[padded(u * R + j)] = v[j];
        __syncthreads();
#pragma unroll
        for (int j = 0; j < R; j++) v[j] = lrow[padded(u + j * U)];
        inv_spread<F64Arith, 8, S1, 0>(v, twi, tw_off, ar);
        mid_store_row_inverse(mid_limb, tile, rl, u, v, ar);
    }
}

// ------------------------------------------------------------------------------------------------------------
// Key switch through the T basis (KeySwitch_23.cuh:225-226): the external product with the key (external_product_T,
// ExternalProduct.cuh:56-83: out[z][o] = sum over the digits d of c[d][o mod T] * key[z][d][o], 128-bit sums, one reduction) and
// the row pass of the inverse transform of every sum in one launch.  A workgroup forms one tile of 16 rows of one output limb in
// the lane layout in which the row pass loads (so the key and the digits are read in full lines) and runs the row pass on it; the
// strided pass follows as a launch of its own.  Against the separate launches this saves one write and one read of every sum.
// N = 2^16, integer back end (the T primes of the reference's sets have 60 bits).
// Order of the workgroups: consecutive workgroups go to the eight XCDs in turn; numbered as below, those of one XCD take the
// output blocks and polynomials of one (tile, T prime) one after the other, so the digit tiles they share (and the prime's
// twiddles) are read from that XCD's L2.
// ------------------------------------------------------------------------------------------------------------
struct ExtRowArgs {
    const u64* c;                // digits over T, NTT domain: limb d * t_num + t
    const u64* key;              // limb z * key_z_stride + d * key_digit_stride + o
    u64* out;                    // limb z * out_z_stride + o: as an in-place inverse transform leaves it between its passes
    const PrimeConst* primes;
    const ulonglong2* tw_inv;    // [prime][N]
    int ndigits, t_num, blocks, prime0;
    long key_digit_stride, key_z_stride, out_z_stride;
};
__global__ __launch_bounds__(256, 4) void ext_row_fused_kernel(ExtRowArgs a) {
    typedef RowCfg<8, 8> C;
    constexpr int S1 = C::S1, R = C::R, N2 = C::N2, U = C::U, N1 = C::N1, ROWS = C::ROWS;
    constexpr long N = 1l << 16;
    static_assert(R == 16 && U == 16 && ROWS == 16, "tile shape");
    __shared__ u64 lds[C::LDS_WORDS];
    const unsigned tid = threadIdx.x;
    unsigned w = blockIdx.x;
    const unsigned t = w % (unsigned)a.t_num; w /= (unsigned)a.t_num;
    const unsigned z = w & 1u; w >>= 1;
    const unsigned blk = w % (unsigned)a.blocks, tile = w / (unsigned)a.blocks;
    const unsigned o = blk * (unsigned)a.t_num + t;
    const int prime = a.prime0 + (int)t;
    const PrimeConst& pr = a.primes[prime];
    const IntArith ar(pr);
    const ulonglong2* tw = a.tw_inv + (long)prime * N;
    const unsigned u = tid % U, rl = tid / U;
    const unsigned row = tile * ROWS + rl;
    u64* lrow = lds + rl * C::PITCH;
    const unsigned tw_off = N1 + row;
    const long at = (long)row * N2 + u;
    // The product phase.  Its sums go through LDS before the row pass, so its lanes need not own the words that the pass gives
    // them: lane tid takes words 2 (tid % 128) and the next of rows tid / 128 + 2 r, r = 0 .. 7, with 16-byte loads - a wave reads
    // 1 KiB of a key row in one instruction, where eight-byte loads on the pass's own assignment read four 128-byte pieces.
    // Four words (two loads) at a time: the 128-bit sums of all sixteen would take half of the registers that let four workgroups
    // share a compute unit.  Two digits' words are in flight: (x, k) holds the even digits, (xn, kn) the odd ones, each
    // refilled right after its use.
    {
        const unsigned pu = (tid & 127u) * 2u, pr0 = tid >> 7;
        const long pat = (long)(tile * ROWS + pr0) * N2 + pu;
        const ulonglong2* cp2 = reinterpret_cast<const ulonglong2*>(a.c + (long)t * N + pat);
        const ulonglong2* kp2 = reinterpret_cast<const ulonglong2*>(a.key + ((long)z * a.key_z_stride + o) * N + pat);
        const long c_step = (long)a.t_num * (N / 2), k_step = a.key_digit_stride * (N / 2);       // in 16-byte words
        constexpr int H = 2;                                    // loads per chunk; a load's two rows apart = N2 16-byte words
#pragma unroll 1
        for (int j0 = 0; j0 < ROWS / 2; j0 += H) {
            u128w acc[2 * H];
            ulonglong2 x[H], k[H], xn[H], kn[H];
#pragma unroll
            for (int j = 0; j < H; j++) {
                acc[2 * j] = u128w{0, 0};
                acc[2 * j + 1] = u128w{0, 0};
                x[j] = cp2[(j0 + j) * N2];
                k[j] = kp2[(j0 + j) * N2];
            }
            if (a.ndigits > 1) {
#pragma unroll
                for (int j = 0; j < H; j++) { xn[j] = cp2[c_step + (j0 + j) * N2]; kn[j] = kp2[k_step + (j0 + j) * N2]; }
            }
            for (int d = 0; d < a.ndigits; d += 2) {
#pragma unroll
                for (int j = 0; j < H; j++) { mac128(acc[2 * j], x[j].x, k[j].x); mac128(acc[2 * j + 1], x[j].y, k[j].y); }
                if (d + 2 < a.ndigits) {
#pragma unroll
                    for (int j = 0; j < H; j++) { x[j] = cp2[(d + 2) * c_step + (j0 + j) * N2]; k[j] = kp2[(d + 2) * k_step + (j0 + j) * N2]; }
                }
                if (d + 1 < a.ndigits) {
#pragma unroll
                    for (int j = 0; j < H; j++) { mac128(acc[2 * j], xn[j].x, kn[j].x); mac128(acc[2 * j + 1], xn[j].y, kn[j].y); }
                    if (d + 3 < a.ndigits) {
#pragma unroll
                        for (int j = 0; j < H; j++) { xn[j] = cp2[(d + 3) * c_step + (j0 + j) * N2]; kn[j] = kp2[(d + 3) * k_step + (j0 + j) * N2]; }
                    }
                }
            }
#pragma unroll
            for (int j = 0; j < H; j++) {
                u64* srow = lds + (pr0 + 2 * (j0 + j)) * C::PITCH;
                srow[padded(pu)] = barrett128(acc[2 * j], pr.q, pr.mu_hi, pr.mu_lo);
                srow[padded(pu + 1)] = barrett128(acc[2 * j + 1], pr.q, pr.mu_hi, pr.mu_lo);
            }
        }
    }
    // the row pass of the inverse transform (row_tile, inverse branch) on the sums
    __syncthreads();
    u64 v[R];
#pragma unroll
    for (int j = 0; j < R; j++) v[j] = lrow[padded(u * R + j)];
    inv_packed<IntArith, 8, S1>(v, tw, tw_off, u, ar);
    __syncthreads();
#pragma unroll
    for (int j = 0; j < R; j++) lrow[padded(u * R + j)] = v[j];
    __syncthreads();
#pragma unroll
    for (int j = 0; j < R; j++) v[j] = lrow[padded(u + j * U)];
    inv_spread<IntArith, 8, S1, 0>(v, tw, tw_off, ar);
    u64* rp = a.out + ((long)z * a.out_z_stride + o) * N + at;
#pragma unroll
    for (int j = 0; j < R; j++) rp[j * U] = ar.to_mid_inv(v[j]);
}

// ------------------------------------------------------------------------------------------------------------
// End of a key switch: ModDown and the first pass of the forward transform of its result in one launch.  The strided pass
// of limb q_i of polynomial z takes each of its inputs from the K special-prime limbs and limb q_i of the extended
// polynomial (BasisConv.cuh:257-326: out = (c_q - sum_i [c_p_i * pHat_i^-1]_p_i * pHat_i) * P^-1 mod q) instead of reading
// a stored result, so the ModDown output is never written in the coefficient domain.  The special-prime limbs are read once
// per output prime (from the L2 after the first); the arithmetic is that of the stand-alone FP64 ModDown kernel.
// ------------------------------------------------------------------------------------------------------------
struct KsModDownArgs {
    const u64* in;               // two extended polynomials, coefficient domain: limb i < K modulo p_i, limb K + i modulo q_i
    long in_z_stride;            // words between the two polynomials
    char* mid;                   // where the first pass of the results' forward transform goes, in the form MID: limb (i, z) lies
    long mid_stride_i, mid_stride_z;   //   at mid + i * mid_stride_i + z * mid_stride_z bytes
    const PrimeConst* primes;
    const double* tw_fwd;
    const u64* pHatVecModq;      // [q index][K]
    const u64* pHatInv;          // [K]
    const u64* PinvModq;         // [q index]
    int K;
    int pre_scaled;              // the special-prime limbs already hold [c_p_i * pHat_i^-1]_p_i (canonical)
};
template <class AR>
__device__ __forceinline__ double canon_f(const AR& ar, double r) { return canon_f64(r, ar.q, ar.qinv); }               // any |r| < 2^52 -> [0, q)
// With the wide arithmetic every constant enters balanced and at most 8 special primes are admitted: a term of the sum lies within
// 0.88 q of zero (its operand, a residue modulo p_i, may be up to twice q), so eight of them stay below 2^53.
template <class AR, class MID>
__global__ __launch_bounds__(256) void ks_moddown_strided_kernel(KsModDownArgs a) {
    typedef StridedCfg<8, 8> C;
    constexpr int S1 = C::S1, R = C::R, N2 = C::N2, G = C::G, CW = C::CW;
    constexpr long N = 1l << 16;
    __shared__ double lds[C::LDS_WORDS];
    // tiles are the slow grid dimension: the workgroups in flight share a few tiles' worth of special-prime columns, which the L2 holds
    const unsigned tile = blockIdx.y, limb = blockIdx.x, iq = limb >> 1, z = limb & 1, tid = threadIdx.x;
    const unsigned cl = tid % CW, g = tid / CW;
    const int prime = a.K + (int)iq;
    const AR ar(a.primes[prime]);
    const u64* col = a.in + (long)z * a.in_z_stride + tile * CW + cl;
    double acc[R];
#pragma unroll
    for (int j = 0; j < R; j++) acc[j] = 0.0;
    // the limbs are read one ahead of their use: limb i + 1 (or, after the last special prime, limb q) travels while limb i is worked on
    u64 x[R], xn[R];
#pragma unroll
    for (int j = 0; j < R; j++) x[j] = col[(long)(g + j * G) * N2];
    for (int i = 0; i < a.K; i++) {
        const AR ap(a.primes[i]);
        const double hinv = ap.from_canonical(a.pHatInv[i]), hat = ar.from_canonical(a.pHatVecModq[(long)iq * a.K + i]);
        const u64* nl = col + (long)(i + 1 < a.K ? i + 1 : prime) * N;
#pragma unroll
        for (int j = 0; j < R; j++) xn[j] = nl[(long)(g + j * G) * N2];
#pragma unroll
        for (int j = 0; j < R; j++) {
            // the canonical representative of each scaled special-prime residue enters the sum, as in the stand-alone kernel
            if (a.K == 1) acc[j] = exact_u2d(x[j]);                                                  // BasisConv.cuh:274
            else if (a.pre_scaled) acc[j] += ar.mulmod(exact_u2d(x[j]), hat);
            else acc[j] += ar.mulmod(canon_f(ap, ap.mulmod(exact_u2d(x[j]), hinv)), hat);
        }
#pragma unroll
        for (int j = 0; j < R; j++) x[j] = xn[j];
    }
    const double pinv = ar.from_canonical(a.PinvModq[iq]);
    double v[R];
#pragma unroll
    for (int j = 0; j < R; j++) v[j] = ar.mulmod(ar.q - canon_f(ar, acc[j]) + exact_u2d(x[j]), pinv);      // in (-0.51 q, 0.51 q)
    const double* tw = a.tw_fwd + (long)prime * N;
    ar.round_end(v);
    fwd_spread<AR, 8, S1>(v, tw, 1u, ar);
    ar.round_end(v);
#pragma unroll
    for (int j = 0; j < R; j++) lds[(g + j * G) * CW + cl] = v[j];
    __syncthreads();
#pragma unroll
    for (int j = 0; j < R; j++) v[j] = lds[(g * R + j) * CW + cl];
    fwd_packed<AR, 8, S1>(v, tw, 1u, g, ar);
    MID::store_columns(a.mid + iq * a.mid_stride_i + z * a.mid_stride_z, tile, g, cl, v, ar);
}

// ------------------------------------------------------------------------------------------------------------
// End of the hybrid key switch in one launch less: the strided (last) pass of the sums' inverse transform and the ModDown
// pass above share their column tiling, so a ModDown workgroup (q limb, polynomial z, 16 columns) needs from that inverse
// pass exactly the same 16 columns of its own limb and of the K special-prime limbs.  Here it runs the inverse pass of its own
// limb itself and keeps the coefficients in registers (they come out in the lane layout the ModDown reads them in), and the
// special-prime limbs' passes are 2 K 16 workgroups at the front of the grid that write their (scaled) coefficients as shared
// stores and count themselves done per (z, tile).  The coefficients of the q limbs are never written: a write and a read of
// 2 (l + 1) limbs and one launch less.  A waiting workgroup waits only for workgroups of lower index that wait for nothing.
// Each (z, tile) has two counters: the special-prime workgroups that are done (waited for until it reads K) and the ModDown
// workgroups that have seen that; the last of those returns both to zero, so a launch leaves the counters as it found them
// and needs nothing from the host (it can be replayed from a captured graph).
// The row pass of the results follows in the same workgroup after the hand-over of the paired transform (the sixteen tiles of
// a limb are consecutive workgroups).
// ------------------------------------------------------------------------------------------------------------
struct KsBackArgs {
    const char* mid_in;          // sums after the row pass of their inverse transform: limb o * 2 + z, 5-byte form
    u64* sums;                   // [2][z_stride]: only the K special-prime limbs of each polynomial are written
    long z_stride;               // words between the two polynomials
    char* mid_out;               // between the passes of the results' forward transform: limb iq * 2 + z, 5-byte form
    u64* out;                    // results: limb iq of polynomial z at out + (z * out_z_stride + iq * N) words, NTT domain
    long out_z_stride;
    PairArgs pair;               // completion words of the hand-over between those two passes, limb index iq * 2 + z
    const PrimeConst* primes;    // constants whose special-prime entries carry (P/p_i)^-1 in N^-1 and the last twiddle
    const double* tw_inv;
    const double* tw_fwd;
    const u64* pHatVecModq;      // [q index][K]
    const u64* PinvModq;         // [q index]
    unsigned* count;             // [2 * 16] pairs (done, seen), one pair per 128-byte line; zero between launches
    int K, nq;
};
__global__ __launch_bounds__(256, 4) void ks_back_kernel(KsBackArgs a) {
    typedef StridedCfg<8, 8> C;
    constexpr int S1 = C::S1, R = C::R, N2 = C::N2, G = C::G, CW = C::CW;
    constexpr long N = 1l << 16;
    constexpr int LDS_WORDS = C::LDS_WORDS > RowCfg<8, 8>::LDS_WORDS ? C::LDS_WORDS : RowCfg<8, 8>::LDS_WORDS;
    __shared__ double lds[LDS_WORDS];
    __shared__ unsigned go;
    const unsigned tid = threadIdx.x, cl = tid % CW, g = tid / CW;
    const unsigned producers = (unsigned)a.K * 32u;
    const bool special = blockIdx.x < producers;
    const unsigned b = special ? blockIdx.x : blockIdx.x - producers;
    const unsigned li = b / 32u, z = (b / 16u) & 1u, tile = b % 16u;       // li: special prime i, or q index iq
    const int prime = special ? (int)li : a.K + (int)li;
    const F64Arith ar(a.primes[prime]);
    // last pass of the inverse transform of limb `prime` of polynomial z, columns of `tile`
    double v[R];
    {
        const char* piece = mid_piece(const_cast<char*>(a.mid_in) + ((long)prime * 2 + z) * MID_LIMB_BYTES, tile, g);
#pragma unroll
        for (int j = 0; j < R; j++)
            v[j] = ar.dec40(*reinterpret_cast<const unsigned*>(piece + (j * 16 + cl) * 4), *reinterpret_cast<const unsigned char*>(piece + 1024 + j * 16 + cl));
    }
    const double* twi = a.tw_inv + (long)prime * N;
    inv_packed<F64Arith, 8, S1>(v, twi, 1u, g, ar);
#pragma unroll
    for (int j = 0; j < R; j++) lds[(g * R + j) * CW + cl] = v[j];
    __syncthreads();
#pragma unroll
    for (int j = 0; j < R; j++) v[j] = lds[(g + j * G) * CW + cl];
    inv_spread<F64Arith, 8, S1, 1>(v, twi, 1u, ar);
    u64 own[R];                                                       // coefficient of row g + j G, canonical
#pragma unroll
    for (int j = 0; j < R / 2; j++) ar.gs_last(v[j], v[j + R / 2], own[j], own[j + R / 2]);
    unsigned* word = a.count + (size_t)(z * 16u + tile) * PAIR_WORD_STRIDE;
    if (special) {
        u64* col = a.sums + (long)z * a.z_stride + (long)li * N + tile * CW + cl;
#pragma unroll
        for (int j = 0; j < R; j++) put<true>(col + (long)(g + j * G) * N2, own[j]);
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        __builtin_amdgcn_s_waitcnt(0);                                // this wave's shared stores have been acknowledged
        __syncthreads();
        if (tid == 0) (void)__hip_atomic_fetch_add(word, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        return;
    }
    if (tid == 0) {
        unsigned ok = 0;
        for (unsigned n = 0; n < a.pair.spin_max; n++) {
            if (__hip_atomic_load(word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) >= (unsigned)a.K) { ok = 1; break; }
            __builtin_amdgcn_s_sleep(4);
        }
        if (!ok) __hip_atomic_store(a.pair.fail, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
        else if (__hip_atomic_fetch_add(word + 1, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + 1u == (unsigned)a.nq) {
            // every ModDown workgroup of this (z, tile) has seen the count: back to zero for the next launch
            __hip_atomic_store(word, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(word + 1, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        go = ok;
    }
    __syncthreads();                                                  // also: every lane is done with the LDS tile of the inverse pass
    if (!go) return;
    // ModDown (BasisConv.cuh:257-326) on the scaled special-prime coefficients, as in ks_moddown_strided_kernel with pre_scaled
    const u64* col = a.sums + (long)z * a.z_stride + tile * CW + cl;
    // The sum starts from minus the limb's own coefficient (the ModDown is (own - sum) P^-1 mod q): the sixteen coefficients need
    // no registers of their own from here on, which is what lets four of these workgroups share a compute unit.
    double acc[R];
#pragma unroll
    for (int j = 0; j < R; j++) acc[j] = -exact_u2d(own[j]);
    // half a limb ahead: the loads of one half of the rows are in flight while the other half is multiplied
    u64 xa[R / 2], xb[R / 2];
#pragma unroll
    for (int j = 0; j < R / 2; j++) xa[j] = get<true>(col + (long)(g + j * G) * N2);
    for (int i = 0; i < a.K; i++) {
        const double hat = exact_u2d(a.pHatVecModq[(long)li * a.K + i]);
        const u64* cur = col + (long)i * N;
#pragma unroll
        for (int j = 0; j < R / 2; j++) xb[j] = get<true>(cur + (long)(g + (j + R / 2) * G) * N2);
#pragma unroll
        for (int j = 0; j < R / 2; j++) {
            if (a.K == 1) acc[j] += exact_u2d(xa[j]);                                                // BasisConv.cuh:274
            else acc[j] += ar.mulmod(exact_u2d(xa[j]), hat);
        }
        if (i + 1 < a.K) {
#pragma unroll
            for (int j = 0; j < R / 2; j++) xa[j] = get<true>(cur + N + (long)(g + j * G) * N2);
        }
#pragma unroll
        for (int j = 0; j < R / 2; j++) {
            if (a.K == 1) acc[j + R / 2] += exact_u2d(xb[j]);
            else acc[j + R / 2] += ar.mulmod(exact_u2d(xb[j]), hat);
        }
    }
    const double pinv = exact_u2d(a.PinvModq[li]);
#pragma unroll
    for (int j = 0; j < R; j++) v[j] = ar.mulmod(ar.q - canon_f(ar, acc[j]), pinv);      // (own - sum) P^-1, in (-0.51 q, 0.51 q)
    const double* twf = a.tw_fwd + (long)prime * N;
    fwd_spread<F64Arith, 8, S1>(v, twf, 1u, ar);
#pragma unroll
    for (int j = 0; j < R; j++) lds[(g + j * G) * CW + cl] = v[j];
    __syncthreads();
#pragma unroll
    for (int j = 0; j < R; j++) v[j] = lds[(g * R + j) * CW + cl];
    fwd_packed<F64Arith, 8, S1>(v, twf, 1u, g, ar);
    char* mid_limb = a.mid_out + ((long)li * 2 + z) * MID_LIMB_BYTES;
    mid_store_columns<F64Arith, true>(mid_limb, tile, g, cl, v, ar);
    // second pass of the result's forward transform, once the limb's sixteen first-pass tiles are there (each of them is the
    // work above of one workgroup: nothing to take over)
    pair_run(a.pair, li * 2u + z, tile, &go, false, [](unsigned, const TileClaim&) {},
             [&](unsigned t, const TileClaim& out) { row_tile<F64Arith, 8, 8, false, false, true, true>(a.out + (long)z * a.out_z_stride + (long)li * N, t, twf, ar, lds, tid, mid_limb, out); });
}

// The stage-fusing launches below keep data in the 5-byte inter-pass form and compute in FP64: N = 2^16, automatic back end and
// transform modes, every prime involved below 2^39.  The context option "ks_split" switches them off, for tuning and tests.
// How the stage-fused launches can run on primes first_prime .. first_prime + prime_count - 1: 0 not at all, 1 with the 5-byte
// inter-pass pieces (all primes below 2^39), 2 with whole limbs between the passes and the wide FP64 arithmetic (all below 2^50).
static int stage_fusion_form(const ckks_ctx* c, int first_prime, int prime_count) {
    if (c->ks_split || c->logN != 16 || c->arith_mode != 0 || c->ntt_mode != 0 || c->ev_mid_armed) return 0;
    if (first_prime < 0 || prime_count < 1 || first_prime + prime_count > c->nprimes) return 0;
    int form = 1;
    for (int j = first_prime; j < first_prime + prime_count; j++) {
        if (c->pqt[j] >= (1ull << 50)) return 0;
        if (c->pqt[j] >= (1ull << 39)) form = 2;
    }
    return form;
}
static bool stage_fusion_applies(const ckks_ctx* c, int first_prime, int prime_count) { return stage_fusion_form(c, first_prime, prime_count) == 1; }

static int ensure_mid(ckks_ctx* c, size_t need) {
    if (need <= c->ntt_mid_cap) return CKKS_OK;
    if (c->d_ntt_mid) { (void)hipDeviceSynchronize(); (void)hipFree(c->d_ntt_mid); c->d_ntt_mid = nullptr; c->ntt_mid_cap = 0; }
    if (hipMalloc(&c->d_ntt_mid, need) != hipSuccess) { set_error("NTT: cannot allocate the inter-pass buffer"); return CKKS_E_NOMEM; }
    c->ntt_mid_cap = need;
    return CKKS_OK;
}

// ------------------------------------------------------------------------------------------------------------
// Start of the hybrid key switch: the exact conversion of every digit (BasisConv.cuh:18-58) inside the first pass of the
// forward transform of the digit's limbs.  y: the digit residues already scaled by (D/d_j)^-1 (left by the inverse transform
// that ran with the scaled constants), v: the quotient estimates.  Workgroup (tile, o * ndigits + d) produces the 16 columns
// of limb o of digit d: sum_j y_j * ((D/d_j) mod r_o) - v * (D mod r_o), then the strided pass on them.  For a prime of the
// digit itself the constants give the residue back.  The extended digits are never written in the coefficient domain.
// ------------------------------------------------------------------------------------------------------------
struct KsModUpArgs {
    const u64* y;                // l + 1 limbs
    signed char* v;              // [digit][N]
    char* mid;                   // inter-pass buffer of the digits' forward transform, limb index o * ndigits + d
    const ConvBlock* blocks;     // one per digit, target k = prime k
    const PrimeConst* primes;
    const double* tw_fwd;
    int ndigits, p_num;
};
__global__ __launch_bounds__(256) void ks_modup_quotient_kernel(KsModUpArgs a) {
    constexpr long N = 1l << 16;
    const ConvBlock& __restrict__ b = a.blocks[blockIdx.y];
    const long x = (long)blockIdx.x * 256 + threadIdx.x;
    double vv = 0.0;
    for (int j = 0; j < b.nsrc; j++) vv += exact_u2d(a.y[(long)b.src_limb[j] * N + x]) / a.primes[b.src_prime[j]].qd;   // in index order
    a.v[(long)blockIdx.y * N + x] = (signed char)(int)vv;
}
__global__ __launch_bounds__(256) void ks_modup_strided_kernel(KsModUpArgs a) {
    typedef StridedCfg<8, 8> C;
    constexpr int S1 = C::S1, R = C::R, N2 = C::N2, G = C::G, CW = C::CW;
    constexpr long N = 1l << 16;
    __shared__ double lds[C::LDS_WORDS];
    // tiles are the slow grid dimension: the workgroups in flight share a few tiles' worth of columns of y, which the L2 holds
    const unsigned tile = blockIdx.y, limb = blockIdx.x, o = limb / a.ndigits, d = limb % a.ndigits, tid = threadIdx.x;
    const unsigned cl = tid % CW, g = tid / CW;
    if ((int)o >= a.p_num && ((int)o - a.p_num) / a.p_num == (int)d) return;       // the digit's own limb: taken from the input later
    const ConvBlock& __restrict__ b = a.blocks[d];
    const F64Arith ar(a.primes[o]);
    const unsigned col = tile * CW + cl;
    const int nsrc = b.nsrc;
    double acc[R];
    {
        const signed char* vp = a.v + (long)d * N + col;
        const double dm = b.dmod_d[o];
#pragma unroll
        for (int j = 0; j < R; j++) acc[j] = -(double)vp[(long)(g + j * G) * N2] * dm;        // |v| <= nsrc, |dmod| <= q/2: exact
    }
    // the limbs are read one ahead of their use
    u64 x[R], xn[R];
    {
        const u64* yl = a.y + (long)b.src_limb[0] * N + col;
#pragma unroll
        for (int j = 0; j < R; j++) x[j] = yl[(long)(g + j * G) * N2];
    }
    for (int s = 0; s < nsrc; s++) {
        const double hat = b.hat_d[o][s];
        const u64* yl = a.y + (long)b.src_limb[s + 1 < nsrc ? s + 1 : s] * N + col;
#pragma unroll
        for (int j = 0; j < R; j++) xn[j] = yl[(long)(g + j * G) * N2];
#pragma unroll
        for (int j = 0; j < R; j++) acc[j] += ar.mulmod(exact_u2d(x[j]), hat);
#pragma unroll
        for (int j = 0; j < R; j++) x[j] = xn[j];
    }
    double v[R];
#pragma unroll
    for (int j = 0; j < R; j++) v[j] = ar.balance(acc[j]);
    const double* tw = a.tw_fwd + (long)o * N;
    fwd_spread<F64Arith, 8, S1>(v, tw, 1u, ar);
#pragma unroll
    for (int j = 0; j < R; j++) lds[(g + j * G) * CW + cl] = v[j];
    __syncthreads();
#pragma unroll
    for (int j = 0; j < R; j++) v[j] = lds[(g * R + j) * CW + cl];
    fwd_packed<F64Arith, 8, S1>(v, tw, 1u, g, ar);
    mid_store_columns(a.mid + (long)limb * MID_LIMB_BYTES, tile, g, cl, v, ar);
}
int launch_hybrid_front_fused(ckks_ctx* c, const uint64_t* in_ntt, uint64_t* work, uint64_t* sums, const uint64_t* key, int l, bool* done,
                              uint64_t* out, int out_poly_mod_len, bool* finished) {
    *done = false;
    if (finished) *finished = false;
    if (ntt_pair_failed(c)) { set_error("an earlier one-launch transform of this context gave up a wait: the context is unusable"); return CKKS_E_UNAVAILABLE; }
    const int P = c->p_num, Q = c->q_num, W = P + Q;
    if (P <= 0 || l < 0 || l > c->L || !stage_fusion_applies(c, 0, P + l + 1)) return CKKS_OK;
    const int mod_num = P + l + 1, ndigits = (l + 1 + P - 1) / P, dnum = (Q + P - 1) / P;
    const ConvPlan& plan = c->plan_hybrid_all[l];
    if (plan.count != ndigits || !plan.f64_ok || !c->d_primes_modup) return CKKS_OK;
    const size_t in_bytes = (size_t)ndigits * mod_num * MID_LIMB_BYTES, out_bytes = (size_t)2 * mod_num * MID_LIMB_BYTES;
    if (in_bytes + out_bytes > (1ul << 30)) return CKKS_OK;
    int rc = ensure_mid(c, in_bytes + out_bytes);
    if (rc) return rc;
    typedef StridedCfg<8, 8> CS;
    typedef RowCfg<8, 8> CR;
    const long N = c->N;
    char* mid = (char*)c->d_ntt_mid;
    // inverse transform of the input; the second pass writes the scaled residues to `work` and leaves the input alone
    NttArgs args;
    args.primes = c->d_primes; args.tw = c->d_twd_inv; args.mid = mid;
    args.start_poly_idx = 0; args.start_mod_idx = P; args.poly_num = 1; args.mod_num = l + 1; args.poly_mod_len = Q;
    args.batch_stride_limbs = 0; args.limb_base = 0; args.limbs_total = (unsigned)(l + 1);
    args.data = (u64*)in_ntt;
    KsModUpArgs u;
    u.y = (const u64*)work; u.v = (signed char*)(work + (size_t)(l + 1) * N); u.mid = mid; u.blocks = c->d_conv + plan.first;
    u.primes = c->d_primes; u.tw_fwd = c->d_twd_fwd; u.ndigits = ndigits; u.p_num = P;
    if (pair_applies(c, l + 1, PAIR_KIND_F64)) {
        // one launch: the constants that differ between the two tables (N^-1 and the last twiddle) only enter the second pass
        args.primes = c->d_primes_modup + (size_t)l * c->nprimes;
        args.out_delta = (long)((u64*)work - (u64*)in_ntt);
        if ((rc = launch_pair<F64Arith, 8, 8>(c, args, l + 1, true, true, mid))) return rc;
        args.out_delta = 0;
    } else {
        hipLaunchKernelGGL((ntt_row_pass<F64Arith, 8, 8, true, true>), dim3(CR::TILES, l + 1), dim3(CR::THREADS), 0, c->stream, args);
        args.data = (u64*)work; args.primes = c->d_primes_modup + (size_t)l * c->nprimes;
        hipLaunchKernelGGL((ntt_strided_pass<F64Arith, 8, 8, true, true>), dim3(CS::TILES, l + 1), dim3(CS::THREADS), 0, c->stream, args);
    }
    // quotient estimates, then the conversion inside the first pass of the digits' forward transform
    hipLaunchKernelGGL(ks_modup_quotient_kernel, dim3((unsigned)(N / 256), ndigits), dim3(256), 0, c->stream, u);
    hipLaunchKernelGGL(ks_modup_strided_kernel, dim3(ndigits * mod_num, CS::TILES), dim3(256), 0, c->stream, u);
    // row passes of both transforms around the inner product
    KsRowArgs k;
    k.mid_in = mid; k.mid_out = mid + in_bytes; k.key = (const u64*)key; k.primes = c->d_primes;
    k.tw_fwd = c->d_twd_fwd; k.tw_inv = c->d_twd_inv; k.ndigits = ndigits; k.key_digit_stride = W; k.key_z_stride = (long)dnum * W;
    k.in_ntt = (const u64*)in_ntt; k.p_num = P;
    hipLaunchKernelGGL(ks_row_fused_kernel, dim3(CR::TILES, mod_num), dim3(256), 0, c->stream, k);
    // The last launch's ModDown workgroups wait for the special-prime workgroups at the front of the same grid, which is only sound
    // while the whole grid is resident at once; otherwise (and with the tuning switch set) the steps go out as separate launches.
    const bool back_fits = (unsigned)(P + l + 1) * 32u <= c->pair_resident_blocks[PAIR_KIND_KS_BACK];
    if (out && finished && !c->ks_back_split && back_fits && c->d_ntt_pair && pair_applies(c, 2 * mod_num, PAIR_KIND_KS_BACK)) {
        // last pass of the sums' inverse transform, ModDown and both passes of the results' forward transform in one launch
        KsBackArgs bk;
        bk.mid_in = k.mid_out; bk.sums = (u64*)sums; bk.z_stride = (long)W * N; bk.mid_out = mid;
        bk.primes = c->d_primes_moddown; bk.tw_inv = c->d_twd_inv; bk.tw_fwd = c->d_twd_fwd;
        bk.pHatVecModq = c->d_pHatVecModq; bk.PinvModq = c->d_PinvModq;
        bk.count = (unsigned*)c->d_ntt_pair + (size_t)PAIR_MAX_LIMBS * PAIR_WORD_STRIDE;
        bk.pair = pair_args(c, 2 * (l + 1));
        bk.out = (u64*)out; bk.out_z_stride = (long)out_poly_mod_len * N;
        bk.K = P; bk.nq = l + 1;
        hipLaunchKernelGGL(ks_back_kernel, dim3((unsigned)(P + l + 1) * 32u), dim3(256), 0, c->stream, bk);
        CKKS_HIP_TRY(hipGetLastError());
        *done = true;
        *finished = true;
        return CKKS_OK;
    }
    // second pass of the sums' inverse transform, special-prime limbs scaled for the ModDown that follows
    args.data = (u64*)sums; args.primes = c->d_primes_moddown; args.tw = c->d_twd_inv; args.mid = k.mid_out;
    args.start_mod_idx = 0; args.poly_num = 2; args.mod_num = mod_num; args.poly_mod_len = W; args.limbs_total = (unsigned)(2 * mod_num);
    hipLaunchKernelGGL((ntt_strided_pass<F64Arith, 8, 8, true, true>), dim3(CS::TILES, 2 * mod_num), dim3(CS::THREADS), 0, c->stream, args);
    CKKS_HIP_TRY(hipGetLastError());
    *done = true;
    return CKKS_OK;
}

// ------------------------------------------------------------------------------------------------------------
// Ring packing: the row pass of the forward transform of the embedded polynomials and their inner product with the repacking
// keys (mlweCipherPacking, PCMM_Scheme.cuh:389-401) in one launch.  Workgroup (16 rows, limb, chunk) runs the row pass of the
// polynomials of its chunk one after the other and accumulates their products with both key polynomials in registers; the
// chunks' partial sums (canonical residues) are added by a second small kernel.  The transformed polynomials, two limbs each,
// are never written: that is a write and a read of 2 * rank limbs less than the separate launches.
// ------------------------------------------------------------------------------------------------------------
struct RepackRowArgs {
    const char* mid;             // embedded polynomials after the first pass of their forward transform: limb (i, im) lies
    long stride_i, stride_im;    //   at mid + i * stride_i + im * stride_im bytes, in the form MID
    const u64* keys;             // key i = [a: 2 limbs | b: 2 limbs], NTT domain
    u64* partial;                // [chunk][z][im][N]
    const PrimeConst* primes;
    const double* tw_fwd;
    int rank, chunk, prime0;     // limb im is modulo prime prime0 + im of the context
};
template <class AR, class MID>
__global__ __launch_bounds__(256, 2) void repack_row_fused_kernel(RepackRowArgs a) {
    typedef RowCfg<8, 8> C;
    constexpr bool WIDE = std::is_same<AR, F64WideArith>::value;
    constexpr int S1 = C::S1, R = C::R, N2 = C::N2, U = C::U, N1 = C::N1, ROWS = C::ROWS;
    constexpr long N = 1l << 16;
    __shared__ double lds[C::LDS_WORDS];
    const unsigned tile = blockIdx.x, im = blockIdx.y, tid = threadIdx.x;
    const int prime = a.prime0 + (int)im;
    const AR ar(a.primes[prime]);
    const double* twf = a.tw_fwd + (long)prime * N;
    const unsigned u = tid % U, rl = tid / U;
    const unsigned row = tile * ROWS + rl;
    double* lrow = lds + rl * C::PITCH;
    const unsigned tw_off = N1 + row;
    const int i0 = (int)blockIdx.z * a.chunk, i1 = min(a.rank, i0 + a.chunk);
    double acc[2][R];
#pragma unroll
    for (int j = 0; j < R; j++) acc[0][j] = acc[1][j] = 0.0;
    typename MID::Raw raw;
    auto request = [&](int i) { MID::request(a.mid + i * a.stride_i + im * a.stride_im, tile, rl, u, raw); };
    if (i0 < i1) request(i0);
    for (int i = i0; i < i1; i++) {
        const u64* ka = a.keys + ((long)i * 4 + im) * N + (long)row * N2 + u;
        const u64* kb = ka + 2 * N;
        double v[R];
        unsigned two = tw_off;                              // opaque per polynomial: the twiddle loads stay inside the loop
        asm volatile("" : "+v"(two));
#pragma unroll
        for (int j = 0; j < R; j++) v[j] = MID::decode(ar, raw, j, rl);
        fwd_spread<AR, 8, S1>(v, twf, two, ar);
        ar.round_end(v);
#pragma unroll
        for (int j = 0; j < R; j++) lrow[padded(u + j * U)] = v[j];           // the words this lane read last: no barrier before
        __syncthreads();
#pragma unroll
        for (int j = 0; j < R; j++) v[j] = lrow[padded(u * R + j)];
        fwd_packed<AR, 8, S1>(v, twf, two, u, ar);
        __syncthreads();
#pragma unroll
        for (int j = 0; j < R; j++) lrow[padded(u * R + j)] = v[j];
        u64 k0[R], k1[R];
#pragma unroll
        for (int j = 0; j < R; j++) { k0[j] = ka[j * U]; k1[j] = kb[j * U]; }
        if (i + 1 < i1) request(i + 1);
        __syncthreads();
#pragma unroll
        for (int j = 0; j < R; j++) {
            const double x = ar.balance(lrow[padded(u + j * U)]);
            if constexpr (WIDE) {                                             // key words balanced: each term within 0.6 q of zero
                acc[0][j] += ar.mulmod(x, ar.from_canonical(k0[j]));
                acc[1][j] += ar.mulmod(x, ar.from_canonical(k1[j]));
            } else {
                acc[0][j] += ar.mulmod(x, (double)(long long)k0[j]);          // each term in (-0.51 q, 0.51 q): exact over any chunk
                acc[1][j] += ar.mulmod(x, (double)(long long)k1[j]);          // of fewer than 2^13 polynomials
            }
        }
        if constexpr (WIDE) {
            if (((i - i0) & 3) == 3) {                                        // four terms on a balanced sum: below 3 q < 2^52
#pragma unroll
                for (int j = 0; j < R; j++) { acc[0][j] = ar.balance(acc[0][j]); acc[1][j] = ar.balance(acc[1][j]); }
            }
        }
    }
#pragma unroll
    for (int z = 0; z < 2; z++) {
        u64* out = a.partial + (((long)blockIdx.z * 2 + z) * 2 + im) * N + (long)row * N2 + u;
#pragma unroll
        for (int j = 0; j < R; j++) out[j * U] = ar.canon(ar.balance(acc[z][j]));
    }
}
template <class AR>
__global__ __launch_bounds__(256) void repack_reduce_kernel(const u64* partial, u64* acc, const PrimeConst* primes, int prime0, int chunks) {
    constexpr long N = 1l << 16;
    const long x = (long)blockIdx.x * 256 + threadIdx.x;
    const int zi = blockIdx.y;                               // z * 2 + im
    const AR ar(primes[prime0 + (zi & 1)]);
    double s = 0.0;
    for (int ch = 0; ch < chunks; ch++) s += ar.from_canonical(partial[((long)ch * 4 + zi) * N + x]);      // at most 16 terms below q (q / 2 for wide primes): exact
    acc[(long)zi * N + x] = ar.canon(ar.balance(s));
}

// work: 2 * rank limbs (the area of the embedded polynomials, which this path never writes); acc: [z][im][N] sums, NTT domain.
// *done = false (nothing launched) where it does not apply.
int launch_repack_front_fused(ckks_ctx* c, uint64_t* work, uint64_t* acc, const uint64_t* keys, int rank, int prime0,
                              const NttEmbedSource& src, bool* done) {
    *done = false;
    const int form = rank < 1 ? 0 : stage_fusion_form(c, prime0, 2);
    if (form == 0) return CKKS_OK;
    if (!src.mlwe || src.logk < 0 || src.loggap < 0 || src.loggap > src.logk || src.n1 <= 0 || ((long)src.n1 << src.logk) != c->N ||
        (1 << src.logk) != rank) return CKKS_OK;
    int chunks = 16;
    while (chunks > 1 && (chunks * 4 > 2 * rank || chunks > rank)) chunks >>= 1;
    const int chunk = (rank + chunks - 1) / chunks;
    if (chunks * 4 > 2 * rank || chunk >= (1 << 13)) return CKKS_OK;
    // form 1: first pass into the inter-pass pieces, partial sums into `work`; form 2: first pass into `work` as whole limbs
    // (polynomial i, limb im at limb index 2 i + im), partial sums into the inter-pass area
    const size_t mid_bytes = form == 1 ? (size_t)2 * rank * MidPieces::LIMB_BYTES : (size_t)chunks * 4 * c->N * sizeof(u64);
    if (mid_bytes > (1ul << 30)) return CKKS_OK;
    int rc = ensure_mid(c, mid_bytes);
    if (rc) return rc;
    typedef StridedCfg<8, 8> CS;
    NttArgs args;
    args.data = (u64*)work; args.primes = c->d_primes; args.tw = c->d_twd_fwd; args.mid = form == 1 ? (char*)c->d_ntt_mid : nullptr;
    args.start_poly_idx = 0; args.start_mod_idx = prime0; args.poly_num = rank; args.mod_num = 2; args.poly_mod_len = 2;
    args.batch_stride_limbs = 0; args.limb_base = 0; args.limbs_total = (unsigned)(2 * rank);
    args.embed_mlwe = (const u64* const*)src.mlwe;
    args.embed_p0 = src.p0; args.embed_q0 = src.q0;
    args.embed_logk = src.logk; args.embed_loggap = src.loggap; args.embed_n1 = src.n1;
    args.embed_no_wrap = src.q0 / 2 < src.p0 ? 1 : 0;
    RepackRowArgs r;
    r.keys = (const u64*)keys; r.primes = c->d_primes; r.tw_fwd = c->d_twd_fwd;
    r.rank = rank; r.chunk = chunk; r.prime0 = prime0;
    const dim3 gs(CS::TILES, 2 * rank), gr(RowCfg<8, 8>::TILES, 2, chunks), gd((unsigned)(c->N / 256), 4);
    if (form == 1) {
        r.mid = (const char*)c->d_ntt_mid; r.stride_i = MidPieces::LIMB_BYTES; r.stride_im = (long)rank * MidPieces::LIMB_BYTES;
        r.partial = (u64*)work;
        hipLaunchKernelGGL((ntt_strided_pass<F64Arith, 8, 8, false, true, true>), gs, dim3(CS::THREADS), 0, c->stream, args);
        hipLaunchKernelGGL((repack_row_fused_kernel<F64Arith, MidPieces>), gr, dim3(256), 0, c->stream, r);
        hipLaunchKernelGGL(repack_reduce_kernel<F64Arith>, gd, dim3(256), 0, c->stream, (const u64*)r.partial, (u64*)acc,
                           (const PrimeConst*)c->d_primes, prime0, chunks);
    } else {
        r.mid = (const char*)work; r.stride_i = 2 * MidLimb::LIMB_BYTES; r.stride_im = MidLimb::LIMB_BYTES;
        r.partial = (u64*)c->d_ntt_mid;
        hipLaunchKernelGGL((ntt_strided_pass<F64WideArith, 8, 8, false, false, true>), gs, dim3(CS::THREADS), 0, c->stream, args);
        hipLaunchKernelGGL((repack_row_fused_kernel<F64WideArith, MidLimb>), gr, dim3(256), 0, c->stream, r);
        hipLaunchKernelGGL(repack_reduce_kernel<F64WideArith>, gd, dim3(256), 0, c->stream, (const u64*)r.partial, (u64*)acc,
                           (const PrimeConst*)c->d_primes, prime0, chunks);
    }
    CKKS_HIP_TRY(hipGetLastError());
    *done = true;
    return CKKS_OK;
}

// ------------------------------------------------------------------------------------------------------------
// Rescale (Scheme_23.cuh:321-385) after the inverse transform of the last limb: the reduction of that limb modulo every
// remaining prime happens while the first pass of its forward transform loads it, and the final (c_i - x) * q_l^-1 in the
// second pass, on the values it has just computed, before it stores.  Two launches where the separate steps take four.
// ------------------------------------------------------------------------------------------------------------
struct RescaleArgs {
    u64* cipher;                 // [2][poly_mod_len] limbs; limb l in the coefficient domain, limbs < l in the NTT domain
    char* mid;                   // limb index i * 2 + z
    const PrimeConst* primes;
    const double* tw_fwd;
    const u64* inv;              // q_l^-1 mod q_i, i < l
    int l, poly_mod_len, prime0; // limb i is modulo prime prime0 + i
};
// SHARED: the two tiles are the halves of one paired launch (what the first hands to the second moves as shared accesses)
template <class AR, class MID, bool SHARED>
__device__ __forceinline__ void rescale_strided_tile(const RescaleArgs& a, unsigned limb, unsigned tile, double* lds, const TileClaim& claim = TileClaim()) {
    typedef StridedCfg<8, 8> C;
    constexpr int S1 = C::S1, R = C::R, N2 = C::N2, G = C::G, CW = C::CW;
    constexpr long N = 1l << 16;
    const unsigned i = limb >> 1, z = limb & 1, tid = threadIdx.x;
    const unsigned cl = tid % CW, g = tid / CW;
    const int prime = a.prime0 + (int)i;
    const AR ar(a.primes[prime]);
    const u64* col = a.cipher + ((long)z * a.poly_mod_len + a.l) * N + tile * CW + cl;
    double v[R];
#pragma unroll
    for (int j = 0; j < R; j++) v[j] = ar.balance(exact_u2d(col[(long)(g + j * G) * N2]));      // x mod q_i, |.| <= q_i / 2
    const unsigned claimed = claim.start(tid);
    const double* tw = a.tw_fwd + (long)prime * N;
    fwd_spread<AR, 8, S1>(v, tw, 1u, ar);
    ar.round_end(v);
#pragma unroll
    for (int j = 0; j < R; j++) lds[(g + j * G) * CW + cl] = v[j];
    claim.publish(tid, claimed);
    __syncthreads();
    if (claim.lost()) return;
#pragma unroll
    for (int j = 0; j < R; j++) v[j] = lds[(g * R + j) * CW + cl];
    fwd_packed<AR, 8, S1>(v, tw, 1u, g, ar);
    MID::template store_columns<AR, SHARED>(a.mid + (long)limb * MID::LIMB_BYTES, tile, g, cl, v, ar);
}
template <class AR, class MID, bool SHARED>
__device__ __forceinline__ void rescale_row_tile(const RescaleArgs& a, unsigned limb, unsigned tile, double* lds, const TileClaim& claim = TileClaim()) {
    typedef RowCfg<8, 8> C;
    constexpr int S1 = C::S1, R = C::R, N2 = C::N2, U = C::U, N1 = C::N1, ROWS = C::ROWS;
    constexpr long N = 1l << 16;
    const unsigned i = limb >> 1, z = limb & 1, tid = threadIdx.x;
    const int prime = a.prime0 + (int)i;
    const AR ar(a.primes[prime]);
    const double* tw = a.tw_fwd + (long)prime * N;
    const unsigned u = tid % U, rl = tid / U;
    const unsigned row = tile * ROWS + rl;
    double* lrow = lds + rl * C::PITCH;
    const unsigned tw_off = N1 + row;
    u64* rp = a.cipher + ((long)z * a.poly_mod_len + i) * N + (long)row * N2 + u;
    typename MID::Raw raw;
    MID::template request<SHARED>(a.mid + (long)limb * MID::LIMB_BYTES, tile, rl, u, raw);
    u64 c[R];                                            // the limb's own words, needed after the butterflies
#pragma unroll
    for (int j = 0; j < R; j++) c[j] = rp[j * U];
    const unsigned counted = claim.start(tid);
    double v[R];
#pragma unroll
    for (int j = 0; j < R; j++) v[j] = MID::decode(ar, raw, j, rl);
    fwd_spread<AR, 8, S1>(v, tw, tw_off, ar);
    ar.round_end(v);
#pragma unroll
    for (int j = 0; j < R; j++) lrow[padded(u + j * U)] = v[j];
    __syncthreads();
#pragma unroll
    for (int j = 0; j < R; j++) v[j] = lrow[padded(u * R + j)];
    fwd_packed<AR, 8, S1>(v, tw, tw_off, u, ar);
    __syncthreads();
#pragma unroll
    for (int j = 0; j < R; j++) lrow[padded(u * R + j)] = v[j];
    __syncthreads();
    const double inv = ar.from_canonical(a.inv[i]);     // balanced for wide primes: the product's quotient estimate needs |inv| <= q / 2
#pragma unroll
    for (int j = 0; j < R; j++) {
        const double x = ar.balance(lrow[padded(u + j * U)]);
        rp[j * U] = ar.canon(ar.mulmod(exact_u2d(c[j]) - x, inv));          // |c - x| < 1.5 q
    }
    claim.publish(tid, counted);
}
template <class AR, class MID>
__global__ __launch_bounds__(256) void rescale_strided_kernel(RescaleArgs a) {
    __shared__ double lds[StridedCfg<8, 8>::LDS_WORDS];
    rescale_strided_tile<AR, MID, false>(a, blockIdx.x, blockIdx.y, lds);
}
template <class AR, class MID>
__global__ __launch_bounds__(256) void rescale_row_kernel(RescaleArgs a) {
    __shared__ double lds[RowCfg<8, 8>::LDS_WORDS];
    rescale_row_tile<AR, MID, false>(a, blockIdx.y, blockIdx.x, lds);
}
// both in one launch, paired like ntt_pair_kernel
template <class AR, class MID>
__global__ __launch_bounds__(256, 4) void rescale_pair_kernel(RescaleArgs a, PairArgs p) {
    constexpr int LDS_WORDS = StridedCfg<8, 8>::LDS_WORDS > RowCfg<8, 8>::LDS_WORDS ? StridedCfg<8, 8>::LDS_WORDS : RowCfg<8, 8>::LDS_WORDS;
    constexpr unsigned TILES = StridedCfg<8, 8>::TILES;
    static_assert(TILES == RowCfg<8, 8>::TILES, "tile counts");
    __shared__ double lds[LDS_WORDS];
    __shared__ unsigned go;
    unsigned limb, tile;
    pair_block(p, blockIdx.x, TILES, limb, tile);
    if (limb >= p.limbs) return;
    pair_run(p, limb, tile, &go, true, [&](unsigned t, const TileClaim& claim) { rescale_strided_tile<AR, MID, true>(a, limb, t, lds, claim); },
             [&](unsigned t, const TileClaim& out) { rescale_row_tile<AR, MID, true>(a, limb, t, lds, out); });
}
// cipher: [2][poly_mod_len] limbs over q_0 .. (prime indices K + i); limb l already in the coefficient domain.
// *done = false (nothing launched) where it does not apply.
int launch_rescale_fused(ckks_ctx* c, uint64_t* cipher, int l, const uint64_t* inv, bool* done) {
    *done = false;
    if (ntt_pair_failed(c)) { set_error("an earlier one-launch transform of this context gave up a wait: the context is unusable"); return CKKS_E_UNAVAILABLE; }
    const int form = l < 1 || l > c->L ? 0 : stage_fusion_form(c, c->K, l + 1);
    if (form == 0) return CKKS_OK;
    const int limbs = 2 * l;
    int rc = ensure_mid(c, (size_t)limbs * (form == 1 ? MidPieces::LIMB_BYTES : MidLimb::LIMB_BYTES));
    if (rc) return rc;
    RescaleArgs r;
    r.cipher = (u64*)cipher; r.mid = (char*)c->d_ntt_mid; r.primes = c->d_primes; r.tw_fwd = c->d_twd_fwd; r.inv = (const u64*)inv;
    r.l = l; r.poly_mod_len = c->L + 1; r.prime0 = c->K;
    const dim3 gs(limbs, StridedCfg<8, 8>::TILES), gr(RowCfg<8, 8>::TILES, limbs);
    if (pair_applies(c, limbs, form == 1 ? PAIR_KIND_RESCALE : PAIR_KIND_RESCALE_WIDE) && c->d_ntt_pair) {
        const PairArgs p = pair_args(c, limbs);
        const dim3 gp(pair_blocks(limbs, StridedCfg<8, 8>::TILES));
        if (form == 1) hipLaunchKernelGGL((rescale_pair_kernel<F64Arith, MidPieces>), gp, dim3(256), 0, c->stream, r, p);
        else hipLaunchKernelGGL((rescale_pair_kernel<F64WideArith, MidLimb>), gp, dim3(256), 0, c->stream, r, p);
    } else if (form == 1) {
        hipLaunchKernelGGL((rescale_strided_kernel<F64Arith, MidPieces>), gs, dim3(256), 0, c->stream, r);
        hipLaunchKernelGGL((rescale_row_kernel<F64Arith, MidPieces>), gr, dim3(256), 0, c->stream, r);
    } else {
        hipLaunchKernelGGL((rescale_strided_kernel<F64WideArith, MidLimb>), gs, dim3(256), 0, c->stream, r);
        hipLaunchKernelGGL((rescale_row_kernel<F64WideArith, MidLimb>), gr, dim3(256), 0, c->stream, r);
    }
    CKKS_HIP_TRY(hipGetLastError());
    *done = true;
    return CKKS_OK;
}

// in: two extended polynomials [P | Q_l] in the coefficient domain, in_z_stride words apart; out: two polynomials of
// out_poly_mod_len limbs, written in the NTT domain on limbs 0 .. l.  *done = false (nothing launched) where it does not apply.
int launch_ks_moddown_fused(ckks_ctx* c, uint64_t* out, const uint64_t* in, long in_z_stride, int l, int out_poly_mod_len, bool pre_scaled,
                            bool* done, const uint64_t* addend, long addend_poly_stride) {
    *done = false;
    const int form = c->p_num <= 0 || l < 0 || l > c->L ? 0 : stage_fusion_form(c, 0, c->K + l + 1);
    if (form == 0 || (form == 2 && c->K > 8)) return CKKS_OK;
    const int limbs = 2 * (l + 1);
    const long N = c->N;
    KsModDownArgs m;
    m.in = (const u64*)in; m.in_z_stride = in_z_stride; m.primes = c->d_primes; m.tw_fwd = c->d_twd_fwd;
    m.pHatVecModq = c->d_pHatVecModq; m.pHatInv = c->d_pHatInvVecModp; m.PinvModq = c->d_PinvModq; m.K = c->K; m.pre_scaled = pre_scaled ? 1 : 0;
    NttArgs args;
    args.data = (u64*)out; args.primes = c->d_primes; args.tw = c->d_twd_fwd;
    args.start_poly_idx = 0; args.start_mod_idx = c->K; args.poly_num = 2; args.mod_num = l + 1; args.poly_mod_len = out_poly_mod_len;
    args.batch_stride_limbs = 0; args.limb_base = 0; args.limbs_total = (unsigned)limbs;
    const dim3 gs(limbs, StridedCfg<8, 8>::TILES), gr(RowCfg<8, 8>::TILES, limbs);
    if (form == 1) {
        int rc = ensure_mid(c, (size_t)limbs * MidPieces::LIMB_BYTES);
        if (rc) return rc;
        m.mid = (char*)c->d_ntt_mid; m.mid_stride_i = 2 * MidPieces::LIMB_BYTES; m.mid_stride_z = MidPieces::LIMB_BYTES;
        args.mid = (char*)c->d_ntt_mid;
        hipLaunchKernelGGL((ks_moddown_strided_kernel<F64Arith, MidPieces>), gs, dim3(256), 0, c->stream, m);
        if (addend) hipLaunchKernelGGL((ntt_row_pass_add<F64Arith, 8, 8, true>), gr, dim3(RowCfg<8, 8>::THREADS), 0, c->stream, args, (const u64*)addend, addend_poly_stride);
        else hipLaunchKernelGGL((ntt_row_pass<F64Arith, 8, 8, false, true>), gr, dim3(RowCfg<8, 8>::THREADS), 0, c->stream, args);
    } else {
        // wide primes: the first pass writes the output limbs themselves, as an in-place transform leaves them between its passes
        m.mid = (char*)out; m.mid_stride_i = N * (long)sizeof(u64); m.mid_stride_z = (long)out_poly_mod_len * N * (long)sizeof(u64);
        args.mid = nullptr;
        hipLaunchKernelGGL((ks_moddown_strided_kernel<F64WideArith, MidLimb>), gs, dim3(256), 0, c->stream, m);
        if (addend) hipLaunchKernelGGL((ntt_row_pass_add<F64WideArith, 8, 8, false>), gr, dim3(RowCfg<8, 8>::THREADS), 0, c->stream, args, (const u64*)addend, addend_poly_stride);
        else hipLaunchKernelGGL((ntt_row_pass<F64WideArith, 8, 8, false, false>), gr, dim3(RowCfg<8, 8>::THREADS), 0, c->stream, args);
    }
    CKKS_HIP_TRY(hipGetLastError());
    *done = true;
    return CKKS_OK;
}

// External product with the switching key and inverse transform of the sums (KeySwitch_23.cuh:225-226) in two launches where the
// separate steps take three (or two with a write and a read of every sum between them); *done = false where it does not apply.
int launch_ext_product_inverse_fused(ckks_ctx* c, uint64_t* ext, const uint64_t* up, const uint64_t* swk, int l, bool* done) {
    *done = false;
    if (c->ks_split || c->logN != 16 || c->ntt_mode != 0 || c->ev_mid_armed || c->t_num <= 0 || c->gamma <= 0 || c->p_num <= 0) return CKKS_OK;
    if ((((uintptr_t)up | (uintptr_t)swk) & 15u) != 0) return CKKS_OK;                      // the product phase reads 16 bytes at a time
    const int T = c->t_num, prime0 = c->p_num + c->q_num;
    // the integer back end is what the transforms over T would run on: every T prime too wide for the FP64 forms, or the context set to integers
    for (int j = 0; j < T; j++)
        if (c->arith_mode == 0 && c->pqt[prime0 + j] < (1ull << 50)) return CKKS_OK;
    const int ndigits = (l + 1 + c->p_num - 1) / c->p_num;                                   // cipher_blockNum, ExternalProduct.cuh:87
    if (ndigits > c->dnum) { set_error("external_product_T: the level needs more digits than the key holds (q_num is no multiple of p_num)"); return CKKS_E_INVALID; }
    const int blocks = (c->p_num + l + 1 + c->gamma - 1) / c->gamma;                         // :88
    ExtRowArgs a;
    a.c = (const u64*)up; a.key = (const u64*)swk; a.out = (u64*)ext; a.primes = c->d_primes; a.tw_inv = (const ulonglong2*)c->d_tw_inv;
    a.ndigits = ndigits; a.t_num = T; a.blocks = blocks; a.prime0 = prime0;
    a.key_digit_stride = (long)T * c->Ri_blockNum; a.key_z_stride = (long)c->Ri_blockNum * T * c->dnum; a.out_z_stride = (long)c->Ri_blockNum * T;
    const int limbs = 2 * blocks * T;
    hipLaunchKernelGGL(ext_row_fused_kernel, dim3((unsigned)(RowCfg<8, 8>::TILES * limbs)), dim3(256), 0, c->stream, a);
    NttArgs args;
    args.data = (u64*)ext; args.primes = c->d_primes; args.tw = c->d_tw_inv;
    args.start_poly_idx = 0; args.start_mod_idx = prime0; args.poly_num = blocks; args.mod_num = T; args.poly_mod_len = T;
    args.batch_stride_limbs = a.out_z_stride; args.limb_base = 0; args.limbs_total = (unsigned)limbs; args.mid = nullptr;
    hipLaunchKernelGGL((ntt_strided_pass<IntArith, 8, 8, true, false>), dim3(StridedCfg<8, 8>::TILES, limbs), dim3(StridedCfg<8, 8>::THREADS), 0, c->stream, args);
    CKKS_HIP_TRY(hipGetLastError());
    *done = true;
    return CKKS_OK;
}

// Workgroups of each one-launch kernel that the chip holds at once: its occupancy times the compute units.
static void pair_resident_blocks(ckks_ctx* c) {
    const unsigned cus = (unsigned)(c->cu_count > 0 ? c->cu_count : 1);
    auto ask = [&](int kind, auto kernel) {
        int n = 0;
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, kernel, 256, 0) != hipSuccess) { (void)hipGetLastError(); n = 1; }
        if (n < 1) n = 1;
        const unsigned blocks = (unsigned)n * cus;
        if (c->pair_resident_blocks[kind] == 0 || blocks < c->pair_resident_blocks[kind]) c->pair_resident_blocks[kind] = blocks;
    };
    ask(PAIR_KIND_F64, ntt_pair_kernel<F64Arith, 8, 8, false, true>);
    ask(PAIR_KIND_F64, ntt_pair_kernel<F64Arith, 8, 8, true, true>);
    ask(PAIR_KIND_F64, ntt_pair_kernel<F64Arith, 8, 8, false, false>);
    ask(PAIR_KIND_F64, ntt_pair_kernel<F64Arith, 8, 8, true, false>);
    ask(PAIR_KIND_WIDE, ntt_pair_kernel<F64WideArith, 8, 8, false, false>);
    ask(PAIR_KIND_WIDE, ntt_pair_kernel<F64WideArith, 8, 8, true, false>);
    ask(PAIR_KIND_INT, ntt_pair_kernel<IntArith, 8, 8, false, false>);
    ask(PAIR_KIND_INT, ntt_pair_kernel<IntArith, 8, 8, true, false>);
    ask(PAIR_KIND_RESCALE, rescale_pair_kernel<F64Arith, MidPieces>);
    ask(PAIR_KIND_RESCALE_WIDE, rescale_pair_kernel<F64WideArith, MidLimb>);
    ask(PAIR_KIND_KS_BACK, ks_back_kernel);
}

static int launch_ntt_from(ckks_ctx* c, uint64_t* dev, int start_poly_idx, int start_mod_idx, int poly_num, int mod_num,
                           int poly_mod_len, long batch_stride_limbs, int batch, bool inverse, const NttEmbedSource* src,
                           const NttFixedArea* fixed = nullptr);

int launch_ntt(ckks_ctx* c, uint64_t* dev, int start_poly_idx, int start_mod_idx, int poly_num, int mod_num,
               int poly_mod_len, long batch_stride_limbs, int batch, bool inverse) {
    return launch_ntt_from(c, dev, start_poly_idx, start_mod_idx, poly_num, mod_num, poly_mod_len, batch_stride_limbs, batch, inverse, nullptr);
}
// forward transform of poly_num polynomials that the first pass gathers from MLWE samples instead of reading them from dev
int launch_ntt_embedded(ckks_ctx* c, uint64_t* dev, int start_poly_idx, int start_mod_idx, int poly_num, int mod_num, int poly_mod_len,
                        const NttEmbedSource& src) {
    if (!src.mlwe || src.logk < 0 || src.loggap < 0 || src.loggap > src.logk || src.n1 <= 0 || ((long)src.n1 << src.logk) != c->N) {
        set_error("NTT: bad embedding source");
        return CKKS_E_INVALID;
    }
    if (c->ntt_mode == 3) { set_error("NTT: the embedding source needs the two-launch transform"); return CKKS_E_INVALID; }
    return launch_ntt_from(c, dev, start_poly_idx, start_mod_idx, poly_num, mod_num, poly_mod_len, 0, 1, false, &src);
}

static int launch_ntt_from(ckks_ctx* c, uint64_t* dev, int start_poly_idx, int start_mod_idx, int poly_num, int mod_num,
                           int poly_mod_len, long batch_stride_limbs, int batch, bool inverse, const NttEmbedSource* src,
                           const NttFixedArea* fixed) {
    if (!c || !dev) { set_error("NTT: null argument"); return CKKS_E_INVALID; }
    if (ntt_pair_failed(c)) { set_error("NTT: an earlier one-launch transform of this context gave up waiting for its first pass"); return CKKS_E_UNAVAILABLE; }
    if (poly_num <= 0 || mod_num <= 0 || batch <= 0) return CKKS_OK;      // empty batch: nothing to do
    if (start_mod_idx < 0 || start_mod_idx + mod_num > c->nprimes || start_poly_idx < 0 || poly_mod_len < 0) {
        set_error("NTT: prime range outside the context");
        return CKKS_E_INVALID;
    }
    long limbs = (long)poly_num * mod_num * batch;
    if (limbs > 65535) { set_error("NTT: more than 65535 limbs in one call"); return CKKS_E_INVALID; }
    // back end per prime: 0 = FP64 (q < 2^41), 1 = FP64 with a balance per register round (q < 2^50), 2 = integer
    auto klass = [&](int j) {
        if (c->arith_mode != 0) return 2;
        const u64 m = c->pqt[start_mod_idx + j];
        return m < (1ull << 41) ? 0 : m < (1ull << 50) ? 1 : 2;
    };
    int back_end = klass(0);
    bool mixed = false, compact_ok = true, res36_ok = true;
    for (int j = 0; j < mod_num; j++) {
        mixed = mixed || klass(j) != back_end;
        compact_ok = compact_ok && c->pqt[start_mod_idx + j] < (1ull << 39);
        res36_ok = res36_ok && c->pqt[start_mod_idx + j] < (1ull << 36);
    }
    if (mixed) {
        // a call that spans prime widths ([P | Q | T] of the reference's sets: 49-bit P and Q, 60-bit T) goes out as one launch
        // sequence per run of primes of one back end; the timing hook and the gathering first pass take one back end for all
        if (c->ev_mid_armed || src) back_end = 2;
        else {
            for (int j0 = 0; j0 < mod_num;) {
                int j1 = j0 + 1;
                while (j1 < mod_num && klass(j1) == klass(j0)) j1++;
                const int rc = launch_ntt_from(c, dev, start_poly_idx + j0, start_mod_idx + j0, poly_num, j1 - j0, poly_mod_len, batch_stride_limbs,
                                               batch, inverse, nullptr, fixed);
                if (rc) return rc;
                j0 = j1;
            }
            return CKKS_OK;
        }
    }
    NttArgs args;
    args.data = (u64*)dev;
    args.primes = c->d_primes;
    args.start_poly_idx = start_poly_idx;
    args.start_mod_idx = start_mod_idx;
    args.poly_num = poly_num;
    args.mod_num = mod_num;
    args.poly_mod_len = poly_mod_len;
    args.batch_stride_limbs = batch_stride_limbs;
    if (src) {
        args.embed_mlwe = (const u64* const*)src->mlwe;
        args.embed_p0 = src->p0; args.embed_q0 = src->q0;
        args.embed_logk = src->logk; args.embed_loggap = src->loggap; args.embed_n1 = src->n1;
        args.embed_no_wrap = src->q0 / 2 < src->p0 ? 1 : 0;
    }
    if (back_end == 0) {
        args.tw = inverse ? (const void*)c->d_twd_inv : (const void*)c->d_twd_fwd;
        return dispatch_logn<F64Arith>(c, args, (int)limbs, inverse, compact_ok, res36_ok, fixed);
    }
    if (back_end == 1) {
        args.tw = inverse ? (const void*)c->d_twd_inv : (const void*)c->d_twd_fwd;
        return dispatch_logn<F64WideArith>(c, args, (int)limbs, inverse, false, false, fixed);
    }
    args.tw = inverse ? (const void*)c->d_tw_inv : (const void*)c->d_tw_fwd;
    return dispatch_logn<IntArith>(c, args, (int)limbs, inverse, false, false, fixed);
}

// ------------------------------------------------------------------------------------------------------------
// Transform that allocates nothing.  The two-launch transform at N = 2^16 hands its data from the first pass to the second in
// the 5-byte inter-pass form, in a buffer that the ordinary entry points allocate and grow on demand.  Callers that cannot
// allocate (HIP graph capture, serving loops, harnesses that forbid it) get the same transform with that buffer in a
// file-scope device array instead: NOALLOC_MAX_LIMBS limbs of 320 KiB, held by every GPU the library runs on until the
// process ends.  All calls on one GPU share the array, so calls that overlap on one GPU (two streams, two host threads)
// race; the first pass writes every byte the second pass reads, so nothing has to be cleared between calls.
// ------------------------------------------------------------------------------------------------------------
constexpr int NOALLOC_MAX_LIMBS = 64;
constexpr int NOALLOC_MAX_DEVICES = 64;
static __device__ __align__(256) unsigned char scratch[(size_t)NOALLOC_MAX_LIMBS * MID_LIMB_BYTES];
static std::mutex g_scratch_mutex;
static char* g_scratch_ptr[NOALLOC_MAX_DEVICES] = {};      // device address of `scratch` on each GPU (each GPU has its own copy)

// address of the array on the current device, looked up once per device (called from ckks_ctx_create, and again by the
// entry point for a device that no context was created on)
int ntt_noalloc_init(char** ptr_out) {
    int dev = -1;
    CKKS_HIP_TRY(hipGetDevice(&dev));
    if (dev < 0 || dev >= NOALLOC_MAX_DEVICES) { set_error("NTT: device index out of range"); return CKKS_E_INVALID; }
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void* p = nullptr;
        CKKS_HIP_TRY(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        if (!p) { set_error("NTT: no device address for the fixed inter-pass area"); return CKKS_E_HIP; }
        g_scratch_ptr[dev] = (char*)p;
    }
    if (ptr_out) *ptr_out = g_scratch_ptr[dev];
    return CKKS_OK;
}
int ntt_noalloc_max_limbs() { return NOALLOC_MAX_LIMBS; }

int launch_ntt_noalloc(ckks_ctx* c, uint64_t* dev, int start_poly_idx, int start_mod_idx, int poly_num, int mod_num, int poly_mod_len,
                       bool inverse) {
    if (!c || !dev) { set_error("NTT: null argument"); return CKKS_E_INVALID; }
    const long limbs = (long)poly_num * mod_num;
    if (poly_num > 0 && mod_num > 0 && limbs > NOALLOC_MAX_LIMBS) {
        set_error("ckks_ntt_noalloc: " + std::to_string(limbs) + " limbs in one call, the limit is " + std::to_string(NOALLOC_MAX_LIMBS));
        return CKKS_E_INVALID;
    }
    int cur = -1;
    CKKS_HIP_TRY(hipGetDevice(&cur));
    if (cur != c->device) { set_error("ckks_ntt_noalloc: the context was created on another device than the current one"); return CKKS_E_INVALID; }
    char* ptr = nullptr;
    int rc = ntt_noalloc_init(&ptr);
    if (rc) return rc;
    // two launches, inter-pass data in the fixed area where the 5-byte form applies and in place otherwise; the area travels
    // with the call, nothing of the context is changed
    const NttFixedArea fixed = {ptr, (size_t)NOALLOC_MAX_LIMBS * MID_LIMB_BYTES};
    return launch_ntt_from(c, dev, start_poly_idx, start_mod_idx, poly_num, mod_num, poly_mod_len, 0, 1, inverse, nullptr, &fixed);
}

}  // namespace ckks
