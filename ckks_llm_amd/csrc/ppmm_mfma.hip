// Dense PPMM on the CDNA4 int8 matrix cores.
//
// out[m][i][c] = fused-rescale( sum_n A[m][n] * Ct_n[i][c]  mod q_i )        (semantics: pcmm.hip, PPMM_kernel.cuh:93-252)
//
// Exact integer product through base-256 balanced digits:
//     A[m][n]  = sum_{d<DW} a_d[m][n] * 256^d ,  a_d in [-128,127]   (int8 planes built once per call, shared by all primes)
//     Ct[n][c] = sum_{j<DC} b_j[n][c] * 256^j ,  b_j in [-128,127]   (bytes of (x + 0x8080808080) xor 0x80, int8 planes built once per call)
//     sum_n A*Ct = sum_{e<DW+DC-1} 256^e * S_e ,   S_e = sum_{d+j=e} sum_n a_d*b_j    (int32, |S_e| <= min(DW,DC)*Kin*2^14)
// One v_mfma_i32_16x16x64_i8 per (d, j, 16x16 tile, 64 k) accumulates into the anti-diagonal accumulator S_{d+j}.
// The epilogue recombines the S_e without rounding in FP64 (four diagonals at a time stay below 2^53), reduces modulo q_i
// and applies the fused rescale (PPMM_kernel.cuh:213-249).
// Two residue widths are built: DC = 5 digits for q_i < 2^39 (the 36-bit sets of the benchmarks) and DC = 7 digits for
// q_i < 2^50 (the reference's own 49-bit ring-pack primes), the latter with DW <= 3.
//
#include <cstdlib>
#include <type_traits>

#include "f64_exact.hpp"
#include "pcmm.hpp"

namespace ckks {

typedef int v4i __attribute__((ext_vector_type(4)));

constexpr int CT = 64, KS = 64;                  // column tile and K step; the row tile is 16 rows per wave of the workgroup

typedef __attribute__((address_space(3))) void* lptr_t;
// 16 bytes per lane from global memory straight into LDS (no registers held while the load is in flight):
// lane l of the wave writes lds_base + 16*l.  lds_base must be wave-uniform (it travels in M0).
// Written as inline assembly on purpose: when the compiler sees LDS-DMA loads it makes every later LDS read that it cannot
// prove disjoint wait for ALL outstanding loads (vmcnt(0)), which serialises the ring.  Here the waits are explicit: a
// vmcnt(n) before the workgroup barrier that publishes a slot.  The compiler's own vmcnt bookkeeping stays safe because
// loads complete in order: extra loads in flight can only make one of its waits longer, never shorter.
__device__ __forceinline__ void async_copy16(const void* g, void* lds_base) {
    const unsigned l = (unsigned)(size_t)(lptr_t)lds_base;
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(g), "s"(l) : "memory", "m0");
}

// mulmod_f64, balance_f64 and the per-output statement of the epilogue (ppmm_recombine, ppmm_recombine_wide) are in f64_exact.hpp,
// where a host build checks their ranges

// ------------------------------------------------------------------------------------------------------------
// Pass 1: residue digit planes.  Every residue is read ONCE, split into DC balanced base-256 digits and written in the
// order the MFMA kernel stages it:  Bdig[prime][K step][64-column tile][digit][16-column slab] slabs of 1 KiB, inside a slab
// [16-byte k chunk][column][16 k].
// One workgroup (256 lanes) handles 64 k x 64 columns: coalesced 512 B row reads, a byte transpose in registers,
// LDS to gather the 4 waves' quarter rows, then 16 B per lane coalesced writes.
// ------------------------------------------------------------------------------------------------------------
template <int DC>
__global__ __launch_bounds__(256) void ppmm_pack_kernel(PpmmArgs a, int8_t* __restrict__ bdig) {
    static_assert(DC == 5 || DC == 7, "residue digits");
    constexpr u64 BIAS = DC == 5 ? 0x8080808080ull : 0x80808080808080ull;         // bytes of x + BIAS = balanced digit + 128
    __shared__ __align__(16) int8_t tile[DC][CT][KS];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const unsigned c0 = blockIdx.x * CT;
    const int ks = blockIdx.y, im = blockIdx.z;
    const long col_word = (long)im * a.C + c0 + lane;
    uint4 dig[DC];
    unsigned* dw = reinterpret_cast<unsigned*>(dig);
#pragma unroll
    for (int g = 0; g < 4; g++) {
        u64 y[4];
#pragma unroll
        for (int i = 0; i < 4; i++) y[i] = a.mlwe[ks * KS + 16 * wave + 4 * g + i][col_word] + BIAS;
        const unsigned x0 = (unsigned)y[0], x1 = (unsigned)y[1], x2 = (unsigned)y[2], x3 = (unsigned)y[3];
        const unsigned t0 = __byte_perm(x0, x1, 0x5140), t1 = __byte_perm(x0, x1, 0x7362);
        const unsigned t2 = __byte_perm(x2, x3, 0x5140), t3 = __byte_perm(x2, x3, 0x7362);
        dw[0 * 4 + g] = __byte_perm(t0, t2, 0x5410) ^ 0x80808080u;
        dw[1 * 4 + g] = __byte_perm(t0, t2, 0x7632) ^ 0x80808080u;
        dw[2 * 4 + g] = __byte_perm(t1, t3, 0x5410) ^ 0x80808080u;
        dw[3 * 4 + g] = __byte_perm(t1, t3, 0x7632) ^ 0x80808080u;
        if constexpr (DC == 5) {
            const unsigned h01 = __byte_perm((unsigned)(y[0] >> 32), (unsigned)(y[1] >> 32), 0x0040);
            const unsigned h23 = __byte_perm((unsigned)(y[2] >> 32), (unsigned)(y[3] >> 32), 0x0040);
            dw[4 * 4 + g] = __byte_perm(h01, h23, 0x5410) ^ 0x80808080u;
        } else {
            const unsigned h0 = (unsigned)(y[0] >> 32), h1 = (unsigned)(y[1] >> 32), h2 = (unsigned)(y[2] >> 32), h3 = (unsigned)(y[3] >> 32);
            const unsigned u0 = __byte_perm(h0, h1, 0x5140), u1 = __byte_perm(h0, h1, 0x7362);
            const unsigned u2 = __byte_perm(h2, h3, 0x5140), u3 = __byte_perm(h2, h3, 0x7362);
            dw[4 * 4 + g] = __byte_perm(u0, u2, 0x5410) ^ 0x80808080u;
            dw[5 * 4 + g] = __byte_perm(u0, u2, 0x7632) ^ 0x80808080u;
            dw[6 * 4 + g] = __byte_perm(u1, u3, 0x5410) ^ 0x80808080u;
        }
    }
    // LDS chunk index xor-swizzled with the column so that the 64-byte-strided 16-byte stores spread over the banks
#pragma unroll
    for (int jj = 0; jj < DC; jj++) *reinterpret_cast<uint4*>(&tile[jj][lane][16 * (wave ^ ((lane >> 1) & 3))]) = dig[jj];
    __syncthreads();
    int8_t* dst = bdig + (((long)im * gridDim.y + ks) * gridDim.x + blockIdx.x) * (long)(DC * CT * KS);
#pragma unroll
    for (int t = 0; t < DC * CT * KS / (256 * 16); t++) {
        const int flat = (t * 256 + tid) * 16;                  // byte offset in [digit][16-column slab][16-byte k chunk][column][16]
        const int jj = flat / (CT * KS), col = ((flat >> 10) & 3) * 16 + ((flat >> 4) & 15), chunk = (flat >> 8) & 3;
        *reinterpret_cast<uint4*>(dst + flat) = *reinterpret_cast<const uint4*>(&tile[jj][col][16 * (chunk ^ ((col >> 1) & 3))]);
    }
}

// ------------------------------------------------------------------------------------------------------------
// Pass 2: the contraction.  A workgroup of 512 lanes = 8 waves (two per SIMD, so that one wave's waits and epilogue overlap
// the other's MFMAs) owns a 128 (M) x 64 (columns) output tile for all primes; wave (wm, wc) owns the 32 x 32 sub-tile at
// rows 32*wm, columns 32*wc = 2 x 2 MFMA tiles x (DW+DC-1) accumulators.
// K advances 64 per step through a three-deep LDS ring filled by asynchronous global->LDS loads issued two steps ahead
// (plaintext digit slabs of 16 rows x 64 B, residue digit slabs of 16 columns x 64 B; 1 KiB per wave instruction, nothing
// held in registers).  The ring runs across prime boundaries: global step s = prime iteration * ksteps + K step, slot s % 3.
// Every ring slot is a separate __shared__ object addressed with a compile-time index (the K loop is unrolled by 3 and
// ksteps is a multiple of 3), so that the compiler can tell that the asynchronous writes of a step never alias the
// operands its MFMAs read; otherwise it waits for the loads before the first LDS read and the overlap is lost.
// ------------------------------------------------------------------------------------------------------------
// The kernel is written for NWAVES waves (16 rows of the tile each) and a ring of RING slots; the launcher instantiates
//   NWAVES = 8, RING = 3: 128 x 64 tile, one workgroup per CU (135 KiB of LDS), loads issued two steps ahead.
// The other shape that fits the LDS (NWAVES = 4, RING = 2: 64 x 64 tile, 64 KiB, two workgroups per CU that drift out of phase)
// was measured and is no faster (its single step of load lead time costs what the overlap of the two workgroups gains).
template <int DW, int NWAVES, int RING, int DC>
__global__ __launch_bounds__(64 * NWAVES, 2) void ppmm_mfma_kernel(PpmmArgs a, const int8_t* __restrict__ bdig, int c_tiles, int m_block,
                                                                   int main_blocks, int tail_jobs) {
    constexpr int ND = DW + DC - 1, MT = 16 * NWAVES;
    constexpr bool WIDE = DC > 5;                                // residues of up to 50 bits: three groups of diagonals, wider r_last
    constexpr int A_SLABS = DW * (MT / 16), B_SLABS = DC * 4;    // 1 KiB slabs per step
    constexpr int A_PER_WAVE = (A_SLABS + NWAVES - 1) / NWAVES, B_PER_WAVE = (B_SLABS + NWAVES - 1) / NWAVES;
    constexpr int AHEAD = RING - 1;                              // how many steps ahead of its use a slot is refilled
    static_assert(RING == 2 || RING == 3, "ring depth");
    __shared__ __align__(16) int8_t lds_a0[DW][MT][KS];
    __shared__ __align__(16) int8_t lds_a1[DW][MT][KS];
    __shared__ __align__(16) int8_t lds_a2[RING == 3 ? DW : 1][RING == 3 ? MT : 1][KS];
    __shared__ __align__(16) int8_t lds_b0[DC][CT][KS];
    __shared__ __align__(16) int8_t lds_b1[DC][CT][KS];
    __shared__ __align__(16) int8_t lds_b2[RING == 3 ? DC : 1][RING == 3 ? CT : 1][KS];

    // XCD-aware tile numbering: ids congruent mod 8 share an XCD and start in increasing order there, about 32 at a time (one per
    // CU).  Those 32 should share operands inside the XCD's 4 MiB L2: consecutive ids form an m_block x (32 / m_block) patch of
    // tiles (m_block row tiles that all read the same column panels), and the patches sweep the column panels before moving to the
    // next m_block row tiles.  All workgroups of a patch advance through K at the same pace, so the L2 only has to hold a window of
    // their plaintext and residue slabs.  (With every row tile in one patch, 32 row tiles at M = 4096 re-read the plaintext digit
    // planes, which no longer fit the L2, for every column panel and prime: 40 times the algorithmic traffic.)
    //
    // Tail.  The column panels do not divide among the XCDs in general, and a tile is a long job (all primes): with 1026 panels
    // and six row tiles, six XCDs would sit idle for a whole round while two finish the last two panels.  With tail_jobs > 0 the
    // ids from main_blocks on are those panels' tiles cut into tail_jobs jobs each: a job computes the last prime (every other
    // prime's rescale needs its residues; job 0 stores them) and its share of the other primes, and the jobs spread over all XCDs.
    const unsigned id = blockIdx.x;
    unsigned m_tile, c_tile;
    int prime_lo = 0, prime_hi = a.mod_num - 1;          // the other primes of this workgroup: prime_lo .. prime_hi - 1, after the last one
    bool store_last = true;
    if (tail_jobs > 0 && id >= (unsigned)main_blocks) {
        const unsigned q = id - (unsigned)main_blocks, job = q % (unsigned)tail_jobs, tt = q / (unsigned)tail_jobs;
        const unsigned m_tiles = (unsigned)a.Mpad / MT;
        m_tile = tt % m_tiles;
        c_tile = ((unsigned)c_tiles / 8) * 8 + tt / m_tiles;
        const int others = a.mod_num - 1;
        prime_lo = (int)((long)others * job / tail_jobs);
        prime_hi = (int)((long)others * (job + 1) / tail_jobs);
        store_last = job == 0;
    } else {
        const unsigned xcd = id & 7, j = id >> 3;
        const unsigned c_per_xcd = tail_jobs > 0 ? (unsigned)c_tiles / 8 : ((unsigned)c_tiles + 7) / 8;
        const unsigned ml = j % m_block, t = j / m_block;
        m_tile = (t / c_per_xcd) * m_block + ml;
        c_tile = (t % c_per_xcd) * 8 + xcd;
    }
    if (c_tile >= (unsigned)c_tiles) return;
    const int n_iters = 1 + prime_hi - prime_lo;          // the last prime, then prime_hi - 1 down to prime_lo
    auto prime_of = [&](int it) { return it == 0 ? a.mod_num - 1 : prime_hi - it; };
    const int m0 = m_tile * MT;
    const unsigned c0 = c_tile * CT;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);          // wave-uniform
    const int wm = wave >> 1, wc = wave & 1;
    const int lr = lane & 15, lg = lane >> 4;
    // A 1 KiB slab (16 rows or columns x 64 k) is stored [16-byte k chunk g][row r][16 k] in global memory and in LDS alike, so that
    // lane lr + 16 lg, which needs chunk lg of row lr as its MFMA operand, reads byte 16 * lane of the slab, and the asynchronous load
    // that fills it (lane l writes byte 16 l) fetches 1 KiB of contiguous global memory.  A ds_read_b128 whose lanes read consecutive
    // 16-byte chunks runs at the full 256 B/clk of the LDS; every other assignment of the same 64 chunks to the 64 lanes measured
    // 1.7 times slower on this part, whatever the swizzle.
    const int frag_off = 16 * lane;
    const int ksteps = a.Kpad / KS;
    const long plane = (long)a.Mpad * a.Kpad;
    // plaintext digits: [digit][16-row group][K step] slabs
    const int8_t* a_lane = a.Adig + (long)(m0 / 16) * ksteps * 1024 + 16 * lane;
    // residue digits: [prime][K step][column tile][digit][16-column slab] slabs
    const long b_step = (long)c_tiles * (DC * CT * KS);                 // bytes per (prime, K step)
    const int8_t* b_lane = bdig + (long)c_tile * (DC * CT * KS) + 16 * lane;

    auto issue = [&](int ks, int im, int8_t (*adst)[MT][KS], int8_t (*bdst)[CT][KS]) {
#pragma unroll
        for (int t = 0; t < A_PER_WAVE; t++) {
            int slab = wave + NWAVES * t;
            slab = slab < A_SLABS ? slab : A_SLABS - 1;                  // surplus lanes re-load the last slab (same bytes)
            const int d = slab / (MT / 16), rr = slab % (MT / 16);
            async_copy16(a_lane + d * plane + ((long)rr * ksteps + ks) * 1024, &adst[d][rr * 16][0]);
        }
        const int8_t* bsrc = b_lane + ((long)im * ksteps + ks) * b_step;
#pragma unroll
        for (int t = 0; t < B_PER_WAVE; t++) {
            int slab = wave + NWAVES * t;
            slab = slab < B_SLABS ? slab : B_SLABS - 1;
            async_copy16(bsrc + slab * 1024, &bdst[0][0][0] + slab * 1024);
        }
    };
    auto wait_loads = [&]() {
        __builtin_amdgcn_s_waitcnt(0x0F70);        // vmcnt(0): this wave's asynchronous loads have landed in LDS
        __syncthreads();                            // ... and so have everybody else's
    };

    // (ks2, im2): K step and prime of global step s+AHEAD, advanced without divisions; past the end the loads re-fetch valid
    // data into slots nobody reads again, so that a step has no branches.
    // it2 counts this workgroup's primes; im2 = prime of that iteration, or -1 past the end
    int it2 = 0;
    auto advance = [&](int& ks, int& im) { if (++ks == ksteps) { ks = 0; ++it2; im = it2 < n_iters ? prime_of(it2) : -1; } };
    int ks2 = 0, im2 = a.mod_num - 1;
    issue(ks2, im2, lds_a0, lds_b0);
    advance(ks2, im2);
    if (RING == 3) {
        issue(im2 < 0 ? 0 : ks2, im2 < 0 ? 0 : im2, lds_a1, lds_b1);
        advance(ks2, im2);
    }
    wait_loads();

    v4i acc[ND][2][2];
    // one K step reading ring slot R (compile time), refilling the slot read one step ago for step s + AHEAD
    auto kstep = [&](auto slot) {
        constexpr int R = decltype(slot)::value, W = (R + RING - 1) % RING;
        typedef int8_t (*aslot_t)[MT][KS];
        typedef int8_t (*bslot_t)[CT][KS];
        aslot_t A_cur = R == 0 ? lds_a0 : R == 1 ? lds_a1 : reinterpret_cast<aslot_t>(lds_a2);
        bslot_t B_cur = R == 0 ? lds_b0 : R == 1 ? lds_b1 : reinterpret_cast<bslot_t>(lds_b2);
        aslot_t A_nxt = W == 0 ? lds_a0 : W == 1 ? lds_a1 : reinterpret_cast<aslot_t>(lds_a2);
        bslot_t B_nxt = W == 0 ? lds_b0 : W == 1 ? lds_b1 : reinterpret_cast<bslot_t>(lds_b2);
        // operand reads in the order the MFMAs consume them (LDS reads return in order, so the first MFMA waits for its own two
        // operands only): plaintext chunks of the first 16 rows, residue chunks of the first 16 columns, then the rest
        if constexpr (DC > 5) {
            // seven residue digits: 144 accumulator registers leave no room for both column halves' operands at once, so the
            // residue chunks of one half are read just before its MFMAs (column half outer, row half inner)
            v4i af[2][DW];
#pragma unroll
            for (int mt = 0; mt < 2; mt++)
#pragma unroll
                for (int d = 0; d < DW; d++) af[mt][d] = *reinterpret_cast<const v4i*>(&A_cur[d][wm * 32 + mt * 16][0] + frag_off);
#pragma unroll
            for (int nt = 0; nt < 2; nt++) {
                v4i bf[DC];
#pragma unroll
                for (int jj = 0; jj < DC; jj++) bf[jj] = *reinterpret_cast<const v4i*>(&B_cur[jj][wc * 32 + nt * 16][0] + frag_off);
#pragma unroll
                for (int mt = 0; mt < 2; mt++) {
#pragma unroll
                    for (int jj = 0; jj < DC; jj++)
#pragma unroll
                        for (int d = 0; d < DW; d++)
                            acc[d + jj][mt][nt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(af[mt][d], bf[jj], acc[d + jj][mt][nt], 0, 0, 0);
                    if (mt == 0 && nt == 0) issue(im2 < 0 ? 0 : ks2, im2 < 0 ? 0 : im2, A_nxt, B_nxt);
                }
            }
        } else {
            v4i bf[2][DC], af[2][DW];
#pragma unroll
            for (int d = 0; d < DW; d++) af[0][d] = *reinterpret_cast<const v4i*>(&A_cur[d][wm * 32][0] + frag_off);
#pragma unroll
            for (int nt = 0; nt < 2; nt++)
#pragma unroll
                for (int jj = 0; jj < DC; jj++) bf[nt][jj] = *reinterpret_cast<const v4i*>(&B_cur[jj][wc * 32 + nt * 16][0] + frag_off);
#pragma unroll
            for (int d = 0; d < DW; d++) af[1][d] = *reinterpret_cast<const v4i*>(&A_cur[d][wm * 32 + 16][0] + frag_off);
#pragma unroll
            for (int mt = 0; mt < 2; mt++)
#pragma unroll
                for (int nt = 0; nt < 2; nt++) {
#pragma unroll
                    for (int jj = 0; jj < DC; jj++)
#pragma unroll
                        for (int d = 0; d < DW; d++)
                            acc[d + jj][mt][nt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(af[mt][d], bf[nt][jj], acc[d + jj][mt][nt], 0, 0, 0);
                    // the refill of slot W (read one step ago, released by the barrier that ended that step) goes out behind the operand
                    // reads and the first quarter of the MFMAs, so that the matrix pipe starts as early as possible in a step; the loads
                    // are opaque assembly, the compiler adds no wait for them
                    if (mt == 0 && nt == 0) issue(im2 < 0 ? 0 : ks2, im2 < 0 ? 0 : im2, A_nxt, B_nxt);
                }
        }
        // the loads for step s+1 must have landed: with three slots those were issued one step ago and the ones just issued may
        // stay in flight; with two slots they are the ones just issued
        if (RING == 3) __builtin_amdgcn_s_waitcnt(0x0F70 | (A_PER_WAVE + B_PER_WAVE));      // vmcnt(loads of one step)
        else __builtin_amdgcn_s_waitcnt(0x0F70);                                            // vmcnt(0)
        __syncthreads();
        advance(ks2, im2);
    };

    // r_last (residues modulo the last prime, < 2^39) of this lane's 16 outputs, kept in registers for the fused rescale
    // of the other primes: low words, and the 7 high bits packed four to a word.
    unsigned rl_lo[2][4][2], rl_hi[2][2];
    double rl_wide[WIDE ? 2 : 1][WIDE ? 2 : 1][WIDE ? 4 : 1];           // the wide form keeps r_last as doubles
    // constants of the prime in work, requested before its K loop so that the epilogue does not start with a round trip to memory
    double q = 0, qinv = 0, c32 = 0, c64 = 0, qli = 0;
    auto epilogue = [&](int im, auto last_c, auto full_c) {
        constexpr bool LAST = decltype(last_c)::value, FULL = decltype(full_c)::value;
        // The output addressing starts from a value the optimiser cannot hoist above the K loop (it would otherwise keep
        // the row pointers alive across the loop).
        long row_stride = (long)a.mod_num * a.C;
        asm volatile("" : "+s"(row_stride));
        // (so do the row numbers: formed ahead of the loop over the primes, their 64-bit forms would be kept, or spilled to memory
        // and fetched back one by one, across the K loops)
        int mrow = m0 + wm * 32 + 4 * lg;
        asm volatile("" : "+v"(mrow));
        u64* obase = a.out + (long)im * a.C + c0 + wc * 32 + lr;
#pragma unroll
        for (int mt = 0; mt < 2; mt++) {
            // rows of the M padding are clamped for addressing; their stores are skipped
            u64* orow[4];
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const int row = mrow + mt * 16 + r;
                orow[r] = obase + (long)(FULL || row < a.M ? row : a.M - 1) * row_stride;
            }
#pragma unroll
            for (int nt = 0; nt < 2; nt++) {
                if constexpr (WIDE) {
                    // q < 2^50.  Groups of four diagonals y0 (e < 4), y1 (4 <= e < 8), y2 (e >= 8), each exact below 2^53; y0 and y1
                    // are first brought to (-q/2, q/2] so that the products with 2^32 and 2^64 mod q stay below 2^99 (quotients below
                    // 2^49: the estimate rint(h / q) is off by less than one) and every sum below stays an integer under 2^53.
                    double y0[4], y1[4], y2[4], t[4];
                    constexpr int E1 = ND - 1 < 7 ? ND - 1 : 7;
#pragma unroll
                    for (int r = 0; r < 4; r++) { y0[r] = (double)acc[3][mt][nt][r]; y1[r] = (double)acc[E1][mt][nt][r]; y2[r] = ND > 8 ? (double)acc[ND - 1][mt][nt][r] : 0.0; }
#pragma unroll
                    for (int e = 2; e >= 0; e--)
#pragma unroll
                        for (int r = 0; r < 4; r++) y0[r] = __builtin_fma(y0[r], 256.0, (double)acc[e][mt][nt][r]);
#pragma unroll
                    for (int e = E1 - 1; e >= 4; e--)
#pragma unroll
                        for (int r = 0; r < 4; r++) y1[r] = __builtin_fma(y1[r], 256.0, (double)acc[e][mt][nt][r]);
#pragma unroll
                    for (int e = ND - 2; e >= 8; e--)
#pragma unroll
                        for (int r = 0; r < 4; r++) y2[r] = __builtin_fma(y2[r], 256.0, (double)acc[e][mt][nt][r]);
#pragma unroll
                    for (int r = 0; r < 4; r++) y0[r] = balance_f64(y0[r], q, qinv);
#pragma unroll
                    for (int r = 0; r < 4; r++) y1[r] = balance_f64(y1[r], q, qinv);
#pragma unroll
                    for (int r = 0; r < 4; r++) y1[r] = mulmod_f64(y1[r], c32, q, qinv);
#pragma unroll
                    for (int r = 0; r < 4; r++) y2[r] = mulmod_f64(y2[r], c64, q, qinv);
#pragma unroll
                    for (int r = 0; r < 4; r++) t[r] = balance_f64(y0[r] + y1[r] + y2[r], q, qinv);
                    if (!LAST) {
#pragma unroll
                        for (int r = 0; r < 4; r++) t[r] = balance_f64(mulmod_f64(t[r] - rl_wide[WIDE ? mt : 0][WIDE ? nt : 0][WIDE ? r : 0], qli, q, qinv), q, qinv);
                    }
#pragma unroll
                    for (int r = 0; r < 4; r++) {
                        const double res = t[r] < 0.0 ? t[r] + q : t[r];
                        if (LAST) rl_wide[WIDE ? mt : 0][WIDE ? nt : 0][WIDE ? r : 0] = res;
                        const u64 ures = f64_bits(res + 4503599627370496.0) & 0xFFFFFFFFFFFFFull;
                        if (LAST && !store_last) {}                           // a tail job other than the first: the residues are only needed in registers
                        else if (FULL) orow[r][nt * 16] = ures;
                        else if (mrow + mt * 16 + r < a.M) orow[r][nt * 16] = ures;
                    }
                    continue;
                }
                // The four outputs of a lane in one MFMA tile advance together, one operation at a time: every operation below is
                // a chain link of one output, and four independent links in flight hide the FP64 pipeline latency.
                // Horner inside each group of four diagonals: y_g = sum_{i<4} 256^i S_{4g+i}; |S_e| <= DW * Kpad * 2^14 and the
                // launcher admits DW * Kpad <= 2^14 only, so |S_e| <= 2^28, |y_g| < 2^53 and every step is exact (ppmm_recombine in
                // f64_exact.hpp is this sequence for one output; a host build checks its ranges)
                double y0[4], y1[4], t[4];
#pragma unroll
                for (int r = 0; r < 4; r++) { y0[r] = (double)acc[3][mt][nt][r]; y1[r] = (double)acc[ND - 1][mt][nt][r]; }
#pragma unroll
                for (int e = 2; e >= 0; e--)
#pragma unroll
                    for (int r = 0; r < 4; r++) y0[r] = __builtin_fma(y0[r], 256.0, (double)acc[e][mt][nt][r]);
#pragma unroll
                for (int e = ND - 2; e >= 4; e--)
#pragma unroll
                    for (int r = 0; r < 4; r++) y1[r] = __builtin_fma(y1[r], 256.0, (double)acc[e][mt][nt][r]);
                // |y0 + (y1 * 2^32 mod q)| < 2^53 + 0.51 q: one exact addition, one reduction to (-0.51 q, 0.51 q)
                {
                    double h[4], l[4], c[4];
#pragma unroll
                    for (int r = 0; r < 4; r++) h[r] = y1[r] * c32;
#pragma unroll
                    for (int r = 0; r < 4; r++) l[r] = __builtin_fma(y1[r], c32, -h[r]);
#pragma unroll
                    for (int r = 0; r < 4; r++) c[r] = __builtin_rint(h[r] * qinv);
#pragma unroll
                    for (int r = 0; r < 4; r++) t[r] = y0[r] + (__builtin_fma(-c[r], q, h[r]) + l[r]);
#pragma unroll
                    for (int r = 0; r < 4; r++) c[r] = __builtin_rint(t[r] * qinv);
#pragma unroll
                    for (int r = 0; r < 4; r++) t[r] = __builtin_fma(-c[r], q, t[r]);
                }
                if (!LAST) {
                    // (r_i + q_i - r_last) * q_last^-1 mod q_i ; r_last is used as an integer without reduction modulo q_i, as in
                    // PPMM_kernel.cuh:243-247
                    double h[4], l[4], c[4];
#pragma unroll
                    for (int r = 0; r < 4; r++) {
                        // read through values the optimiser cannot see through: the conversions are the same for every prime but
                        // the last, and hoisted out of the loop over the primes they would occupy 32 registers across the K loops
                        unsigned lo = rl_lo[mt][r][nt], hw = rl_hi[mt][nt];
                        asm volatile("" : "+v"(lo), "+v"(hw));
                        const unsigned hi = (hw >> (8 * r)) & 0xff;
                        t[r] -= __builtin_fma((double)hi, 4294967296.0, (double)lo);
                    }
#pragma unroll
                    for (int r = 0; r < 4; r++) h[r] = t[r] * qli;
#pragma unroll
                    for (int r = 0; r < 4; r++) l[r] = __builtin_fma(t[r], qli, -h[r]);
#pragma unroll
                    for (int r = 0; r < 4; r++) c[r] = __builtin_rint(h[r] * qinv);
#pragma unroll
                    for (int r = 0; r < 4; r++) t[r] = __builtin_fma(-c[r], q, h[r]) + l[r];
                }
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const double res = t[r] < 0.0 ? t[r] + q : t[r];
                    // res is an integer in [0, q): adding 2^52 leaves it in the low mantissa bits
                    const u64 ures = f64_bits(res + 4503599627370496.0) & 0xFFFFFFFFFFull;
                    if (LAST) {
                        rl_lo[mt][r][nt] = (unsigned)ures;
                        rl_hi[mt][nt] = (r == 0 ? 0u : rl_hi[mt][nt]) | ((unsigned)(ures >> 32) << (8 * r));
                    }
                    if (LAST && !store_last) {}
                    else if (FULL) orow[r][nt * 16] = ures;
                    else if (mrow + mt * 16 + r < a.M) orow[r][nt * 16] = ures;
                }
            }
        }
    };

    for (int it = 0; it < n_iters; it++) {
        const int im = prime_of(it);
        q = a.pq[a.np + im].qd;
        qinv = a.pq[a.np + im].qinv_d;
        c32 = f64_from_bits(a.consts[2 * PPMM_MAX_MODS + im]);   // 2^32 mod q (balanced)
        if (WIDE) c64 = f64_from_bits(a.consts[3 * PPMM_MAX_MODS + im]);   // 2^64 mod q (balanced)
        qli = f64_from_bits(a.consts[4 * PPMM_MAX_MODS + im]);   // q_last^-1 mod q
#pragma unroll
        for (int e = 0; e < ND; e++)
#pragma unroll
            for (int mt = 0; mt < 2; mt++)
#pragma unroll
                for (int nt = 0; nt < 2; nt++) acc[e][mt][nt] = v4i{0, 0, 0, 0};

        for (int ks = 0; ks < ksteps; ks += RING) {
            kstep(std::integral_constant<int, 0>{});
            kstep(std::integral_constant<int, 1>{});
            if constexpr (RING == 3) kstep(std::integral_constant<int, 2>{});
        }

        // ---- end of a prime: exact recombination, reduction mod q, fused rescale ----
        // Straight-line code (the prime-position and M-padding cases are resolved once, outside the unrolled loops) so that
        // the independent output chains of a lane can be interleaved.
        const bool last = a.raw_all || im == a.mod_num - 1, full = m0 + MT <= a.M;
        if (last) { if (full) epilogue(im, std::true_type{}, std::true_type{}); else epilogue(im, std::true_type{}, std::false_type{}); }
        else      { if (full) epilogue(im, std::false_type{}, std::true_type{}); else epilogue(im, std::false_type{}, std::false_type{}); }
    }
}

size_t ppmm_bdig_bytes(const PpmmArgs& a, int DC) { return (size_t)a.mod_num * a.Kpad * a.C * (DC <= 5 ? 5 : 7); }

template <int DW, int DC>
static int launch_dw(hipStream_t stream, const PpmmArgs& a, int8_t* bdig, bool pack) {
    const int c_tiles = (int)(a.C / CT);
    if (pack) hipLaunchKernelGGL(ppmm_pack_kernel<DC>, dim3(c_tiles, a.Kpad / KS, a.mod_num), dim3(256), 0, stream, a, bdig);
    const int m_tiles = a.Mpad / 128;
    // row tiles per patch: the largest divisor of m_tiles up to 8.  An XCD's 32 workgroups then form 8 x 4 tiles at M = 4096: every
    // residue slab serves eight of them, and the plaintext slabs, which eight row tiles need more of, come from the memory-side
    // cache, which holds all of them (142 ms against 144.5 ms with patches of 4 x 8; 2 x 16: 151 ms, 16 x 2: 143.5 ms)
    int m_block = 1;
    for (int d = 2; d <= 8; d++) if (m_tiles % d == 0) m_block = d;
    unsigned blocks = (unsigned)((c_tiles + 7) / 8) * 8u * (unsigned)m_tiles;
    // The column panels beyond the last full group of eight (one per XCD) are cut into jobs by prime where that pays: a single patch
    // of row tiles (small M), enough primes to share, and the fused rescale (a job needs the last prime only then).
    const bool no_tail = a.no_tail != 0;                                       // test / tuning switch
    int main_blocks = (int)blocks, tail_jobs = 0;
    const int rest = c_tiles % 8;
    if (!no_tail && rest != 0 && c_tiles >= 8 && m_block == m_tiles && a.mod_num >= 8 && !a.raw_all) {
        tail_jobs = 4;
        main_blocks = (c_tiles / 8) * 8 * m_tiles;
        blocks = (unsigned)main_blocks + (unsigned)(rest * m_tiles * tail_jobs);
    }
    hipLaunchKernelGGL((ppmm_mfma_kernel<DW, 8, 3, DC>), dim3(blocks), dim3(512), 0, stream, a, (const int8_t*)bdig, c_tiles, m_block, main_blocks, tail_jobs);
    CKKS_HIP_TRY(hipGetLastError());
    return CKKS_OK;
}

// The pack pass on its own: the entry point starts it ahead of the host round trip that selects the contraction's instance (the
// residue planes do not depend on the plaintext matrix) and then calls the contraction with pack = false.
int launch_ppmm_pack(hipStream_t stream, const PpmmArgs& a, int DC, int8_t* bdig) {
    const dim3 grid((unsigned)(a.C / CT), (unsigned)(a.Kpad / KS), (unsigned)a.mod_num);
    if (DC <= 5) hipLaunchKernelGGL(ppmm_pack_kernel<5>, grid, dim3(256), 0, stream, a, bdig);
    else hipLaunchKernelGGL(ppmm_pack_kernel<7>, grid, dim3(256), 0, stream, a, bdig);
    CKKS_HIP_TRY(hipGetLastError());
    return CKKS_OK;
}

// pack = false: the digit planes were written by the caller (the gather that emits them directly; 5 residue digits only)
int launch_ppmm_mfma_impl(hipStream_t stream, const PpmmArgs& a, int DW, int DC, int8_t* bdig, bool pack) {
    if (DC > 5) {
        if (DW > 3) { set_error("PPMM: 7 residue digits go with at most 3 plaintext digits per launch"); return CKKS_E_INVALID; }
        return launch_dw<3, 7>(stream, a, bdig, pack);
    }
    if (DW <= 3) return launch_dw<3, 5>(stream, a, bdig, pack);
    return launch_dw<4, 5>(stream, a, bdig, pack);
}

}  // namespace ckks

// ------------------------------------------------------------------------------------------------------------
// Measured ceiling of the matrix pipe: v_mfma_i32_16x16x64_i8 from registers only, eight independent accumulators per wave
// (no LDS, no memory), two workgroups of 512 lanes per compute unit as the contraction kernel runs.  What this loop reaches is
// what the clock under matrix load allows; the contraction's fraction of it says how much of the time its matrix pipe is busy.
// ------------------------------------------------------------------------------------------------------------
namespace {
__global__ __launch_bounds__(512, 2) void mfma_i8_peak_kernel(int* sink, int iters, int seed) {
    typedef int v4i __attribute__((ext_vector_type(4)));
    v4i a = {seed + (int)threadIdx.x, seed, 1, 2}, b = {seed, 3, (int)threadIdx.x, 4};
    v4i acc[8];
#pragma unroll
    for (int i = 0; i < 8; i++) acc[i] = v4i{i, 0, 0, 0};
    for (int n = 0; n < iters; n++) {
#pragma unroll
        for (int i = 0; i < 8; i++) acc[i] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, acc[i], 0, 0, 0);
    }
    v4i s = acc[0];
#pragma unroll
    for (int i = 1; i < 8; i++) s += acc[i];
    if (s[0] + s[1] + s[2] + s[3] == 0x7fffffff) sink[0] = 1;      // never true in practice: keeps the loop alive
}
}  // namespace

// int8 MAC/s of the loop above on the current device (timed with HIP events on `stream` over `reps` launches)
extern "C" int ckks_measure_mfma_i8_peak(void* stream_v, double* macs_per_s) {
    using namespace ckks;
    if (!macs_per_s) return CKKS_E_INVALID;
    hipStream_t stream = (hipStream_t)stream_v;
    int dev = 0, cus = 0;
    CKKS_HIP_TRY(hipGetDevice(&dev));
    CKKS_HIP_TRY(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
    int* sink = nullptr;
    CKKS_HIP_TRY(hipMalloc((void**)&sink, sizeof(int)));
    hipEvent_t e0 = nullptr, e1 = nullptr;
    hipError_t e = hipEventCreate(&e0);
    if (e == hipSuccess) e = hipEventCreate(&e1);
    const int iters = 4096, reps = 5;
    const unsigned blocks = (unsigned)cus * 2u;
    float ms = 0.f;
    if (e == hipSuccess) {
        hipLaunchKernelGGL(mfma_i8_peak_kernel, dim3(blocks), dim3(512), 0, stream, sink, iters, 1);      // warm-up
        e = hipEventRecord(e0, stream);
        for (int r = 0; r < reps; r++) hipLaunchKernelGGL(mfma_i8_peak_kernel, dim3(blocks), dim3(512), 0, stream, sink, iters, r + 2);
        if (e == hipSuccess) e = hipEventRecord(e1, stream);
        if (e == hipSuccess) e = hipEventSynchronize(e1);
        if (e == hipSuccess) e = hipEventElapsedTime(&ms, e0, e1);
    }
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    (void)hipFree(sink);
    if (e != hipSuccess) return hip_fail(e, "ckks_measure_mfma_i8_peak");
    // per wave and iteration: 8 instructions of 16 x 16 x 64 multiply-accumulates
    const double macs = (double)reps * blocks * 8.0 /* waves */ * iters * 8.0 * (16.0 * 16.0 * 64.0);
    *macs_per_s = macs / (ms * 1e-3);
    return CKKS_OK;
}

