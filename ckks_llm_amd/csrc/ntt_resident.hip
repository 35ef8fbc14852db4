// Resident transform at N = 2^16: both passes of a limb in one workgroup, the limb held in registers between them.
//
// Same transform as the two launches of ntt.hip (Context_23::ToNTTInplace / FromNTTInplace, Context_23.cuh:847-930,
// ntt_60bit.cuh:421-1318), same tiles, same butterflies; what changes is where a limb is between its two passes.  The
// two-launch form writes it to memory and reads it back (26 bytes per value through HBM); here a workgroup of 512 lanes keeps
// all 65536 values of its limb in its own registers - 128 values per lane in the 5-byte form of ntt.hip's inter-pass buffer,
// 160 of the 256 registers a lane has - so HBM sees the limb once in and once out: 16 bytes per value.
//
// One persistent workgroup per compute unit (its registers and its LDS leave room for exactly one) walks through its share of
// the limbs.  The workgroup is two groups of 256 lanes; a step handles two tiles, one per group:
//   pass 1, step s: tiles 2s and 2s+1 of the first pass (forward: 16 columns x 256 rows; inverse: 16 rows x 256 columns).
//                   The tile arrives in LDS by asynchronous loads (global_load_lds) requested during the step before, every
//                   wave fetching exactly what its own lanes read, so the only synchronisation is the wave's own counter.
//                   Of its 16 results a lane keeps the 8 that its own group's tiles of pass 2 need and hands the other 8 to
//                   the same lane of the other group (through LDS, in the 5-byte form), receiving 8 of the other tile.
//   pass 2, step s: every lane decodes the 16 values it holds of tile 2s + group and runs the tile; nothing is exchanged
//                   between the groups.
// For that the 16 x 256 tiles are interleaved: tile k of the row pass is the rows 16 m + k (m = 0..15), lane group m taking
// row 16 m + k, which is exactly the set of rows (forward: that a lane of the column pass ends with; inverse: that a lane of
// the column pass starts from).
//
// One twiddle table serves both directions.  The tables hold the powers of psi in bit-reversed order; psi^-k = -psi^(N-k), and in
// that order the exponent N - k sits, within each power-of-two block of the table, at the mirrored index: inverse[j] =
// -forward[3 * 2^s - 1 - j] for 2^s <= j < 2^(s+1), the same bits (the entries are balanced residues, so the sign flips exactly).
// The inverse transform therefore reads the forward table at mirrored places - a contiguous group of twiddles stays a contiguous
// group, of the mirrored row and lane group, in reverse order - and negates what it reads (a source modifier, no instruction).
// Alternating forward and inverse launches then keep one table warm in the memory-side cache instead of displacing each other's
// (measured: a launch that follows the other direction lost 25 - 55 us of 465 us to that).
//
// Vector memory operations complete in the order of their issue and share one counter.  The asynchronous loads are issued
// from inline assembly, invisible to the compiler's own bookkeeping, so a step is written such that no load the compiler
// waits for is older than an asynchronous load still in flight: the twiddles of a step are in registers (drain()) before the
// next tile is requested.
#include <cstdlib>
#include <type_traits>

#include "context.hpp"
#include "ntt_core.hpp"

namespace ckks {

namespace {

#ifdef CKKS_RES_TIMING
__device__ unsigned long long g_res_ticks[8][136];
#define RES_TICK(n) do { if (it == 1 && blockIdx.x < 8 && threadIdx.x == 0) g_res_ticks[blockIdx.x][(n)] = __builtin_readcyclecounter(); } while (0)
#else
#define RES_TICK(n) do { } while (0)
#endif

typedef __attribute__((address_space(3))) void* lptr_t;

constexpr int RES_LANES = 512;
constexpr long RES_N = 65536;
constexpr int RES_PITCH = RowCfg<8, 8>::PITCH;                       // 272: padded row of the row pass
constexpr int RES_P_BYTES = 65536;                                   // staging of the tiles that arrive: 8 KiB per wave
constexpr int RES_R_BYTES = 2 * 16 * RES_PITCH * 8;                  // exchange area of a step: one tile per group (69632 bytes)
constexpr int RES_S_BYTES = 9 * RES_LANES * 4;                       // hand-over between the groups: 9 words per lane
constexpr int RES_T_BYTES = 8 * 1024;                                // row twiddles of a step: the first 512 bytes of 1 KiB per wave

// limb of workgroup b in round `it`: consecutive workgroups of a grid go to the eight XCDs in turn, and the workgroups of one
// XCD take consecutive limbs - limbs are ordered prime-major, so one XCD's compute units read one prime's twiddles from its L2.
__device__ __forceinline__ unsigned resident_limb(unsigned b, unsigned grid, unsigned it) {
    const unsigned per_x = grid / 8;
    return ((b % 8) + 8 * it) * per_x + b / 8;
}

// 16 bytes per lane from global memory into LDS at lds_addr + 16 * lane (lds_addr wave-uniform)
// STREAM: a load of data that is read once (the caches need not keep the line)
template <bool STREAM = false>
__device__ __forceinline__ void dma16(const void* g, unsigned lds_addr) {
    const unsigned base = __builtin_amdgcn_readfirstlane(lds_addr);
    if (STREAM) asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off nt" : : "v"(g), "s"(base) : "memory", "m0");
    else asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(g), "s"(base) : "memory", "m0");
}
// Ordering point for what a wave exchanges with itself through LDS (the hardware carries out a wave's LDS accesses in order; this
// keeps the compiler from reordering them: as one thread sees it, the lane that writes and the lane that reads are unrelated).
__device__ __forceinline__ void wave_sync() { __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront"); __builtin_amdgcn_wave_barrier(); }
#ifdef CKKS_RES_EXP_NOCOLBAR
__device__ __forceinline__ void col_sync() { wave_sync(); }
#else
__device__ __forceinline__ void col_sync() { __syncthreads(); }
#endif
#ifdef CKKS_RES_EXP_NOHANDBAR
__device__ __forceinline__ void hand_sync() { wave_sync(); }
#else
__device__ __forceinline__ void hand_sync() { __syncthreads(); }
#endif
__device__ __forceinline__ void wait_all_vmem() { asm volatile("s_waitcnt vmcnt(0)" : : : "memory"); }

// The fifteen twiddles of the last four stages of an axis (packed layout, lane group g: stage 4 + d, butterfly group k),
// fetched together ahead of their use.
template <class AR>
struct PackedTwiddles {
    typename AR::TW t[15];
    __device__ __forceinline__ void load(const typename AR::TW* __restrict__ tw, unsigned off, unsigned g) {
#pragma unroll
        for (int d = 0; d < 4; d++)
#pragma unroll
            for (int k = 0; k < (1 << d); k++) t[(1 << d) - 1 + k] = tw[(off << (4 + d)) + (g << d) + k];
    }
    // The same in eight loads - a group of 2^d twiddles is contiguous and 8 * 2^d bytes aligned, so sixteen bytes at a time from the
    // second group on - that stay in front of whatever memory access follows them in program order (the compiler would otherwise
    // sink them towards their use, behind the stores in between - and loads and stores complete in the order of their issue):
    // the first is a relaxed atomic load at wavefront scope, an ordinary load instruction that the scheduler does not move
    // across other memory accesses; behind the others stands an empty statement that may touch memory.  Against fifteen 8-byte
    // loads: 448 -> 433 us per inverse launch.
    __device__ __forceinline__ void load_ordered(const typename AR::TW* tw, unsigned off, unsigned g) {
        typedef double d2 __attribute__((ext_vector_type(2)));
        static_assert(sizeof(typename AR::TW) == 8, "pairs of twiddles are read as 16 bytes");
        t[0] = __hip_atomic_load(tw + (off << 4) + g, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WAVEFRONT);
#pragma unroll
        for (int d = 1; d < 4; d++)
#pragma unroll
            for (int k = 0; k < (1 << d); k += 2) {
                const d2 v = *reinterpret_cast<const d2*>(tw + (off << (4 + d)) + (g << d) + k);
                t[(1 << d) - 1 + k] = v.x;
                t[(1 << d) + k] = v.y;
            }
        asm volatile("" : : : "memory");
    }
    // all fifteen are in registers after this (the compiler waits for them here, where no asynchronous load is in flight)
    __device__ __forceinline__ void drain() {
        asm volatile("" : "+v"(t[0]), "+v"(t[1]), "+v"(t[2]), "+v"(t[3]), "+v"(t[4]), "+v"(t[5]), "+v"(t[6]), "+v"(t[7]));
        asm volatile("" : "+v"(t[8]), "+v"(t[9]), "+v"(t[10]), "+v"(t[11]), "+v"(t[12]), "+v"(t[13]), "+v"(t[14]));
    }
};
// Four stages on sixteen register values (the first four of an axis in the spread layout, the last four in the packed layout: the
// same butterfly pattern), the twiddles of a stage fetched while the stage before runs: fetch(s, k) gives the twiddle of the
// round's stage s, butterfly group k = j >> (4 - s).
// The fifteen twiddles of the first four stages of an axis (spread layout: stage s, butterfly group k), fetched together.
template <class AR>
struct SpreadTwiddles {
    typename AR::TW t[15];
    __device__ __forceinline__ void load(const typename AR::TW* __restrict__ tw, unsigned off) {
#pragma unroll
        for (int s = 0; s < 4; s++)
#pragma unroll
            for (int k = 0; k < (1 << s); k++) t[(1 << s) - 1 + k] = tw[(off << s) + k];
    }
};
struct NoHook { __device__ __forceinline__ void operator()(int) const {} };
// after(s) runs behind the butterflies of the round's stage s (the asynchronous loads of the next tile go out there, one per stage)
template <class AR, class F, class H = NoHook>
__device__ __forceinline__ void fwd_round(typename AR::V (&v)[16], const AR& ar, F fetch, H after = H()) {
    typename AR::TW cur[8], nxt[8];
    cur[0] = fetch(0, 0);
#pragma unroll
    for (int s = 0; s < 4; s++) {
        if (s < 3) {
#pragma unroll
            for (int k = 0; k < (2 << s); k++) nxt[k] = fetch(s + 1, k);
        }
        const int half = 8 >> s;
#pragma unroll
        for (int j = 0; j < 16; j++)
            if ((j & half) == 0) ar.ct(v[j], v[j + half], cur[j >> (4 - s)]);
        after(s);
        if (s < 3) {
#pragma unroll
            for (int k = 0; k < (2 << s); k++) cur[k] = nxt[k];
        }
    }
}
template <class AR, int S_STOP, class F, class H = NoHook>
__device__ __forceinline__ void inv_round(typename AR::V (&v)[16], const AR& ar, F fetch, H after = H()) {                          // the round's stages 3 .. S_STOP
    typename AR::TW cur[8], nxt[8];
#pragma unroll
    for (int k = 0; k < 8; k++) cur[k] = fetch(3, k);
#pragma unroll
    for (int s = 3; s >= S_STOP; s--) {
        if (s > S_STOP) {
#pragma unroll
            for (int k = 0; k < (1 << (s - 1)); k++) nxt[k] = fetch(s - 1, k);
        }
        const int half = 8 >> s;
#pragma unroll
        for (int j = 0; j < 16; j++)
            if ((j & half) == 0) ar.gs(v[j], v[j + half], cur[j >> (4 - s)]);
        after(s);
        if (s > S_STOP) {
#pragma unroll
            for (int k = 0; k < (1 << (s - 1)); k++) cur[k] = nxt[k];
        }
    }
}

// The low words of the limb live in the accumulation registers, which only these two moves reach: the register allocator has
// the other half of the lane's registers for a step's working set and cannot be tempted to spill the limb to memory.
__device__ __forceinline__ unsigned to_acc(unsigned x) {
    unsigned a;
    asm volatile("v_accvgpr_write_b32 %0, %1" : "=a"(a) : "v"(x));
    return a;
}
__device__ __forceinline__ unsigned from_acc(unsigned a) {
    unsigned x;
    asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(x) : "a"(a) : "memory");      // "memory": stays behind the barrier in front of its step
    return x;
}

// What a lane keeps of its limb between the passes: per step of pass 1 and per tile of that step, eight 5-byte values
// (low words, and the high bytes four to a register).
struct Stash {
    unsigned lo[8][2][8];
    unsigned hi[8][2];
};

template <bool INVERSE>
__global__ __launch_bounds__(RES_LANES) void ntt_resident_kernel(NttArgs a, unsigned limbs, unsigned backwards) {
    typedef F64Arith AR;
    typedef double V;
    typedef double TW;
    __shared__ __align__(16) unsigned char lds_p[RES_P_BYTES];
    __shared__ __align__(16) unsigned char lds_r[RES_R_BYTES];
    __shared__ __align__(16) unsigned lds_s[RES_S_BYTES / 4];
    __shared__ __align__(16) unsigned char lds_t[RES_T_BYTES];
    __shared__ __align__(16) TW lds_w[256];              // entries 0 .. 255 of the prime's table: twiddles 1 .. 255 are the column pass's, the same for every column
    unsigned grp = threadIdx.x >> 8;
    unsigned tid = threadIdx.x & 255, cl = tid & 15, g = tid >> 4;    // column pass: column within the tile, group of rows; row pass: lane within the row (u = cl), row group (rl = g)
    unsigned wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), wq = wave & 3;
    unsigned lane = threadIdx.x & 63;
    // this wave's part of the staging area, and where this lane reads its sixteen words from (word j at + 512 j)
    unsigned p_wave = (unsigned)(size_t)(lptr_t)lds_p + wave * 8192;
    const u64* p_lane;
    // asynchronous load m (0..7) of a tile moves 1 KiB: words 2m and 2m+1 of every lane of the wave
    unsigned d_chunk, d_i, d_jl;
    V* col_area;                                         // column pass: [row][16 columns]
    V* row_area;                                         // row pass: this lane's row
    Stash st;
    // The lane's coordinates and LDS addresses are formed anew in every step from a value the compiler cannot see through:
    // shared across the 32 unrolled steps they would sit in registers for the whole limb, and the 160 registers of the
    // limb leave no room for that.
    auto coordinates = [&]() __attribute__((always_inline)) {
        unsigned x = threadIdx.x;
        asm volatile("" : "+v"(x));
        // (the wave's number too: the scalar registers are as short as the vector ones, and the addresses that hang on it - staging
        // areas, LDS bases of the asynchronous loads - would otherwise all be formed ahead of the limb and kept)
        asm volatile("" : "+s"(wave));
        wq = wave & 3;
        p_wave = (unsigned)(size_t)(lptr_t)lds_p + wave * 8192;
        grp = x >> 8; tid = x & 255; cl = x & 15; g = tid >> 4; lane = x & 63;
        d_chunk = lane & 7; d_i = (lane >> 3) & 3; d_jl = lane >> 5;
        p_lane = reinterpret_cast<const u64*>(lds_p + wave * 8192 + lane * 8);
        col_area = reinterpret_cast<V*>(lds_r) + grp * 4096;
        row_area = reinterpret_cast<V*>(lds_r) + grp * (16 * RES_PITCH) + g * RES_PITCH;
    };
    coordinates();

    // The kernel's own code, fetched as data.  The code (about 100 KiB, unrolled over the 32 steps of a limb) exceeds the instruction
    // cache, so instruction fetch leans on the L2; a launch that follows a different kernel finds none of its code there and would
    // fetch it line by line, in execution order, from memory - with two waves per SIMD nothing hides that (measured: 20 us of 465 for a
    // launch that follows a copy of itself under another name).  Here every lane reads one word per 128-byte line of the stretch of
    // code between this point and the label in front of the kernel's end, all lines at once: one memory latency, and the
    // instruction fetches that follow hit the L2.  Both labels lie inside this function, so every address between them is this
    // function's code.
    {
        int code_bytes;
        if constexpr (INVERSE) asm volatile("ckks_res_inv_code_begin:\n\ts_mov_b32 %0, ckks_res_inv_code_end-ckks_res_inv_code_begin" : "=s"(code_bytes));
        else asm volatile("ckks_res_fwd_code_begin:\n\ts_mov_b32 %0, ckks_res_fwd_code_end-ckks_res_fwd_code_begin" : "=s"(code_bytes));
        const char* pc = reinterpret_cast<const char*>(__builtin_amdgcn_s_getpc());
        code_bytes -= 1024;                              // the program counter was read a few instructions behind the first label
        if (code_bytes > 0 && code_bytes < (1 << 18)) {
            unsigned seen = 0;
            for (int at = (int)threadIdx.x * 128; at < code_bytes; at += RES_LANES * 128)
                seen |= __hip_atomic_load(reinterpret_cast<const unsigned*>(pc + at), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);      // served by the L2
            asm volatile("" : : "v"(seen));
        }
    }

    // Requests tile (2 s + grp) of the first pass of `limb`.  Inverse transforms: with it the twiddles of the tile's last four
    // stages, which depend on the row only: 15 per row = 8 chunks of 16 bytes (stage 3: 4, stage 2: 2, stage 1: 1, stage 0: the
    // chunk that holds its one twiddle), 4 rows per wave, into this wave's 512 bytes of the twiddle staging of the step's parity.
    // part m (0..7: 1 KiB of the tile; 8: the row twiddles) of the request; part 0 first
    auto request_part = [&](const u64* limb, const TW* tw, int s, int m) __attribute__((always_inline)) {
        const unsigned tile = 2 * s + grp;
        if (m == 0) asm volatile("s_waitcnt lgkmcnt(0)" : : : "memory");       // this wave has read everything it wanted from its staging area
        if (m < 8) {
            const u64* src;
            if (!INVERSE) src = limb + (long)(4 * wq + d_i + 16 * (2 * m + d_jl)) * 256 + tile * 16 + 2 * d_chunk;      // rows g + 16 j of 16 columns
            else src = limb + (long)(16 * (4 * wq + d_i) + tile) * 256 + 16 * (2 * m + d_jl) + 2 * d_chunk;             // columns u + 16 j of row 16 rl + tile
            // the rows of an inverse transform's tile are read as streaming loads (434 -> 427 us per launch); for the columns of a forward
            // transform's tile, 128 bytes per row, the same costs 37 us per launch
            dma16<INVERSE>(src, p_wave + m * 1024);
        } else {
            // the lower half of the wave fetches the 512 bytes (the upper half would only repeat them into the second half of the
            // wave's 1 KiB, which nobody reads: 433 -> 428 us per inverse launch without); the staging is single: the step's own
            // reads of it are over (they come before this in the last round)
            const unsigned i = (lane >> 3) & 3, c = lane & 7;
            const unsigned trow_id = 16 * (4 * wq + i) + tile;
            const unsigned off = 256 + (INVERSE ? 255 - trow_id : trow_id);          // inverse: the mirrored row of the forward table
            // chunk c: 0..3 stage 3 (twiddles 8 off + 2 c ..), 4..5 stage 2 (4 off + 2 (c - 4) ..), 6 stage 1 (2 off ..), 7 the pair that holds stage 0's (off)
            const unsigned sh = (0x01223333u >> (4 * c)) & 15u, add = (0x00206420u >> (4 * c)) & 15u;
            const TW* src = tw + (((off << sh) + add) & ~1u);
            asm volatile("s_waitcnt lgkmcnt(0)" : : : "memory");
            if (lane < 32) dma16(src, (unsigned)(size_t)(lptr_t)lds_t + wave * 1024);
        }
    };
    auto request = [&](const u64* limb, const TW* tw, int s) __attribute__((always_inline)) {
#pragma unroll
        for (int m = 0; m < (INVERSE ? 9 : 8); m++) request_part(limb, tw, s, m);
    };
    // end of a pass-1 step: v[j] (forward: row 16 g + j of the group's column tile; inverse: column tile j of the group's row) ->
    // keep the eight values of the parity of this group, hand the other eight to the partner lane, take its eight
    auto hand_over = [&](const V (&v)[16], const AR& ar, int s) __attribute__((always_inline)) {
        unsigned klo[8], khi = 0, shi = 0;
        // Inverse transforms have no other barrier in a step of pass 1: this one says that the partner has taken what the step
        // before handed over (the waves are about to meet at the next barrier anyway).
        if (INVERSE) hand_sync();
#pragma unroll
        for (int jj = 0; jj < 8; jj++) {
            const V keep = grp ? v[2 * jj + 1] : v[2 * jj], send = grp ? v[2 * jj] : v[2 * jj + 1];
            const u64 ek = ar.enc36(keep), es = ar.enc36(send);
            klo[jj] = (unsigned)ek;
            lds_s[(jj * 2 + grp) * 256 + tid] = (unsigned)es;
            khi |= (unsigned)(ek >> 32) << (4 * jj);
            shi |= (unsigned)(es >> 32) << (4 * jj);
        }
        lds_s[(8 * 2 + grp) * 256 + tid] = shi;
        hand_sync();
#pragma unroll
        for (int jj = 0; jj < 8; jj++) {
            const unsigned r = lds_s[(jj * 2 + (1 - grp)) * 256 + tid];
            st.lo[s][0][jj] = to_acc(grp ? r : klo[jj]);
            st.lo[s][1][jj] = to_acc(grp ? klo[jj] : r);
        }
        const unsigned r = lds_s[(8 * 2 + (1 - grp)) * 256 + tid];
        unsigned h0 = grp ? r : khi, h1 = grp ? khi : r;
        asm volatile("" : "+v"(h0), "+v"(h1));          // formed here, not left in pieces until pass 2 asks for them
        st.hi[s][0] = h0;
        st.hi[s][1] = h1;
    };
    // start of a pass-2 step: the sixteen values this lane holds of tile 2 s + grp
    auto take = [&](V (&v)[16], const AR& ar, int s) __attribute__((always_inline)) {
#pragma unroll
        for (int j = 0; j < 16; j++) {
            // the nibble is cut out here and not ahead of time: seen through, the shifts of all eight steps would be formed where
            // the word is made, and their results kept for the whole limb
            unsigned h = st.hi[j >> 1][j & 1];
            asm volatile("" : "+v"(h) : : "memory");
            v[j] = ar.dec36(from_acc(st.lo[j >> 1][j & 1][s]), (h >> (4 * s)) & 0xfu);
        }
    };

    // Rounds of this workgroup (its limbs lie `gridDim.x` apart, so they are the rounds 0 .. rounds - 1), walked upwards or
    // downwards: a launch that starts where the launch before it ended finds the last-written limbs in the memory-side cache.
    const unsigned first_id = resident_limb(blockIdx.x, gridDim.x, 0);
    if (first_id >= limbs) return;
    const unsigned rounds = (limbs - first_id + gridDim.x - 1) / gridDim.x;
    auto round_limb = [&](unsigned i) { return resident_limb(blockIdx.x, gridDim.x, backwards ? rounds - 1 - i : i); };
    unsigned it = 0;
    unsigned limb_id = round_limb(0);
    int prime;
    u64* limb = limb_ptr(a, limb_id, RES_N, prime);
#ifdef CKKS_RES_EXP_STAGGER
    if ((blockIdx.x >> 3) & 1) { for (int z = 0; z < CKKS_RES_EXP_STAGGER; z++) __builtin_amdgcn_s_sleep(127); }
#endif
    request(limb, (const TW*)a.tw + (long)prime * RES_N, 0);
    PackedTwiddles<AR> wp;                               // second-round twiddles of a row-pass step, fetched a step ahead
    // The first 2 KiB of a prime's table go to lds_w by the same asynchronous loads as the tiles (waves 0 and 1, 1 KiB each), at a
    // point where no wave reads lds_w any more and with a vmcnt(0) of every wave and a barrier between them and the first read.
    auto request_col_twiddles = [&](const TW* t) __attribute__((always_inline)) {
        if (wave < 2) dma16(t + (wave * 64 + lane) * 2, (unsigned)(size_t)(lptr_t)lds_w + wave * 1024);
    };
    if (!INVERSE) request_col_twiddles((const TW*)a.tw + (long)prime * RES_N);
    if (INVERSE) wp.load_ordered((const TW*)a.tw + (long)prime * RES_N, 511 - (16 * g + grp), 15 - cl);
    for (;;) {
        const AR ar(a.primes[prime]);
        const TW* __restrict__ tw = (const TW*)a.tw + (long)prime * RES_N;
        const bool more = it + 1 < rounds;
        const unsigned next_id = more ? round_limb(it + 1) : limb_id;
        int next_prime = prime;
        u64* next_limb = more ? limb_ptr(a, next_id, RES_N, next_prime) : limb;
        const TW* next_tw = (const TW*)a.tw + (long)next_prime * RES_N;

        if (!INVERSE) {
            // ---------------- pass 1: columns (first eight stages) ----------------
#pragma unroll
            for (int s = 0; s < 8; s++) {
                coordinates();
                RES_TICK(8 * s);
                wait_all_vmem();                        // this wave's part of the tile has arrived
                RES_TICK(8 * s + 1);
                V v[16];
#pragma unroll
                for (int j = 0; j < 16; j++) v[j] = ar.from_canonical(p_lane[j * 64]);
                // the same twiddles for every lane: scalar loads; behind each stage one eighth of the next tile is requested
                fwd_round(v, ar, [&](int d, int k) { return tw[(1u << d) + k]; }, [&](int d) { if (s < 7) request_part(limb, tw, s + 1, d); });
#pragma unroll
                for (int j = 0; j < 16; j++) col_area[(g + 16 * j) * 16 + cl] = v[j];
                RES_TICK(8 * s + 5);
                col_sync();
#pragma unroll
                for (int j = 0; j < 16; j++) v[j] = col_area[(g * 16 + j) * 16 + cl];
                if (s == 7) {                           // for the first step of pass 2: its row twiddles, both rounds
                    wp.load_ordered(tw, 256 + 16 * g + grp, cl);
                    request_part(limb, tw, 0, 8);
                }
                fwd_round(v, ar, [&](int d, int k) { return lds_w[(16u << d) + (g << d) + k]; }, [&](int d) { if (s < 7) request_part(limb, tw, s + 1, 4 + d); });
                RES_TICK(8 * s + 6);
                hand_over(v, ar, s);
            }
            // ---------------- pass 2: rows (last eight stages), tile k = rows 16 m + k ----------------
            // Loads and stores complete in the order of their issue, so a load issued behind a step's stores would be waited for
            // until those stores are done.  Both sets of twiddles of a step are therefore requested before the stores of the step
            // before: the fifteen of the first round (the same for the sixteen lanes of a row) into the wave's twiddle staging, the
            // fifteen of the second round into registers.
            // No barrier in this pass: the sixteen lanes of a row are in one wave, so what a wave exchanges through the row area it
            // exchanges with itself, and a wave's LDS accesses are carried out in order.
#pragma unroll
            for (int s = 0; s < 8; s++) {
                coordinates();
                const unsigned row = 16 * g + 2 * s + grp;
                const unsigned tw_off = 256 + row;
                // the staging has arrived: everything but the eight stores behind it is complete
                RES_TICK(64 + 8 * s);
                if (s == 0) asm volatile("s_waitcnt vmcnt(0)" : : : "memory");
                else asm volatile("s_waitcnt vmcnt(8)" : : : "memory");
                RES_TICK(64 + 8 * s + 1);
                const TW* trow = reinterpret_cast<const TW*>(lds_t + wave * 1024 + (lane >> 4) * 128);
                V v[16];
                take(v, ar, s);
                RES_TICK(64 + 8 * s + 2);
                fwd_round(v, ar, [&](int d, int k) { return d == 3 ? trow[k] : d == 2 ? trow[8 + k] : d == 1 ? trow[12 + k] : trow[14 + (tw_off & 1u)]; });
                RES_TICK(64 + 8 * s + 3);
                RES_TICK(64 + 8 * s + 4);
                wave_sync();
#pragma unroll
                for (int j = 0; j < 16; j++) row_area[padded(cl + 16 * j)] = v[j];
                if (s == 7 && more) wp.drain();         // no load of the compiler's is pending when the next limb's tile is requested
                wave_sync();
                RES_TICK(64 + 8 * s + 5);
#pragma unroll
                for (int j = 0; j < 16; j++) v[j] = row_area[padded(cl * 16 + j)];
                fwd_round(v, ar, [&](int d, int k) { return wp.t[(1 << d) - 1 + k]; },
                          [&](int d) { if (s == 7 && more) { request_part(next_limb, next_tw, 0, 2 * d); request_part(next_limb, next_tw, 0, 2 * d + 1); } });
                RES_TICK(64 + 8 * s + 6);
#pragma unroll
                for (int j = 0; j < 16; j++) row_area[padded(cl * 16 + j)] = v[j];
                wave_sync();
                RES_TICK(64 + 8 * s + 7);
                if (s == 6 && more) request_col_twiddles(next_tw);      // the next limb's: nobody has read lds_w since the first pass ended
                if (s < 7) {
                    wp.load_ordered(tw, tw_off + 2, cl);
                    request_part(limb, tw, s + 1, 8);
                }
                // Sixteen bytes per store: the lane takes words 2 cl, 2 cl + 1 (+ 32 j) of its row from the row area instead of the words
                // cl + 16 j that the pass leaves it with - half as many store instructions in the queue that the tile loads share
                // (435 -> 431 us per launch).
                // (streaming stores: the results are not read again in this launch, and lines that linger in the caches as written
                // data cost the loads of this launch and of the next more than the next launch's hits on them would save:
                // 437 -> 417 us per forward launch, 453 -> 434 us per inverse launch, 474 -> 433 us for an inverse that follows a forward)
                typedef u64 u64x2 __attribute__((ext_vector_type(2)));
                u64x2* rp = reinterpret_cast<u64x2*>(limb + (long)row * 256 + 2 * cl);
#pragma unroll
                for (int j = 0; j < 8; j++) {
                    u64x2 o;
                    o.x = ar.to_canonical_fwd(row_area[padded(2 * cl + 32 * j)]);
                    o.y = ar.to_canonical_fwd(row_area[padded(2 * cl + 1 + 32 * j)]);
#ifdef CKKS_RES_EXP_NOSTORE
                    if (o.x == 0x123456789abcull) rp[16 * j] = o;
#else
                    __builtin_nontemporal_store(o, &rp[16 * j]);
#endif
                }
            }
        } else {
            // ---------------- pass 1: rows (stages 15 .. 8), tile k = rows 16 m + k ----------------
            // the row area is exchanged within a wave (the sixteen lanes of a row): no barrier but the hand-over's
#pragma unroll
            for (int s = 0; s < 8; s++) {
                coordinates();
                const unsigned row = 16 * g + 2 * s + grp;
                const unsigned tw_off = 256 + row;
                wait_all_vmem();                        // this wave's part of the tile, its row twiddles and the lane's twiddles have arrived
                if (s == 0) request_col_twiddles(tw);   // for the second pass: the workgroup has left the last limb's second pass behind
#pragma unroll
                for (int j = 0; j < 16; j++) row_area[padded(cl + 16 * j)] = ar.from_canonical(p_lane[j * 64]);
                const TW* trow = reinterpret_cast<const TW*>(lds_t + wave * 1024 + (lane >> 4) * 128);
                wave_sync();
                V v[16];
#pragma unroll
                for (int j = 0; j < 16; j++) v[j] = row_area[padded(cl * 16 + j)];
                // (mirrored groups: twiddle k of stage d is the negative of entry 2^d - 1 - k of the group that was fetched)
                inv_round<AR, 0>(v, ar, [&](int d, int k) { return -wp.t[(2 << d) - 2 - k]; }, [&](int d) { if (s < 7) request_part(limb, tw, s + 1, 3 - d); });
#pragma unroll
                for (int j = 0; j < 16; j++) row_area[padded(cl * 16 + j)] = v[j];
                wave_sync();
#pragma unroll
                for (int j = 0; j < 16; j++) v[j] = row_area[padded(cl + 16 * j)];
                inv_round<AR, 0>(v, ar, [&](int d, int k) { return d == 3 ? -trow[7 - k] : d == 2 ? -trow[11 - k] : d == 1 ? -trow[13 - k] : -trow[15 - (tw_off & 1u)]; },
                                 [&](int d) { if (s < 7) { request_part(limb, tw, s + 1, 7 - d); if (d == 0) request_part(limb, tw, s + 1, 8); } });
                if (s < 7) wp.load_ordered(tw, 511 - (row + 2), 15 - cl);         // the next step's, behind the requests: they arrive together
                hand_over(v, ar, s);                    // balanced to (-q/2, q/2] between the passes, as in the two-launch form
            }
            __syncthreads();                            // (every wave has waited for its loads since the column twiddles were requested)
            // ---------------- pass 2: columns (stages 7 .. 0) ----------------
#pragma unroll
            for (int s = 0; s < 8; s++) {
                coordinates();
                V v[16];
                take(v, ar, s);
                // (mirrored within the power-of-two block, negated: the table in lds_w is the forward one)
                inv_round<AR, 0>(v, ar, [&](int d, int k) { return -lds_w[(16u << d) + ((15u - g) << d) + ((1u << d) - 1u - k)]; });
                col_sync();                             // the exchange area is free
#pragma unroll
                for (int j = 0; j < 16; j++) col_area[(g * 16 + j) * 16 + cl] = v[j];
                col_sync();
#pragma unroll
                for (int j = 0; j < 16; j++) v[j] = col_area[(g + 16 * j) * 16 + cl];
                inv_round<AR, 1>(v, ar, [&](int d, int k) { return -tw[(2u << d) - 1 - k]; },        // scalar loads, mirrored
                                 [&](int d) { if (s == 7 && more) { request_part(next_limb, next_tw, 0, 9 - 3 * d); request_part(next_limb, next_tw, 0, 10 - 3 * d); request_part(next_limb, next_tw, 0, 11 - 3 * d); } });
                if (s == 7 && more) wp.load_ordered(next_tw, 511 - (16 * g + grp), 15 - cl);
                u64* col = limb + (2 * s + grp) * 16 + cl;
#pragma unroll
                for (int j = 0; j < 8; j++) {
                    u64 ox, oy;
                    ar.gs_last(v[j], v[j + 8], ox, oy);
                    __builtin_nontemporal_store(ox, &col[(long)(g + 16 * j) * 256]);          // streaming stores, as in the forward direction
                    __builtin_nontemporal_store(oy, &col[(long)(g + 16 * (j + 8)) * 256]);
                }
            }
        }
        RES_TICK(128);
        if (!more) break;
        __syncthreads();                                // the exchange area is free for the next limb's first step
        it++;
        limb = next_limb;
        prime = next_prime;
    }
    // end of the stretch of code that the kernel's first instructions fetch as data
    if constexpr (INVERSE) asm volatile("ckks_res_inv_code_end:");
    else asm volatile("ckks_res_fwd_code_end:");
}

}  // namespace

// Whether the resident transform takes a call: N = 2^16 and enough limbs to give every compute unit one.
static unsigned resident_grid(const ckks_ctx* c) {
    // one workgroup per compute unit, a multiple of eight so that the XCDs get equal shares
    const unsigned grid = (unsigned)c->cu_count / 8 * 8;
    return grid ? grid : 8;
}
bool ntt_resident_applies(const ckks_ctx* c, int limbs) { return c->logN == 16 && limbs >= (int)resident_grid(c); }
int ntt_resident_round(const ckks_ctx* c) { return (int)resident_grid(c); }

// args: as for the two-launch transform.  FP64 back end, every prime of the call below 2^36 (the 36-bit form of the values between the passes).
int launch_ntt_resident(ckks_ctx* c, const NttArgs& args_in, int limbs, int count, bool inverse) {
    NttArgs args = args_in;
    args.limb_base = 0;
    args.limbs_total = (unsigned)limbs;
    args.mid = nullptr;
    args.tw = c->d_twd_fwd;                             // both directions read the forward table
    const dim3 g(resident_grid(c)), b(RES_LANES);
    // Successive launches of a context walk the rounds in opposite directions: where the same batch goes through several
    // transforms in a row, each starts on the limbs that the one before wrote last.  The order of the limbs has no effect
    // on the results.
    const unsigned backwards = c->res_backwards;
    c->res_backwards ^= 1u;
    if (!inverse) hipLaunchKernelGGL((ntt_resident_kernel<false>), g, b, 0, c->stream, args, (unsigned)count, backwards);
    else hipLaunchKernelGGL((ntt_resident_kernel<true>), g, b, 0, c->stream, args, (unsigned)count, backwards);
    CKKS_HIP_TRY(hipGetLastError());
    return CKKS_OK;
}

#ifdef CKKS_RES_TIMING
extern "C" int ckks_debug_resident_ticks(unsigned long long* out) {
    return hipMemcpyFromSymbol(out, HIP_SYMBOL(g_res_ticks), sizeof(unsigned long long) * 8 * 136) == hipSuccess ? 0 : 1;
}
#endif

}  // namespace ckks
