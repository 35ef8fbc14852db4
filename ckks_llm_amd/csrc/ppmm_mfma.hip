// Dense PPMM on the CDNA4 int8 matrix cores.
//
// out[m][i][c] = fused-rescale( sum_n A[m][n] * Ct_n[i][c]  mod q_i )        (semantics: pcmm.hip, PPMM_kernel.cuh:93-252)
//
// Exact integer product through base-256 balanced digits:
//     A[m][n]  = sum_{d<DW} a_d[m][n] * 256^d ,  a_d in [-128,127]   (int8 planes built once per call, shared by all primes)
//     Ct[n][c] = sum_{j<DC} b_j[n][c] * 256^j ,  b_j in [-128,127]   (bytes of (x + 0x8080808080) xor 0x80, made while staging)
//     sum_n A*Ct = sum_{e<DW+DC-1} 256^e * S_e ,   S_e = sum_{d+j=e} sum_n a_d*b_j    (int32, |S_e| <= min(DW,DC)*Kin*2^14)
// One v_mfma_i32_16x16x64_i8 per (d, j, 16x16 tile, 64 k) accumulates into the anti-diagonal accumulator S_{d+j}.
// The epilogue recombines the S_e without rounding in FP64 (three diagonals at a time fit 48 bits), reduces modulo q_i
// (q_i < 2^39) and applies the fused rescale (PPMM_kernel.cuh:213-249).
//
// Work decomposition: workgroup = 256 lanes = 4 waves owns a 128 (M) x 64 (columns) output tile for ALL primes
// (prime loop outermost, as in the reference: the rescale operand r_last is the lane's own earlier store); each wave owns a
// 64 x 32 sub-tile = 4 x 2 MFMA tiles x (DW+DC-1) accumulators.  K advances 64 at a time through double-buffered LDS:
//   A digits : global int8 planes -> LDS [d][row][64]            (16 B per lane, rows of 64 B)
//   residues : 16 consecutive-k u64 per lane (one column), digit-split and byte-transposed in registers -> LDS [j][col][64]
// so that every MFMA operand is one ds_read_b128.  Workgroups that share a column panel are numbered so that they land on
// the same XCD (ids congruent mod 8) back to back: the panel is fetched from HBM once and re-read from that XCD's L2.
#include <type_traits>

#include "pcmm.hpp"

namespace ckks {

typedef int v4i __attribute__((ext_vector_type(4)));

constexpr int MT = 128, CT = 64, KS = 64;        // workgroup tile and K step
constexpr int WM = 64, WC = 32;                  // wave tile
constexpr int DCMAX = 5;

typedef const __attribute__((address_space(1))) void* gptr_t;
typedef __attribute__((address_space(3))) void* lptr_t;
// 16 bytes per lane from global memory straight into LDS (no registers held while the load is in flight):
// lane l of the wave writes lds_base + 16*l.  lds_base must be wave-uniform.
__device__ __forceinline__ void async_copy16(const void* g, void* lds_base) {
    __builtin_amdgcn_global_load_lds((gptr_t)g, (lptr_t)lds_base, 16, 0, 0);
}

__device__ __forceinline__ double mulmod_f64(double a, double w, double q, double qinv) {
    double h = a * w;
    double l = __builtin_fma(a, w, -h);
    double c = __builtin_rint(h * qinv);
    return __builtin_fma(-c, q, h) + l;
}
__device__ __forceinline__ double balance_f64(double x, double q, double qinv) {
    return __builtin_fma(-__builtin_rint(x * qinv), q, x);
}

// Pipeline (global step s = prime iteration * ksteps + K step, parity p = s & 1; ksteps is even):
//   at the start of step s   : A[p], B[p] hold the digits of step s; RAW[(s+1)&1] holds the raw residues of step s+1
//   during step s            : asynchronous loads  A(s+1) -> A[p^1],  raw(s+2) -> RAW[p]      (nothing in registers)
//                              MFMAs of step s on A[p], B[p]  interleaved with  digit split of RAW[p^1] -> B[p^1]
//   end of step s            : wait for the loads, ONE workgroup barrier
// With four plaintext digits the LDS cannot hold two raw buffers; then raw(s+1) is loaded during step s and split after
// its MFMAs (OVERLAP = false).
// Every LDS buffer is a separate __shared__ object addressed with a compile-time parity, so that the compiler can tell
// that the asynchronous writes of a step never alias the operands the step's MFMAs read (otherwise it waits for the
// loads before the first LDS read and the overlap is lost).
template <int DW>
__global__ __launch_bounds__(256) void ppmm_mfma_kernel(PpmmArgs a, int c_tiles, int m_tiles) {
    constexpr int DC = DCMAX, ND = DW + DC - 1;
    constexpr bool OVERLAP = DW <= 3;
    __shared__ __align__(16) int8_t lds_a0[DW][MT][KS];
    __shared__ __align__(16) int8_t lds_a1[DW][MT][KS];
    __shared__ __align__(16) int8_t lds_b0[DC][CT][KS];       // 16-byte chunks xor-swizzled by column
    __shared__ __align__(16) int8_t lds_b1[DC][CT][KS];
    __shared__ __align__(16) u64 lds_raw0[KS][CT];
    __shared__ __align__(16) u64 lds_raw1[OVERLAP ? KS : 1][CT];

    // XCD-aware tile numbering: ids congruent mod 8 share an XCD; consecutive ones there share the column panel
    const unsigned id = blockIdx.x, xcd = id & 7, j = id >> 3;
    const unsigned m_tile = j % m_tiles, c_tile = (j / m_tiles) * 8 + xcd;
    if (c_tile >= (unsigned)c_tiles) return;
    const int m0 = m_tile * MT;
    const unsigned c0 = c_tile * CT;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);          // wave-uniform
    const int wm = wave >> 1, wc = wave & 1;
    const int lr = lane & 15, lg = lane >> 4;
    const int ksteps = a.Kpad / KS;
    const long plane = (long)a.Mpad * a.Kpad;
    const int8_t* a_tile = a.Adig + (long)m0 * a.Kpad;                   // uniform
    const unsigned a_lane_off = (unsigned)(lane >> 2) * (unsigned)a.Kpad + 16u * (lane & 3);   // row lane/4, chunk lane%4 of a 16-row slab
    const unsigned b_wr = (unsigned)lane * KS + 16u * (wave ^ ((lane >> 1) & 3));

    // Row pointers of the caller's MLWE table for one K step: lanes 0..15 of each wave fetch the 16 rows the wave stages
    // (rows 2*slab, 2*slab+1 for slab = wave + 4t) with ONE vector load, issued a whole step ahead of their use; they are
    // moved to scalar registers when needed.  (A scalar load of the table is not available to the compiler here: the
    // table lives in ordinary global memory that it cannot prove unwritten.)
    auto fetch_row_ptrs = [&](int ks) -> u64 {
        const int t = (lane >> 1) & 7, half = lane & 1;
        int k = ks * KS + 2 * (wave + 4 * t) + half;
        k = k < a.Kin ? k : a.Kin - 1;             // K padding: read a valid row; it is zeroed at the digit split
        return (u64)(uintptr_t)a.mlwe[k];
    };
    // DW*8 slabs of plaintext digits (16 rows x 64 B), 1 KiB each, dealt round-robin to the 4 waves
    auto issue_a = [&](int ks, int8_t (*dst)[MT][KS]) {
#pragma unroll
        for (int t = 0; t < DW * 2; t++) {
            const int slab = wave + 4 * t, d = slab >> 3, rr = slab & 7;
            async_copy16(a_tile + d * plane + (long)(rr * 16) * a.Kpad + ks * KS + a_lane_off, &dst[d][rr * 16][0]);
        }
    };
    // 32 slabs of raw residues (2 rows x 64 columns x 8 B), 1 KiB each
    auto issue_raw = [&](unsigned col_word, u64 row_ptrs, u64 (*dst)[CT]) {
        const unsigned lo = (unsigned)row_ptrs, hi = (unsigned)(row_ptrs >> 32);
#pragma unroll
        for (int t = 0; t < 8; t++) {
            const int slab = wave + 4 * t;                                 // rows 2*slab (lanes 0..31), 2*slab+1 (lanes 32..63)
            // readlane returns a signed int: convert each half to unsigned before widening, or the low half sign-extends
            // into the high half of the address
            const u64 pa = ((u64)(unsigned)__builtin_amdgcn_readlane((int)hi, 2 * t) << 32) | (u64)(unsigned)__builtin_amdgcn_readlane((int)lo, 2 * t);
            const u64 pb = ((u64)(unsigned)__builtin_amdgcn_readlane((int)hi, 2 * t + 1) << 32) | (u64)(unsigned)__builtin_amdgcn_readlane((int)lo, 2 * t + 1);
            const u64* p = (const u64*)(uintptr_t)(lane < 32 ? pa : pb) + col_word + 2 * (lane & 31);
            async_copy16(p, &dst[2 * slab][0]);
        }
    };
    // digit split of the raw residues of K step ks: lane = column, this wave's 16 rows
    auto split_digits = [&](int ks, const u64 (*src)[CT], int8_t (*dst)[CT][KS]) {
        const int kbase = ks * KS + 16 * wave;
        uint4 dig[DC];
        unsigned* dw = reinterpret_cast<unsigned*>(dig);
#pragma unroll
        for (int g = 0; g < 4; g++) {
            u64 y[4];
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const u64 v = src[16 * wave + 4 * g + i][lane];
                // bytes of x + 0x8080808080 are (digit + 128); rows of the K padding contribute zero digits
                y[i] = (kbase + 4 * g + i < a.Kin ? v : 0) + 0x8080808080ull;
            }
            const unsigned x0 = (unsigned)y[0], x1 = (unsigned)y[1], x2 = (unsigned)y[2], x3 = (unsigned)y[3];
            const unsigned t0 = __byte_perm(x0, x1, 0x5140), t1 = __byte_perm(x0, x1, 0x7362);
            const unsigned t2 = __byte_perm(x2, x3, 0x5140), t3 = __byte_perm(x2, x3, 0x7362);
            dw[0 * 4 + g] = __byte_perm(t0, t2, 0x5410) ^ 0x80808080u;
            dw[1 * 4 + g] = __byte_perm(t0, t2, 0x7632) ^ 0x80808080u;
            dw[2 * 4 + g] = __byte_perm(t1, t3, 0x5410) ^ 0x80808080u;
            dw[3 * 4 + g] = __byte_perm(t1, t3, 0x7632) ^ 0x80808080u;
            const unsigned h01 = __byte_perm((unsigned)(y[0] >> 32), (unsigned)(y[1] >> 32), 0x0040);
            const unsigned h23 = __byte_perm((unsigned)(y[2] >> 32), (unsigned)(y[3] >> 32), 0x0040);
            dw[4 * 4 + g] = __byte_perm(h01, h23, 0x5410) ^ 0x80808080u;
        }
#pragma unroll
        for (int jj = 0; jj < DC; jj++) *reinterpret_cast<uint4*>(&dst[jj][0][0] + b_wr) = dig[jj];
    };
    auto wait_loads = [&]() {
        __builtin_amdgcn_s_waitcnt(0x0F70);        // vmcnt(0): this wave's asynchronous loads have landed in LDS
        __syncthreads();                            // ... and so have everybody else's
    };

    // (ks1, im1) / (ks2, im2): K step and prime of the next / next-but-one global step, advanced without divisions;
    // im < 0 means "past the end".
    auto advance = [&](int& ks, int& im) { if (++ks == ksteps) { ks = 0; --im; } };
    auto col_word_of = [&](int im) { return (unsigned)(im < 0 ? 0 : im) * (unsigned)a.C + c0; };   // word offset in one MLWE ciphertext (< 2^32)
    int ks1 = 0, im1 = a.mod_num - 1, ks2, im2;
    u64 ptrs_next;

    // ---- prologue ----
    issue_a(0, lds_a0);
    issue_raw(col_word_of(im1), fetch_row_ptrs(0), lds_raw0);
    advance(ks1, im1);
    ks2 = ks1; im2 = im1;
    advance(ks2, im2);                                  // (ks1, im1) = step 1, (ks2, im2) = step 2
    if (OVERLAP) {
        if (im1 >= 0) issue_raw(col_word_of(im1), fetch_row_ptrs(ks1), lds_raw1);
        ptrs_next = fetch_row_ptrs(im2 >= 0 ? ks2 : 0);          // rows of raw(2), issued by step 0
    } else {
        ptrs_next = fetch_row_ptrs(im1 >= 0 ? ks1 : 0);          // rows of raw(1), issued by step 0
    }
    wait_loads();
    split_digits(0, lds_raw0, lds_b0);
    __syncthreads();

    v4i acc[ND][4][2];
    // one K step with compile-time buffer parity P
    auto kstep = [&](auto parity) {
        constexpr int P = decltype(parity)::value;
        int8_t (*A_cur)[MT][KS] = P ? lds_a1 : lds_a0;
        int8_t (*A_nxt)[MT][KS] = P ? lds_a0 : lds_a1;
        int8_t (*B_cur)[CT][KS] = P ? lds_b1 : lds_b0;
        int8_t (*B_nxt)[CT][KS] = P ? lds_b0 : lds_b1;
        // Branch-free on purpose: past the last step the loads re-fetch valid data into buffers nobody reads again, so the
        // whole step is one basic block and the loads / digit split can be interleaved with the MFMAs.
        const int ksn = im1 >= 0 ? ks1 : 0;
        issue_a(ksn, A_nxt);
        if (OVERLAP) {
            issue_raw(col_word_of(im2), ptrs_next, P ? lds_raw1 : lds_raw0);                    // raw(s+2) -> RAW[p]
            int ks3 = ks2, im3 = im2;
            advance(ks3, im3);
            ptrs_next = fetch_row_ptrs(im3 >= 0 ? ks3 : 0);              // rows of raw(s+3), used by the next step
            split_digits(ksn, P ? lds_raw0 : lds_raw1, B_nxt);          // RAW[p^1] -> B[p^1], overlaps the MFMAs below
        } else {
            issue_raw(col_word_of(im1), ptrs_next, lds_raw0);                                   // raw(s+1)
            ptrs_next = fetch_row_ptrs(im2 >= 0 ? ks2 : 0);
        }
        v4i bf[2][DC];
#pragma unroll
        for (int nt = 0; nt < 2; nt++) {
            const unsigned col = wc * WC + nt * 16 + lr;
            const unsigned rd = col * KS + 16u * (lg ^ ((col >> 1) & 3));
#pragma unroll
            for (int jj = 0; jj < DC; jj++) bf[nt][jj] = *reinterpret_cast<const v4i*>(&B_cur[jj][0][0] + rd);
        }
#pragma unroll
        for (int mt = 0; mt < 4; mt++) {
            v4i af[DW];
#pragma unroll
            for (int d = 0; d < DW; d++) af[d] = *reinterpret_cast<const v4i*>(&A_cur[d][wm * WM + mt * 16 + lr][16 * lg]);
#pragma unroll
            for (int nt = 0; nt < 2; nt++)
#pragma unroll
                for (int d = 0; d < DW; d++)
#pragma unroll
                    for (int jj = 0; jj < DC; jj++)
                        acc[d + jj][mt][nt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(af[d], bf[nt][jj], acc[d + jj][mt][nt], 0, 0, 0);
        }
        if (OVERLAP) {
            // scheduling pattern for the block above: after each MFMA issue up to three other instructions
            // (address arithmetic, asynchronous loads, digit split) while the matrix pipe works
#pragma unroll
            for (int i = 0; i < 4 * 2 * DW * DC; i++) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);      // one MFMA
                __builtin_amdgcn_sched_group_barrier(0x7f6, 3, 0);      // up to three non-MFMA instructions
            }
            wait_loads();
        } else {
            wait_loads();
            split_digits(ksn, lds_raw0, B_nxt);
            __syncthreads();
        }
        advance(ks1, im1);
        advance(ks2, im2);
    };

    // r_last (residues modulo the last prime, < 2^39) of this lane's 32 outputs, kept in registers for the fused rescale
    // of the other primes: low words, and the 7 high bits packed four to a word.
    unsigned rl_lo[4][4][2], rl_hi[4][2];
    auto epilogue = [&](int im, auto last_c, auto full_c) {
        constexpr bool LAST = decltype(last_c)::value, FULL = decltype(full_c)::value;
        // The output addressing starts from a value the optimiser cannot hoist above the K loop (it would otherwise keep
        // 32 row pointers alive across the loop and spill them).
        long row_stride = (long)a.mod_num * a.C;
        asm volatile("" : "+s"(row_stride));
        const PrimeConst& pr = a.pq[a.np + im];
        const double q = pr.qd, qinv = pr.qinv_d;
        const double c24 = __longlong_as_double((long long)a.consts[2 * PPMM_MAX_MODS + im]);   // 2^24 mod q
        const double c48 = __longlong_as_double((long long)a.consts[3 * PPMM_MAX_MODS + im]);   // 2^48 mod q
        const double qli = __longlong_as_double((long long)a.consts[4 * PPMM_MAX_MODS + im]);   // q_last^-1 mod q
        const int mrow = m0 + wm * WM + 4 * lg;
        u64* obase = a.out + (long)im * a.C + c0 + wc * WC + lr;
#pragma unroll
        for (int mt = 0; mt < 4; mt++) {
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const int row = mrow + mt * 16 + r;
                // rows of the M padding are clamped for addressing; their stores are skipped
                u64* orow = obase + (long)(FULL || row < a.M ? row : a.M - 1) * row_stride;
#pragma unroll
                for (int nt = 0; nt < 2; nt++) {
                    double y[3] = {0.0, 0.0, 0.0};
#pragma unroll
                    for (int e = ND - 1; e >= 0; e--) {
                        // Horner inside each group of three diagonals: y_g = S_3g + 256*S_3g+1 + 65536*S_3g+2  (|y_g| < 2^48, exact)
                        const int g = e / 3;
                        y[g] = __builtin_fma(y[g], 256.0, (double)acc[e][mt][nt][r]);
                    }
                    double t = balance_f64(y[0], q, qinv);
                    if (ND > 3) t += mulmod_f64(y[1], c24, q, qinv);
                    if (ND > 6) t += mulmod_f64(y[2], c48, q, qinv);
                    t = balance_f64(t, q, qinv);                                           // in (-0.51 q, 0.51 q)
                    double res;
                    if (LAST) {
                        res = t;
                    } else {
                        // (r_i + q_i - r_last) * q_last^-1 mod q_i ; r_last is used as an integer without reduction
                        // modulo q_i, as in PPMM_kernel.cuh:243-247
                        const unsigned hi = (rl_hi[mt][nt] >> (8 * r)) & 0xff;
                        const double rlast = __builtin_fma((double)hi, 4294967296.0, (double)rl_lo[mt][r][nt]);
                        res = mulmod_f64(t - rlast, qli, q, qinv);
                    }
                    res = res < 0.0 ? res + q : res;
                    const u64 ures = (u64)(long long)res;
                    if (LAST) {
                        rl_lo[mt][r][nt] = (unsigned)ures;
                        rl_hi[mt][nt] = (r == 0 ? 0u : rl_hi[mt][nt]) | ((unsigned)(ures >> 32) << (8 * r));
                    }
                    if (FULL) orow[nt * 16] = ures;
                    else if (row < a.M) orow[nt * 16] = ures;
                }
            }
        }
    };

    for (int im = a.mod_num - 1; im >= 0; im--) {
#pragma unroll
        for (int e = 0; e < ND; e++)
#pragma unroll
            for (int mt = 0; mt < 4; mt++)
#pragma unroll
                for (int nt = 0; nt < 2; nt++) acc[e][mt][nt] = v4i{0, 0, 0, 0};

        for (int ks = 0; ks < ksteps; ks += 2) {
            kstep(std::integral_constant<int, 0>{});
            kstep(std::integral_constant<int, 1>{});
        }

        // ---- end of a prime: exact recombination, reduction mod q, fused rescale ----
        // Straight-line code (the prime-position and M-padding cases are resolved once, outside the unrolled loops) so that
        // the 32 independent output chains of a lane can be interleaved.
        const bool last = im == a.mod_num - 1, full = m0 + MT <= a.M;
        if (last) { if (full) epilogue(im, std::true_type{}, std::true_type{}); else epilogue(im, std::true_type{}, std::false_type{}); }
        else      { if (full) epilogue(im, std::false_type{}, std::true_type{}); else epilogue(im, std::false_type{}, std::false_type{}); }
    }
}

template <int DW>
static int launch_dw(hipStream_t stream, const PpmmArgs& a) {
    const int c_tiles = (int)(a.C / CT), m_tiles = a.Mpad / MT;
    const unsigned blocks = (unsigned)((c_tiles + 7) / 8) * 8u * (unsigned)m_tiles;
    hipLaunchKernelGGL(ppmm_mfma_kernel<DW>, dim3(blocks), dim3(256), 0, stream, a, c_tiles, m_tiles);
    CKKS_HIP_TRY(hipGetLastError());
    return CKKS_OK;
}

int launch_ppmm_mfma_impl(hipStream_t stream, const PpmmArgs& a, int DW) {
    if (DW <= 3) return launch_dw<3>(stream, a);
    return launch_dw<4>(stream, a);
}

}  // namespace ckks
