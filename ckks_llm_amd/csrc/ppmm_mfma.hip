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
#include "pcmm.hpp"

namespace ckks {

typedef int v4i __attribute__((ext_vector_type(4)));

constexpr int MT = 128, CT = 64, KS = 64;        // workgroup tile and K step
constexpr int WM = 64, WC = 32;                  // wave tile
constexpr int DCMAX = 5;

template <int DW>
struct Smem {
    int8_t a[2][DW][MT][KS];          // plaintext digits, double buffered
    int8_t b[2][DCMAX][CT][KS];       // residue digits, double buffered (16-byte chunks xor-swizzled by column)
    u64 raw[KS][CT];                  // landing zone of the asynchronous residue loads of the next K step
};

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

template <int DW>
__global__ __launch_bounds__(256) void ppmm_mfma_kernel(PpmmArgs a, int c_tiles, int m_tiles) {
    constexpr int DC = DCMAX, ND = DW + DC - 1;
    extern __shared__ __align__(16) unsigned char smem_raw[];
    Smem<DW>& sm = *reinterpret_cast<Smem<DW>*>(smem_raw);

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

    // Asynchronous staging of K step ks: DW*8 slabs of plaintext digits (16 rows x 64 B) and 32 slabs of raw residues
    // (2 rows x 64 columns x 8 B), 1 KiB each, dealt round-robin to the 4 waves.
    auto issue_loads = [&](int ks, int buf, unsigned col_word) {
        const int k0 = ks * KS;
#pragma unroll
        for (int t = 0; t < DW * 2; t++) {
            const int slab = wave + 4 * t, d = slab >> 3, rr = slab & 7;
            async_copy16(a_tile + d * plane + (long)(rr * 16) * a.Kpad + k0 + a_lane_off, &sm.a[buf][d][rr * 16][0]);
        }
#pragma unroll
        for (int t = 0; t < 8; t++) {
            const int slab = wave + 4 * t;                                 // rows 2*slab, 2*slab+1
            int ka = k0 + 2 * slab, kb = ka + 1;
            ka = ka < a.Kin ? ka : a.Kin - 1;                              // K padding: read a valid row; it is zeroed at the digit split
            kb = kb < a.Kin ? kb : a.Kin - 1;
            const u64* pa = a.mlwe[ka];                                    // scalar loads
            const u64* pb = a.mlwe[kb];
            const u64* p = (lane < 32 ? pa : pb) + col_word + 2 * (lane & 31);
            async_copy16(p, &sm.raw[2 * slab][0]);
        }
    };
    // digit split of the raw residues of K step ks into b[buf]: lane = column, this wave's 16 rows
    auto split_digits = [&](int ks, int buf) {
        const int kbase = ks * KS + 16 * wave;
        uint4 dig[DC];
        unsigned* dw = reinterpret_cast<unsigned*>(dig);
#pragma unroll
        for (int g = 0; g < 4; g++) {
            u64 y[4];
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const u64 v = sm.raw[16 * wave + 4 * g + i][lane];
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
        for (int jj = 0; jj < DC; jj++) *reinterpret_cast<uint4*>(&sm.b[buf][jj][0][0] + b_wr) = dig[jj];
    };
    auto wait_loads = [&]() {
        __builtin_amdgcn_s_waitcnt(0x0F70);        // vmcnt(0): this wave's asynchronous loads have landed in LDS
        __syncthreads();                            // ... and so have everybody else's
    };

    for (int im = a.mod_num - 1; im >= 0; im--) {
        v4i acc[ND][4][2];
#pragma unroll
        for (int e = 0; e < ND; e++)
#pragma unroll
            for (int mt = 0; mt < 4; mt++)
#pragma unroll
                for (int nt = 0; nt < 2; nt++) acc[e][mt][nt] = v4i{0, 0, 0, 0};

        const unsigned col_word = (unsigned)im * (unsigned)a.C + c0;       // word offset inside one MLWE ciphertext (< 2^32)
        issue_loads(0, 0, col_word);
        wait_loads();
        split_digits(0, 0);
        __syncthreads();
        for (int ks = 0; ks < ksteps; ks++) {
            const int buf = ks & 1;
            if (ks + 1 < ksteps) issue_loads(ks + 1, buf ^ 1, col_word);
            v4i bf[2][DC];
#pragma unroll
            for (int nt = 0; nt < 2; nt++) {
                const unsigned col = wc * WC + nt * 16 + lr;
                const unsigned rd = col * KS + 16u * (lg ^ ((col >> 1) & 3));
#pragma unroll
                for (int jj = 0; jj < DC; jj++) bf[nt][jj] = *reinterpret_cast<const v4i*>(&sm.b[buf][jj][0][0] + rd);
            }
#pragma unroll
            for (int mt = 0; mt < 4; mt++) {
                v4i af[DW];
#pragma unroll
                for (int d = 0; d < DW; d++) af[d] = *reinterpret_cast<const v4i*>(&sm.a[buf][d][wm * WM + mt * 16 + lr][16 * lg]);
#pragma unroll
                for (int nt = 0; nt < 2; nt++)
#pragma unroll
                    for (int d = 0; d < DW; d++)
#pragma unroll
                        for (int jj = 0; jj < DC; jj++)
                            acc[d + jj][mt][nt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(af[d], bf[nt][jj], acc[d + jj][mt][nt], 0, 0, 0);
            }
            if (ks + 1 < ksteps) {
                wait_loads();
                split_digits(ks + 1, buf ^ 1);
            }
            __syncthreads();
        }

        // ---- epilogue: exact recombination, reduction mod q, fused rescale ----
        // The output addressing starts from a value the optimiser cannot hoist above the K loop (it would otherwise keep
        // 32 row pointers alive across the loop and spill them).
        long row_stride = (long)a.mod_num * a.C;
        asm volatile("" : "+s"(row_stride));
        const PrimeConst& pr = a.pq[a.np + im];
        const double q = pr.qd, qinv = pr.qinv_d;
        const double c24 = __longlong_as_double((long long)a.consts[2 * PPMM_MAX_MODS + im]);   // 2^24 mod q
        const double c48 = __longlong_as_double((long long)a.consts[3 * PPMM_MAX_MODS + im]);   // 2^48 mod q
        const double qli = __longlong_as_double((long long)a.consts[4 * PPMM_MAX_MODS + im]);   // q_last^-1 mod q
        const bool last = im == a.mod_num - 1;
        const int mrow = m0 + wm * WM + 4 * lg;
        u64* obase = a.out + (long)mrow * row_stride + (long)im * a.C + c0 + wc * WC + lr;
        const long last_off = (long)(a.mod_num - 1 - im) * a.C;
#pragma unroll
        for (int mt = 0; mt < 4; mt++)
#pragma unroll
            for (int r = 0; r < 4; r++) {
                u64* orow = obase + (long)(mt * 16 + r) * row_stride;
                const bool row_ok = mrow + mt * 16 + r < a.M;
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
                    if (row_ok) {
                        double res;
                        if (last) {
                            res = t < 0.0 ? t + q : t;
                        } else {
                            // (r_i + q_i - r_last) * q_last^-1 mod q_i ; r_last is this lane's own earlier store, used as an
                            // integer without reduction modulo q_i, as in PPMM_kernel.cuh:243-247
                            const double rl = (double)(long long)orow[nt * 16 + last_off];
                            res = mulmod_f64(t - rl, qli, q, qinv);
                            res = res < 0.0 ? res + q : res;
                        }
                        orow[nt * 16] = (u64)(long long)res;
                    }
                }
            }
        __syncthreads();
    }
}

template <int DW>
static int launch_dw(hipStream_t stream, const PpmmArgs& a) {
    const int c_tiles = (int)(a.C / CT), m_tiles = a.Mpad / MT;
    const unsigned blocks = (unsigned)((c_tiles + 7) / 8) * 8u * (unsigned)m_tiles;
    const size_t smem = sizeof(Smem<DW>);
    static bool attr_set = false;
    if (!attr_set) {
        CKKS_HIP_TRY(hipFuncSetAttribute((const void*)ppmm_mfma_kernel<DW>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
        attr_set = true;
    }
    hipLaunchKernelGGL(ppmm_mfma_kernel<DW>, dim3(blocks), dim3(256), smem, stream, a, c_tiles, m_tiles);
    CKKS_HIP_TRY(hipGetLastError());
    return CKKS_OK;
}

int launch_ppmm_mfma_impl(hipStream_t stream, const PpmmArgs& a, int DW) {
    if (DW <= 3) return launch_dw<3>(stream, a);
    return launch_dw<4>(stream, a);
}

}  // namespace ckks
