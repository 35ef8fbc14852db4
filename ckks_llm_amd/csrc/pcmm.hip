// Ring-packed plaintext x ciphertext matrix product (PPMM) and the RLWE -> MLWE gather for gfx950.
//
// Replaces PCMM_Context (pcmm/PCMM_Context.cuh:7-57), the gather kernel of PCMM_Scheme::rlweCipherDecompose
// (pcmm/PCMM_Scheme.cuh:50-125) and pcmm_cuda_core_kernel / PCMM_Scheme::PPMM (pcmm/PPMM_kernel.cuh:93-349).
//
// PPMM semantics (per ring-pack prime q_i, i = mod_num-1 .. 0; C = (rank+1)*N1 columns):
//     A[m][n]   = (int64) ((double) W[m][n] * scaler)                     truncation toward zero  (PPMM_kernel.cuh:148)
//     r_i[m][c] = sum_n A[m][n] * Ct_n[i][c]  mod q_i                     (the reference maps A <= 0 to q + A, :25)
//     out[m][last][c] = r_last ;  out[m][i][c] = (r_i + q_i - r_last) * q_last^-1 mod q_i   (fused rescale, :213-249)
// The reference fixes mod_num = 2 (its rescale table offset is hard-wired to l = 1, :298); this implementation takes
// any mod_num >= 1 and uses q_last^-1 mod q_i, which is the same constant when mod_num = 2.
//
// Two kernels compute it:
//   * ppmm_mfma_kernel  - the dense path.  A is split once into DW balanced base-256 digits (int8 planes shared by
//     all primes); a first pass splits every residue into DC balanced digits (bytes of x + 0x80..80, each xor 0x80)
//     laid out as the MFMA operand slabs; v_mfma_i32_16x16x64_i8 accumulates the DW*DC digit products into DW+DC-1
//     int32 anti-diagonal accumulators; the epilogue recombines them exactly and reduces modulo q_i.
//   * ppmm_generic_kernel - one output per lane with 128-bit accumulation, for shapes the MFMA tiling does not cover
//     (C not a multiple of 64, primes of 40 bits and more, |A| >= 2^31, DW * Kin > 2^14).
#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <vector>

#include "pcmm.hpp"
#include "host_math.hpp"

namespace ckks {

// ------------------------------------------------------------------------------------------------------------
// RLWE -> MLWE gather (PCMM_Scheme.cuh:50-88)
// ------------------------------------------------------------------------------------------------------------
struct GatherArgs {
    const u64* rlwe;
    u64* const* mlwe;
    const PrimeConst* primes;   // context primes
    long N;
    int N1, rank, mlwe_num, L, p_num;
};
__global__ __launch_bounds__(256) void rlwe_gather_kernel(GatherArgs a) {
    // one lane per output word: flat index over (row i in [0, rank], g in [0, N1))
    const long flat = (long)blockIdx.x * 256 + threadIdx.x;
    const int k = a.rank, N1 = a.N1;
    if (flat >= (long)(k + 1) * N1) return;
    const int i = (int)(flat / N1), g = (int)(flat % N1);
    const int im = blockIdx.y, m = blockIdx.z;
    const u64 q = a.primes[a.p_num + im].q;
    const u64* A = a.rlwe + a.N * im;
    const u64* B = a.rlwe + a.N * (a.L + 1 + im);
    u64* dst = a.mlwe[m] + (long)N1 * (k + 1) * im;
    const int gap = k / a.mlwe_num;
    u64 v;
    if (i == k) {                                           // b row
        long addr = (long)m * gap + (long)g * k;
        v = addr >= a.N ? negate_mod(B[addr - a.N], q) : B[addr];
    } else if (i == 0) {
        long addr = (long)m * gap + (long)g * k;
        v = addr >= a.N ? negate_mod(A[addr - a.N], q) : A[addr];
    } else if (g == 0) {
        long addr = (long)(N1 - 1) * k + (k - i) + (long)m * gap;
        v = addr >= a.N ? A[addr - a.N] : negate_mod(A[addr], q);
    } else {
        long addr = (long)(g - 1) * k + (k - i) + (long)m * gap;
        v = addr >= a.N ? negate_mod(A[addr - a.N], q) : A[addr];
    }
    dst[(long)i * N1 + g] = v;
}

// The same gather through LDS.  Row i of sample m is the negacyclic polynomial a read at positions g*k + (m*gap - i), g = 0..N1-1
// (positions below zero wrap to the top with a sign change), so for a tile of G consecutive g every row needs the contiguous
// window [g0*k - (k-1), (g0+G)*k): it is loaded once, coalesced, into LDS (one pad word per k so that lanes on consecutive g hit
// different banks) and every output row segment (G words = 64 or 128 contiguous bytes) is written from there.  The output is
// k times larger than the input; the kernel is bound by its writes.
constexpr int GATHER_M_CHUNK = 8;          // samples per workgroup
template <int G>
__global__ __launch_bounds__(256) void rlwe_gather_tiled_kernel(GatherArgs a) {
    extern __shared__ u64 win[];                                     // (G + 1) * (k + 1) words
    const int k = a.rank, N1 = a.N1, im = blockIdx.y, g0 = blockIdx.x * G;
    const int gap = k / a.mlwe_num;
    const u64 q = a.primes[a.p_num + im].q;
    const u64* A = a.rlwe + a.N * im;
    const u64* B = a.rlwe + a.N * (a.L + 1 + im);
    // window position u = p - g0*k + k, p = polynomial position; LDS index u + u / k
    for (int u = threadIdx.x + 1; u < (G + 1) * k; u += 256) {
        const long p = (long)g0 * k + u - k;
        win[u + u / k] = p >= 0 ? A[p] : negate_mod(A[a.N + p], q);
    }
    __syncthreads();
    const int gl = threadIdx.x % G, slot = threadIdx.x / G;
    constexpr int SLOTS = 256 / G;
    const int m_end = min(a.mlwe_num, (int)(blockIdx.z + 1) * GATHER_M_CHUNK);
    for (int m = blockIdx.z * GATHER_M_CHUNK; m < m_end; m++) {
        u64* dst = a.mlwe[m] + (long)N1 * (k + 1) * im + g0 + gl;
        const int base = gl * k + k + m * gap;                       // u of row 0
        for (int i = slot; i < k; i += SLOTS) {
            const int u = base - i;
            dst[(long)i * N1] = win[u + u / k];
        }
        if (slot == 0) dst[(long)k * N1] = B[(long)m * gap + (long)(g0 + gl) * k];       // b row: no shift, never wraps
    }
}

// The gather writing PPMM's operand directly: the same window in LDS, but instead of 8-byte words in the MLWE layout the five
// balanced base-256 digits of every value go straight into the residue digit planes of the MFMA kernel
// (Bdig[prime][K step][64-column tile][digit][16-column slab], slab = [16-byte k chunk][column][16 k]; sample = k index,
// column = row i * N1 + g).  A workgroup owns 16 consecutive g of one prime and 64 consecutive samples; a wave takes a row i at
// a time, lane (col, kc) = 16 samples of one column, so that a wave writes one whole 1 KiB slab per digit with one store.
// The MLWE samples never exist as 8-byte words: 5 bytes are written per value instead of 8 written, 8 read and 5 written.
struct GatherDigitsArgs {
    const u64* rlwe;
    int8_t* bdig;
    const PrimeConst* primes;
    long N;
    int N1, rank, mlwe_num, L, p_num, kstep0, ksteps, c_tiles;
};
__global__ __launch_bounds__(256) void rlwe_gather_digits_kernel(GatherDigitsArgs a) {
    extern __shared__ u64 win[];                                     // 17 * (k + 1) words
    constexpr int G = 16;
    const int k = a.rank, N1 = a.N1, im = blockIdx.y, g0 = blockIdx.x * G;
    const int gap = k / a.mlwe_num;
    const u64 q = a.primes[a.p_num + im].q;
    const u64* A = a.rlwe + a.N * im;
    const u64* B = a.rlwe + a.N * (a.L + 1 + im);
    for (int u = threadIdx.x + 1; u < (G + 1) * k; u += 256) {
        const long p = (long)g0 * k + u - k;
        win[u + u / k] = p >= 0 ? A[p] : negate_mod(A[a.N + p], q);
    }
    __syncthreads();
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int col = lane & 15, kc = lane >> 4;
    const int m0 = blockIdx.z * 64 + 16 * kc;                        // first of this lane's 16 samples
    int8_t* step_base = a.bdig + ((long)im * a.ksteps + a.kstep0 + blockIdx.z) * (long)a.c_tiles * (5 * 64 * 64) + kc * 256 + col * 16;
    for (int i = wave; i <= k; i += 4) {
        uint4 dig[5];
        unsigned* dw = reinterpret_cast<unsigned*>(dig);
#pragma unroll
        for (int grp = 0; grp < 4; grp++) {
            u64 y[4];
#pragma unroll
            for (int t = 0; t < 4; t++) {
                const int m = m0 + 4 * grp + t;
                u64 x;
                if (i < k) {
                    const int d = m * gap - i;                       // in (-k, k)
                    x = win[(col + 1) * k + d + col + 1 - (d < 0)];
                } else {
                    x = B[(long)m * gap + (long)(g0 + col) * k];     // b row: no shift, never wraps
                }
                y[t] = x + 0x8080808080ull;                          // bytes = digit + 128
            }
            const unsigned x0 = (unsigned)y[0], x1 = (unsigned)y[1], x2 = (unsigned)y[2], x3 = (unsigned)y[3];
            const unsigned t0 = __byte_perm(x0, x1, 0x5140), t1 = __byte_perm(x0, x1, 0x7362);
            const unsigned t2 = __byte_perm(x2, x3, 0x5140), t3 = __byte_perm(x2, x3, 0x7362);
            dw[0 * 4 + grp] = __byte_perm(t0, t2, 0x5410) ^ 0x80808080u;
            dw[1 * 4 + grp] = __byte_perm(t0, t2, 0x7632) ^ 0x80808080u;
            dw[2 * 4 + grp] = __byte_perm(t1, t3, 0x5410) ^ 0x80808080u;
            dw[3 * 4 + grp] = __byte_perm(t1, t3, 0x7632) ^ 0x80808080u;
            const unsigned h01 = __byte_perm((unsigned)(y[0] >> 32), (unsigned)(y[1] >> 32), 0x0040);
            const unsigned h23 = __byte_perm((unsigned)(y[2] >> 32), (unsigned)(y[3] >> 32), 0x0040);
            dw[4 * 4 + grp] = __byte_perm(h01, h23, 0x5410) ^ 0x80808080u;
        }
        const long c = (long)i * N1 + g0;                            // first column of this wave's slab
        int8_t* dst = step_base + (c / 64) * (5 * 64 * 64) + ((c % 64) / 16) * 1024;
#pragma unroll
        for (int jj = 0; jj < 5; jj++) *reinterpret_cast<uint4*>(dst + jj * 4096) = dig[jj];
    }
}

// ------------------------------------------------------------------------------------------------------------
// plaintext quantisation: A = (int64)(float * double), |A| maximum, balanced base-256 digit planes
// ------------------------------------------------------------------------------------------------------------
constexpr int QUANT_PER_LANE = 8;
__global__ __launch_bounds__(256) void quantise_kernel(const float* W, long long* A, unsigned long long* absmax, long count, double scaler) {
    __shared__ unsigned long long wave_max[4];
    unsigned long long m = 0;
    const long base = (long)blockIdx.x * 256 * QUANT_PER_LANE + threadIdx.x;
#pragma unroll
    for (int t = 0; t < QUANT_PER_LANE; t++) {
        const long i = base + t * 256;
        if (i < count) {
            long long v = (long long)((double)W[i] * scaler);
            A[i] = v;
            const unsigned long long av = (unsigned long long)(v < 0 ? -v : v);
            m = av > m ? av : m;
        }
    }
    for (int off = 32; off > 0; off >>= 1) {
        unsigned long long o = __shfl_down(m, off);
        m = o > m ? o : m;
    }
    // one atomic per workgroup: thousands of atomics on one word were most of this kernel's time
    if ((threadIdx.x & 63) == 0) wave_max[threadIdx.x >> 6] = m;
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < 4; w++) m = wave_max[w] > m ? wave_max[w] : m;
        if (m) atomicMax(absmax, m);
    }
}
// digit d of A (balanced, in [-128, 127]): byte d of (A + 0x80..80) xor 0x80.  The planes are written in the order the MFMA kernel
// stages them: [digit][16-row group][64-deep K step] slabs of 1 KiB, inside a slab [16-byte k chunk][row][16 k].
__global__ __launch_bounds__(256) void digits_kernel(const long long* A, int8_t* dig, int M, int Kin, int Mpad, int Kpad, int DW) {
    long i = (long)blockIdx.x * 256 + threadIdx.x;
    if (i >= (long)Mpad * Kpad) return;
    int m = (int)(i / Kpad), n = (int)(i % Kpad);
    unsigned long long biased = 0x8080808080808080ull;
    if (m < M && n < Kin) biased += (unsigned long long)A[(long)m * Kin + n];
    const long pos = ((long)(m >> 4) * (Kpad >> 6) + (n >> 6)) * 1024 + ((n & 63) >> 4) * 256 + (m & 15) * 16 + (n & 15);
    // digits above the eighth are zero: the MFMA path takes |A| below the smallest prime, far below 2^63
    for (int d = 0; d < DW; d++) dig[(long)d * Mpad * Kpad + pos] = d < 8 ? (int8_t)(((biased >> (8 * d)) & 0xff) ^ 0x80) : (int8_t)0;
}

// ------------------------------------------------------------------------------------------------------------
// generic kernel: one output per lane, 128-bit accumulation (the reference's arithmetic, PPMM_kernel.cuh:12-31)
// ------------------------------------------------------------------------------------------------------------
__device__ __forceinline__ const u64* mlwe_row(const PpmmArgs& a, int n) { return a.mlwe[n]; }
__global__ __launch_bounds__(256) void ppmm_generic_kernel(PpmmArgs a) {
    const long c = (long)blockIdx.x * 256 + threadIdx.x;
    const int m = blockIdx.y;
    if (c >= a.C) return;
    u64* o = a.out + (long)m * a.C * a.mod_num;
    u64 r_last = 0;
    for (int im = a.mod_num - 1; im >= 0; im--) {
        const PrimeConst& pr = a.pq[a.np + im];
        u128w acc = {0, 0};
        for (int n = 0; n < a.Kin; n++) {
            long long t = a.A[(long)m * a.Kin + n];
            u64 w = t > 0 ? (u64)t : pr.q + (u64)t;                       // PPMM_kernel.cuh:25
            mac128(acc, w, mlwe_row(a, n)[(long)im * a.C + c]);
        }
        u64 r = barrett128(acc, pr.q, pr.mu_hi, pr.mu_lo);
        if (im == a.mod_num - 1) {
            r_last = r;
            o[(long)im * a.C + c] = r;
        } else {
            u64 temp = r + pr.q - r_last;                                   // :244
            o[(long)im * a.C + c] = mul_shoup(temp, a.consts[im], a.consts[PPMM_MAX_MODS + im], pr.q);
        }
    }
}

// ------------------------------------------------------------------------------------------------------------
// Plaintext matrices wider than one MFMA launch takes (more than 4 balanced digits, 3 with the 7-digit residues) are cut into
// slices of three digits, A = sum_s A_s 2^(24 s): one launch per slice writes the residues of A_s x Ct as they are, and this
// kernel forms sum_s (2^(24 s) mod q) * slice_s mod q and then the fused rescale of PPMM_kernel.cuh:213-249 - the same
// integers as one pass over the whole of A, since every step is exact modulo the prime.
// ------------------------------------------------------------------------------------------------------------
struct PpmmCombineArgs {
    u64* out;                     // slice 0 on entry, the result on return; [M][mod_num][C]
    const u64* more;              // slices 1 .. slices-1, each [M][mod_num][C]
    const PrimeConst* pq;
    const u64* consts;            // row 0: q_last^-1 mod q_i, row 1: its Shoup word
    long C, per_slice;            // per_slice = M * mod_num * C
    int M, mod_num, np, slices;
    u64 w[2][PPMM_MAX_MODS];      // 2^24 mod q_i, 2^48 mod q_i
};
__global__ __launch_bounds__(256) void ppmm_combine_kernel(PpmmCombineArgs a) {
    const long c = (long)blockIdx.x * 256 + threadIdx.x;
    const int m = blockIdx.y;
    if (c >= a.C) return;
    u64* o = a.out + (long)m * a.C * a.mod_num;
    const u64* t = a.more + (long)m * a.C * a.mod_num;
    u64 r_last = 0;
    for (int im = a.mod_num - 1; im >= 0; im--) {
        const PrimeConst& pr = a.pq[a.np + im];
        const long idx = (long)im * a.C + c;
        u128w acc = {o[idx], 0};
        for (int s = 1; s < a.slices; s++) mac128(acc, t[(long)(s - 1) * a.per_slice + idx], a.w[s - 1][im]);
        const u64 r = barrett128(acc, pr.q, pr.mu_hi, pr.mu_lo);
        if (im == a.mod_num - 1) {
            r_last = r;
            o[idx] = r;
        } else {
            const u64 temp = r + pr.q - r_last;                             // PPMM_kernel.cuh:244
            o[idx] = mul_shoup(temp, a.consts[im], a.consts[PPMM_MAX_MODS + im], pr.q);
        }
    }
}

}  // namespace ckks

using namespace ckks;
namespace H = ckks_host;

// every live handle, for pcmm_forget_weights
static std::mutex g_handles_mutex;
static std::vector<pcmm_ctx*> g_handles;
static void drop_weights(pcmm_ctx* h, pcmm_ctx::Weights* w);
extern "C" int pcmm_ctx_create(pcmm_ctx** out, ckks_ctx* ctx, int N1, int rank, const uint64_t* p, int np, const uint64_t* q, int nq) {
    if (!out || !ctx || N1 <= 0 || rank <= 0 || nq < 1 || np < 0 || (np > 0 && !p) || !q) { set_error("pcmm_ctx_create: bad argument"); return CKKS_E_INVALID; }
    if ((long)N1 * rank != ctx->N) { set_error("pcmm_ctx_create: N1 * mlwe_rank must equal N"); return CKKS_E_INVALID; }
    pcmm_ctx* h = new pcmm_ctx();
    h->ctx = ctx; h->N1 = N1; h->rank = rank; h->np = np; h->nq = nq;
    for (int i = 0; i < np; i++) h->pq.push_back(p[i]);
    for (int i = 0; i < nq; i++) h->pq.push_back(q[i]);
    std::vector<PrimeConst> pc(h->pq.size());
    for (size_t i = 0; i < h->pq.size(); i++) {
        uint64_t m = h->pq[i];
        if (m < 3 || (m & 1) == 0 || m >= (1ull << 62)) { delete h; set_error("pcmm_ctx_create: moduli must be odd and < 2^62"); return CKKS_E_INVALID; }
        PrimeConst& P = pc[i];
        memset(&P, 0, sizeof(P));
        uint64_t hi, lo;
        H::barrett_mu(m, hi, lo);
        P.q = m; P.mu_hi = hi; P.mu_lo = lo; P.qd = (double)m; P.qinv_d = 1.0 / (double)m; P.f64_ok = m < (1ull << 41);
    }
    hipError_t e = hipMalloc((void**)&h->d_pq, pc.size() * sizeof(PrimeConst));
    if (e == hipSuccess) e = hipMemcpy(h->d_pq, pc.data(), pc.size() * sizeof(PrimeConst), hipMemcpyHostToDevice);
    if (e == hipSuccess) e = hipMalloc((void**)&h->d_absmax, sizeof(unsigned long long) * (1 + PPMM_CONST_WORDS));
    if (e != hipSuccess) { pcmm_ctx_destroy(h); return hip_fail(e, "pcmm_ctx_create"); }
    { std::lock_guard<std::mutex> lock(g_handles_mutex); g_handles.push_back(h); }
    *out = h;
    return CKKS_OK;
}
extern "C" int pcmm_ctx_destroy(pcmm_ctx* h) {
    if (!h) return CKKS_OK;
    { std::lock_guard<std::mutex> lock(g_handles_mutex); g_handles.erase(std::remove(g_handles.begin(), g_handles.end(), h), g_handles.end()); }
    (void)hipDeviceSynchronize();
    void* ptrs[] = {h->d_pq, h->d_ptrs, h->d_absmax, h->d_zero, h->d_Bdig, h->d_small_tw, h->d_slices, h->d_workA, h->d_workAdig};
    for (void* p : ptrs) if (p) (void)hipFree(p);
    for (auto& w : h->weights) { if (w.d_A) (void)hipFree(w.d_A); if (w.d_Adig) (void)hipFree(w.d_Adig); }
    if (h->pin) (void)hipHostFree(h->pin);
    if (h->pin_ev) (void)hipEventDestroy(h->pin_ev);
    if (h->h_absmax) (void)hipHostFree(h->h_absmax);
    if (h->ev_absmax) (void)hipEventDestroy(h->ev_absmax);
    if (h->small) ckks_ctx_destroy(h->small);
    delete h;
    return CKKS_OK;
}

static int upload_ptrs(pcmm_ctx* h, const uint64_t* const* host_ptrs, int count) {
    h->tab_sent.clear();                                                   // the table PPMM last sent is overwritten
    if (count > h->ptr_cap) {
        if (h->d_ptrs) { (void)hipDeviceSynchronize(); (void)hipFree(h->d_ptrs); h->d_ptrs = nullptr; }
        int cap = std::max(count, 3072);                                   // PCMM_Scheme.cuh:16-18 sizes its table for 3072
        CKKS_HIP_TRY(hipMalloc((void**)&h->d_ptrs, (size_t)cap * sizeof(uint64_t*)));
        h->ptr_cap = cap;
    }
    CKKS_HIP_TRY(hipMemcpyAsync(h->d_ptrs, host_ptrs, (size_t)count * sizeof(uint64_t*), hipMemcpyHostToDevice, h->ctx->stream));
    return CKKS_OK;
}

extern "C" int pcmm_rlwe_decompose(pcmm_ctx* h, const uint64_t* rlwe, uint64_t* const* mlwe_ptrs_host, int mlwe_num, int l) {
    if (!h || !rlwe || !mlwe_ptrs_host) return CKKS_E_INVALID;
    ckks_ctx* c = h->ctx;
    if (mlwe_num > h->rank) { set_error("rlweCipherDecompose extract number must be <= mlwe_rank"); return CKKS_E_INVALID; }   // PCMM_Scheme.cuh:103-106
    if (mlwe_num <= 0 || l < 0 || l > c->L) { set_error("rlweCipherDecompose: bad mlwe_num or level"); return CKKS_E_INVALID; }
    int rc = upload_ptrs(h, mlwe_ptrs_host, mlwe_num);
    if (rc) return rc;
    GatherArgs a;
    a.rlwe = rlwe; a.mlwe = h->d_ptrs; a.primes = c->d_primes; a.N = c->N; a.N1 = h->N1; a.rank = h->rank; a.mlwe_num = mlwe_num;
    a.L = c->L; a.p_num = c->p_num;
    const int k = h->rank;
    const bool force_plain = h->gather_plain;                                     // test hook: the one-lane-per-word kernel
    // 16-word row segments (one 128-byte line) when the window fits the LDS a workgroup may ask for, else 8-word segments
    static const bool big_lds = hipFuncSetAttribute(reinterpret_cast<const void*>(rlwe_gather_tiled_kernel<16>),
                                                    hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024) == hipSuccess;
    const size_t lds_cap = big_lds ? 96 * 1024 : 64 * 1024;
    const int G = (h->N1 % 16 == 0 && (size_t)17 * (k + 1) * 8 <= lds_cap) ? 16 : 8;
    if (!force_plain && h->N1 % G == 0 && k % mlwe_num == 0 && (size_t)(G + 1) * (k + 1) * 8 <= (G == 16 ? lds_cap : 64 * 1024)) {
        dim3 grid(h->N1 / G, l + 1, (mlwe_num + GATHER_M_CHUNK - 1) / GATHER_M_CHUNK), block(256);
        const size_t lds = (size_t)(G + 1) * (k + 1) * sizeof(u64);
        if (G == 16) hipLaunchKernelGGL(rlwe_gather_tiled_kernel<16>, grid, block, lds, c->stream, a);
        else hipLaunchKernelGGL(rlwe_gather_tiled_kernel<8>, grid, block, lds, c->stream, a);
    } else {
        long per = (long)(h->rank + 1) * h->N1;
        dim3 grid((unsigned)((per + 255) / 256), l + 1, mlwe_num), block(256);
        hipLaunchKernelGGL(rlwe_gather_kernel, grid, block, 0, c->stream, a);
    }
    CKKS_HIP_TRY(hipGetLastError());
    // the pointer table was copied asynchronously from the caller's host array: make sure it is consumed before returning
    CKKS_HIP_TRY(hipStreamSynchronize(c->stream));
    return CKKS_OK;
}
extern "C" int pcmm_rlwe_decompose_ntt(pcmm_ctx* h, uint64_t* rlwe, uint64_t* const* mlwe_ptrs_host, int mlwe_num, int l) {
    if (!h || !rlwe) return CKKS_E_INVALID;
    ckks_ctx* c = h->ctx;
    if (l < 0 || l > c->L) { set_error("rlweCipherDecompose: bad level"); return CKKS_E_INVALID; }
    int rc = launch_ntt(c, rlwe, 0, c->K, 2, l + 1, c->L + 1, 0, 1, true);             // PCMM_Scheme.cuh:107
    if (rc) return rc;
    if ((rc = pcmm_rlwe_decompose(h, rlwe, mlwe_ptrs_host, mlwe_num, l))) return rc;
    return launch_ntt(c, rlwe, 0, c->K, 2, l + 1, c->L + 1, 0, 1, false);              // :124
}


// ------------------------------------------------------------------------------------------------------------
// MLWE -> RLWE packing: PCMM_Scheme::mlweCipherPacking (PCMM_Scheme.cuh:361-425)
//   embed  : k+1 big polynomials over [p0, q0]; coefficient n*k + m*gap of big polynomial i is coefficient n of row i of MLWE
//            sample m (zero elsewhere), lifted to p0 around zero (mlweCipherEmbedding_new_kernel, :309-340)
//   NTT of the k "a" polynomials, inner product with the k repacking keys (mlweCipherMultRepackingKey_kernel, :262-289),
//   iNTT, division by p0 (ringpacking_ModDown_kernel, :291-306), + (0, b), NTT.
// All three kernels stream: one pass over their inputs, coalesced on both sides.
// ------------------------------------------------------------------------------------------------------------
struct EmbedArgs {
    const u64* const* mlwe;       // mlwe_num pointers, each [(k+1)][N1] (one modulus)
    u64* embed;                   // [(k+1)][2][N]
    long N;
    int N1, rank, mlwe_num, first_poly;
    u64 p0, q0;
};
constexpr int EMBED_ROWS = 8;     // coefficients n of the small ring per workgroup
__global__ __launch_bounds__(256) void mlwe_embed_kernel(EmbedArgs a) {
    extern __shared__ u64 tile[];                       // [EMBED_ROWS][rank]
    const int k = a.rank, i = blockIdx.y + a.first_poly, n0 = blockIdx.x * EMBED_ROWS, gap = k / a.mlwe_num;
    for (int t = threadIdx.x; t < EMBED_ROWS * k; t += 256) tile[t] = 0;
    __syncthreads();
    // 8 lanes read 64 contiguous bytes of one sample; the tile turns (sample, n) into (n, position inside the big coefficient group)
    for (int t = threadIdx.x; t < EMBED_ROWS * a.mlwe_num; t += 256) {
        const int m = t / EMBED_ROWS, j = t % EMBED_ROWS;
        tile[j * k + m * gap] = a.mlwe[m][(long)i * a.N1 + n0 + j];
    }
    __syncthreads();
    u64* big = a.embed + (long)i * 2 * a.N;
    for (int t = threadIdx.x; t < EMBED_ROWS * k; t += 256) {
        const u64 v = tile[t];
        const long pos = (long)n0 * k + t;              // (n0 + t / k) * k + t % k
        big[a.N + pos] = v;                                                         // mod q0
        u64 lifted = v;                                                             // mod p0, lifted around zero (:335-339)
        if (v > a.q0 / 2) {
            lifted = a.p0 - (a.q0 - v);
            if (a.q0 / 2 >= a.p0) lifted %= a.p0;                                   // the reference's `% p0`; the identity when q0 / 2 < p0
        }
        big[pos] = lifted;
    }
}

struct RepackArgs {
    const u64* embed;             // [(k+1)][2][N], the first k polynomials in NTT form
    const u64* keys;              // [k][a: 2 limbs | b: 2 limbs][N]
    u64* acc;                     // [2][2][N]
    u64* rlwe;                    // [a: L+1 limbs | b: L+1 limbs]
    const PrimeConst* pq;         // ring-pack primes [p0, q0, ...]
    long N;
    int rank, L;
    u64 pinv, pinv_s;             // p0^-1 mod q0 and its Shoup word
};
__global__ __launch_bounds__(256) void repack_mult_kernel(RepackArgs a) {
    const long x = (long)blockIdx.x * 256 + threadIdx.x;
    const int im = blockIdx.y;
    const PrimeConst pr = a.pq[im];
    u128w sa = {0, 0}, sb = {0, 0};
    const u64* e = a.embed + (long)im * a.N + x;
    const u64* ka = a.keys + (long)im * a.N + x;
    const u64* kb = ka + 2 * a.N;
#pragma unroll 4
    for (int i = 0; i < a.rank; i++) {
        const u64 c = e[(long)i * 2 * a.N];
        mac128(sa, c, ka[(long)i * 4 * a.N]);
        mac128(sb, c, kb[(long)i * 4 * a.N]);
    }
    a.acc[(long)im * a.N + x] = barrett128(sa, pr.q, pr.mu_hi, pr.mu_lo);
    a.acc[(long)(2 + im) * a.N + x] = barrett128(sb, pr.q, pr.mu_hi, pr.mu_lo);
}
__global__ __launch_bounds__(256) void repack_moddown_kernel(RepackArgs a) {
    const long x = (long)blockIdx.x * 256 + threadIdx.x;
    const int y = blockIdx.y;
    const u64 q0 = a.pq[1].q;
    const u64* in = a.acc + (long)y * 2 * a.N;
    u64 ra = in[x] % q0;                                                            // :300
    ra = q0 - ra + in[a.N + x];
    u64 r = mul_shoup(ra, a.pinv, a.pinv_s, q0);
    if (y == 1) r = csub(r + a.embed[(long)a.rank * 2 * a.N + a.N + x], q0);        // + (0, b), poly_arithmetic.cuh:111-121
    a.rlwe[(long)y * a.N * (a.L + 1) + x] = r;
}

extern "C" int pcmm_mlwe_pack(pcmm_ctx* h, uint64_t* rlwe_out, const uint64_t* const* mlwe_ptrs_host, int mlwe_num,
                              const uint64_t* repacking_keys, uint64_t* embed_scratch, uint64_t* mult_scratch) {
    if (!h || !rlwe_out || !mlwe_ptrs_host || !repacking_keys || !embed_scratch || !mult_scratch) return CKKS_E_INVALID;
    ckks_ctx* c = h->ctx;
    const int k = h->rank, N1 = h->N1, K = c->K;
    if (h->np != 1 || h->nq != 2) {
        set_error("mlweCipherPacking: one special ring-pack prime and two ring-pack moduli are supported (the reference's embedding overlaps otherwise)");
        return CKKS_E_INVALID;
    }
    if (mlwe_num <= 0 || mlwe_num > k || k % mlwe_num || (long)N1 * k != c->N || N1 % EMBED_ROWS || K < 1 || c->N % 256) {
        set_error("mlweCipherPacking: bad mlwe_num or ring shape");
        return CKKS_E_INVALID;
    }
    if (c->pqt[K - 1] != h->pq[0] || c->pqt[K] != h->pq[1]) {
        set_error("mlweCipherPacking: the ring-pack primes must be the context's last special prime and q0");
        return CKKS_E_INVALID;
    }
    if ((size_t)EMBED_ROWS * k * sizeof(u64) > 64 * 1024) { set_error("mlweCipherPacking: rank too large"); return CKKS_E_INVALID; }
    int rc = upload_ptrs(h, mlwe_ptrs_host, mlwe_num);
    if (rc) return rc;
    EmbedArgs ea;
    ea.mlwe = (const u64* const*)h->d_ptrs; ea.embed = embed_scratch; ea.N = c->N; ea.N1 = N1; ea.rank = k; ea.mlwe_num = mlwe_num;
    ea.p0 = h->pq[0]; ea.q0 = h->pq[1];
    // Only the b polynomial is written out in coefficient form (the ModDown adds it at the end).  The k "a" polynomials are
    // needed in NTT form only: the first pass of their transform gathers them from the samples, which saves writing and
    // re-reading 2 k limbs (a quarter of this entry point's memory traffic).
    ea.first_poly = k;
    hipLaunchKernelGGL(mlwe_embed_kernel, dim3(N1 / EMBED_ROWS, 1), dim3(256), (size_t)EMBED_ROWS * k * sizeof(u64), c->stream, ea);
    NttEmbedSource src;
    src.mlwe = (const uint64_t* const*)h->d_ptrs; src.p0 = h->pq[0]; src.q0 = h->pq[1]; src.n1 = N1;
    src.logk = 0; while ((1 << src.logk) < k) src.logk++;
    src.loggap = 0; while ((mlwe_num << src.loggap) < k) src.loggap++;
    RepackArgs ra;
    ra.embed = embed_scratch; ra.keys = repacking_keys; ra.acc = mult_scratch; ra.rlwe = rlwe_out; ra.pq = h->d_pq; ra.N = c->N;
    ra.rank = k; ra.L = c->L;
    ra.pinv = H::invmod(h->pq[0] % h->pq[1], h->pq[1]); ra.pinv_s = H::shoup(ra.pinv, h->pq[1]);
    bool fused = false;
    if ((rc = launch_repack_front_fused(c, embed_scratch, mult_scratch, repacking_keys, k, K - 1, src, &fused))) return rc;
    if (!fused) {
        if ((rc = launch_ntt_embedded(c, embed_scratch, 0, K - 1, k, 2, 2, src))) return rc;       // :389
        hipLaunchKernelGGL(repack_mult_kernel, dim3((unsigned)(c->N / 256), 2), dim3(256), 0, c->stream, ra);
    }
    if ((rc = launch_ntt(c, mult_scratch, 0, K - 1, 2, 2, 2, 0, 1, true))) return rc;              // :405
    hipLaunchKernelGGL(repack_moddown_kernel, dim3((unsigned)(c->N / 256), 2), dim3(256), 0, c->stream, ra);
    CKKS_HIP_TRY(hipGetLastError());
    if ((rc = launch_ntt(c, rlwe_out, 0, K, 2, 1, c->L + 1, 0, 1, false))) return rc;              // :419
    CKKS_HIP_TRY(hipStreamSynchronize(c->stream));      // the pointer table came from the caller's host array
    return CKKS_OK;
}


// ------------------------------------------------------------------------------------------------------------
// size-N1 transforms over the ring-pack primes: PCMM_Context::ToNTTInplace / FromNTTInplace (PCMM_Context.cuh:243-273,
// kernels smallntt_60bit.cuh:7-152).  Same negacyclic transform, root rule and table convention as the big ring.  For
// N1 >= 256 the big ring's kernels run it from a table set built for N1; the reference's layout [batch][mod][poly][N1] is
// one launch per (batch, modulus) with poly_mod_len = 1.  For N1 < 256 (the BERT layer runs N1 = 128 = token count) a
// wave per polynomial runs all stages in LDS.  The reference runs N1 = 256 only and returns without work otherwise (:256,271).
// ------------------------------------------------------------------------------------------------------------
struct SmallRingArgs {
    u64* data;
    const u64* tw;                // [ring-pack prime][forward | inverse][N1]: psi_table / psiinv_table of the size-N1 ring
    const PrimeConst* pq;
    long polys;                   // batch * mod_num * poly_num
    int N1, poly_num, mod_num, start_mod, inverse;
    u64 n_inv[8];
};
__device__ __forceinline__ u64 small_mulmod(u64 a, u64 b, const PrimeConst& p) {
    u128w acc{0, 0};
    mac128(acc, a, b);
    return barrett128(acc, p.q, p.mu_hi, p.mu_lo);
}
__global__ __launch_bounds__(256) void small_ring_ntt_kernel(SmallRingArgs a) {
    __shared__ u64 buf[4][128];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const long poly = (long)blockIdx.x * 4 + wave;
    const bool live = poly < a.polys;
    const int n = a.N1, half = n >> 1;
    const int j = live ? (int)((poly / a.poly_num) % a.mod_num) : 0;
    const PrimeConst p = a.pq[a.start_mod + j];
    const u64* tw = a.tw + ((size_t)(a.start_mod + j) * 2 + (a.inverse ? 1 : 0)) * n;
    u64* x = a.data + (live ? poly : 0) * n;
    u64* b = buf[wave];
    if (live)
        for (int i = lane; i < n; i += 64) b[i] = x[i];
    __syncthreads();
    const bool work = live && lane < half;
    if (!a.inverse) {
        for (int m = 1, t = half; m < n; m <<= 1, t >>= 1) {
            if (work) {
                const int i = lane / t, lo = 2 * i * t + lane % t;
                const u64 U = b[lo], V = small_mulmod(b[lo + t], tw[m + i], p);
                b[lo] = csub(U + V, p.q);
                b[lo + t] = csub(U + p.q - V, p.q);
            }
            __syncthreads();
        }
    } else {
        for (int h = half, t = 1; h >= 1; h >>= 1, t <<= 1) {
            if (work) {
                const int i = lane / t, lo = 2 * i * t + lane % t;
                const u64 U = b[lo], V = b[lo + t];
                const u64 s = csub(U + V, p.q), d = csub(U + p.q - V, p.q);
                b[lo] = h == 1 ? small_mulmod(s, a.n_inv[a.start_mod + j], p) : s;
                b[lo + t] = small_mulmod(d, tw[h + i], p);            // the table's entry 1 already carries N1^-1 (Utils.cuh:200)
            }
            __syncthreads();
        }
    }
    if (live)
        for (int i = lane; i < n; i += 64) x[i] = b[i];
}

static int pcmm_tiny_ntt(pcmm_ctx* h, int logN1, uint64_t* data, int poly_num, int mod_num, int start_mod_idx, int mod_batch_size, bool inverse) {
    const int n = h->N1, tot = h->np + h->nq;
    if (logN1 < 1 || tot > 8) { set_error("PCMM NTT: N1 must be at least 2 and at most 8 ring-pack primes"); return CKKS_E_INVALID; }
    if (!h->d_small_tw) {
        std::vector<u64> tab((size_t)tot * 2 * n);
        for (int i = 0; i < tot; i++) {
            const u64 q = h->pq[i];
            if ((q - 1) % (2 * (u64)n)) { set_error("PCMM NTT: a ring-pack prime is not 1 modulo 2 * N1"); return CKKS_E_INVALID; }
            const u64 psi = H::mth_root(2 * (u64)n, q), psiinv = H::invmod(psi, q);
            u64 pw = 1, ipw = 1;
            for (int k = 0; k < n; k++) {                                  // fillTablePsi128_special (Utils.cuh:190-201)
                const uint32_t r = H::bitrev((uint32_t)k, logN1);
                tab[((size_t)i * 2 + 0) * n + r] = pw;
                tab[((size_t)i * 2 + 1) * n + r] = ipw;
                pw = H::mulmod(pw, psi, q);
                ipw = H::mulmod(ipw, psiinv, q);
            }
            h->small_n_inv[i] = H::invmod((u64)n % q, q);
            tab[((size_t)i * 2 + 1) * n + 1] = H::mulmod(tab[((size_t)i * 2 + 1) * n + 1], h->small_n_inv[i], q);
        }
        CKKS_HIP_TRY(hipMalloc((void**)&h->d_small_tw, tab.size() * sizeof(u64)));
        CKKS_HIP_TRY(hipMemcpy(h->d_small_tw, tab.data(), tab.size() * sizeof(u64), hipMemcpyHostToDevice));
    }
    SmallRingArgs a;
    a.data = (u64*)data; a.tw = h->d_small_tw; a.pq = h->d_pq;
    a.polys = (long)mod_batch_size * mod_num * poly_num;
    a.N1 = n; a.poly_num = poly_num; a.mod_num = mod_num; a.start_mod = start_mod_idx; a.inverse = inverse ? 1 : 0;
    for (int i = 0; i < 8; i++) a.n_inv[i] = i < tot ? h->small_n_inv[i] : 0;
    hipLaunchKernelGGL(small_ring_ntt_kernel, dim3((unsigned)((a.polys + 3) / 4)), dim3(256), 0, h->ctx->stream, a);
    CKKS_HIP_TRY(hipGetLastError());
    return CKKS_OK;
}

static int pcmm_small_ntt(pcmm_ctx* h, uint64_t* data, int poly_num, int mod_num, int start_mod_idx, int mod_batch_size, bool inverse) {
    if (!h || !data) return CKKS_E_INVALID;
    if (poly_num <= 0 || mod_num <= 0 || mod_batch_size <= 0) return CKKS_OK;
    if (start_mod_idx < 0 || start_mod_idx + mod_num > h->np + h->nq) { set_error("PCMM NTT: modulus range outside the ring-pack primes"); return CKKS_E_INVALID; }
    int logN1 = 0;
    while ((1 << logN1) < h->N1) logN1++;
    if ((1 << logN1) != h->N1) { set_error("PCMM NTT: N1 must be a power of two"); return CKKS_E_INVALID; }
    if (logN1 < 8) return pcmm_tiny_ntt(h, logN1, data, poly_num, mod_num, start_mod_idx, mod_batch_size, inverse);
    if (!h->small) {
        int rc = ckks_ctx_create(&h->small, logN1, nullptr, 0, h->pq.data(), h->np + h->nq, nullptr, 0, 0);
        if (rc) return rc;
    }
    h->small->stream = h->ctx->stream;
    for (int z = 0; z < mod_batch_size; z++)
        for (int j = 0; j < mod_num; j++) {
            uint64_t* base = data + ((size_t)z * mod_num + j) * poly_num * h->N1;
            int rc = launch_ntt(h->small, base, 0, start_mod_idx + j, poly_num, 1, 1, 0, 1, inverse);
            if (rc) return rc;
        }
    return CKKS_OK;
}
extern "C" int pcmm_ntt_fwd(pcmm_ctx* h, uint64_t* data, int poly_num, int mod_num, int start_poly_idx, int start_mod_idx, int mod_batch_size) {
    (void)start_poly_idx;                  // carried for the reference's signature; its kernels do not use it (smallntt_60bit.cuh:27-29)
    return pcmm_small_ntt(h, data, poly_num, mod_num, start_mod_idx, mod_batch_size, false);
}
extern "C" int pcmm_ntt_inv(pcmm_ctx* h, uint64_t* data, int poly_num, int mod_num, int start_poly_idx, int start_mod_idx, int mod_batch_size) {
    (void)start_poly_idx;
    return pcmm_small_ntt(h, data, poly_num, mod_num, start_mod_idx, mod_batch_size, true);
}

// Small host arrays (row-pointer table, epilogue constants) go to the device through a pinned staging area owned by the handle:
// the copy is asynchronous for real and the caller's memory is free on return.  The area is reused, so a second upload first
// waits for the first one's copy (an event, not the stream).
static int stage_to_device(pcmm_ctx* h, void* dst, const void* src, size_t bytes) {
    if (!h->pin_ev) CKKS_HIP_TRY(hipEventCreateWithFlags(&h->pin_ev, hipEventDisableTiming));
    else CKKS_HIP_TRY(hipEventSynchronize(h->pin_ev));
    if (bytes > h->pin_cap) {
        if (h->pin) (void)hipHostFree(h->pin);
        h->pin = nullptr; h->pin_cap = 0;
        const size_t cap = std::max(bytes, (size_t)64 * 1024);
        CKKS_HIP_TRY(hipHostMalloc(&h->pin, cap, hipHostMallocDefault));
        h->pin_cap = cap;
    }
    memcpy(h->pin, src, bytes);
    CKKS_HIP_TRY(hipMemcpyAsync(dst, h->pin, bytes, hipMemcpyHostToDevice, h->ctx->stream));
    CKKS_HIP_TRY(hipEventRecord(h->pin_ev, h->ctx->stream));
    return CKKS_OK;
}
uint64_t** pcmm_ctx::d_ptrs_slot(int count) {
    if (count > ptr_cap) {
        if (d_ptrs) { (void)hipDeviceSynchronize(); (void)hipFree(d_ptrs); d_ptrs = nullptr; ptr_cap = 0; }
        const int cap = std::max(count, 3072);                             // PCMM_Scheme.cuh:16-18 sizes its table for 3072
        if (hipMalloc((void**)&d_ptrs, (size_t)cap * sizeof(uint64_t*)) != hipSuccess) return nullptr;
        ptr_cap = cap;
        tab_sent.clear();
    }
    return d_ptrs;
}
// prepared plaintext matrices: at most WEIGHTS_MAX_BYTES of device memory, least recently used first out
constexpr size_t WEIGHTS_MAX_BYTES = (size_t)4 << 30;
static void drop_weights(pcmm_ctx* h, pcmm_ctx::Weights* w) {
    (void)hipStreamSynchronize(h->ctx->stream);
    if (w->d_A) (void)hipFree(w->d_A);
    if (w->d_Adig) (void)hipFree(w->d_Adig);
    const size_t idx = (size_t)(w - h->weights.data());
    if (idx < h->weights.size()) {
        h->weights_bytes -= w->bytes;
        h->weights.erase(h->weights.begin() + (long)idx);
    }
}
void pcmm_forget_weights(const void* lo, size_t bytes, bool freed) {
    std::lock_guard<std::mutex> lock(g_handles_mutex);
    const uintptr_t a = (uintptr_t)lo, b = a + bytes;
    for (pcmm_ctx* h : g_handles) {
        if (freed)                                        // memory that goes back to the allocator is nobody's static matrix any more
            for (size_t i = h->static_ranges.size(); i-- > 0;)
                if (h->static_ranges[i].first < b && a < h->static_ranges[i].first + h->static_ranges[i].second)
                    h->static_ranges.erase(h->static_ranges.begin() + (long)i);
        for (size_t i = h->weights.size(); i-- > 0;) {
            const uintptr_t wa = (uintptr_t)h->weights[i].W, wb = wa + (size_t)h->weights[i].M * h->weights[i].Kin * sizeof(float);
            if (wa < b && a < wb) drop_weights(h, &h->weights[i]);
        }
    }
}
// whether the prepared form of the matrix at W is kept between calls
static bool weights_kept(const pcmm_ctx* h, const float* W) {
    if (h->weights_cached) return true;
    const uintptr_t a = (uintptr_t)W;
    for (const auto& r : h->static_ranges) if (a >= r.first && a < r.first + r.second) return true;
    return false;
}
static pcmm_ctx::Weights* keep_weights(pcmm_ctx* h, const pcmm_ctx::Weights& fresh) {
    while (!h->weights.empty() && h->weights_bytes + fresh.bytes > WEIGHTS_MAX_BYTES) {
        size_t old = 0;
        for (size_t i = 1; i < h->weights.size(); i++) if (h->weights[i].stamp < h->weights[old].stamp) old = i;
        drop_weights(h, &h->weights[old]);
    }
    h->weights.push_back(fresh);
    h->weights_bytes += fresh.bytes;
    return &h->weights.back();
}

static int ppmm_common(pcmm_ctx* h, const float* W, const uint64_t* const* ptrs_host, const uint64_t* strided, uint64_t* out,
                       int M, int Kin, int mod_num, double scaler, bool packed = false) {
    if (!h || !W || !out || (!ptrs_host && !strided && !packed)) return CKKS_E_INVALID;
    if (M <= 0 || Kin <= 0 || mod_num < 1 || mod_num > h->nq || mod_num > 64) { set_error("PPMM: bad shape or mod_num"); return CKKS_E_INVALID; }
    ckks_ctx* c = h->ctx;
    const long C = (long)(h->rank + 1) * h->N1;
    int rc;
    // Row-pointer table on the device, padded to Kpad entries: rows of the K padding point to a zero buffer, so the dense
    // kernel needs no bounds checks along K.  A contiguous operand goes through a generated table.
    const int Kpad_tab = (Kin + 191) / 192 * 192;
    size_t zero_words = (size_t)mod_num * C;
    if (!packed && Kpad_tab > Kin && zero_words > h->zero_cap) {
        if (h->d_zero) { (void)hipDeviceSynchronize(); (void)hipFree(h->d_zero); h->d_zero = nullptr; }
        CKKS_HIP_TRY(hipMalloc((void**)&h->d_zero, zero_words * sizeof(uint64_t)));
        CKKS_HIP_TRY(hipMemset(h->d_zero, 0, zero_words * sizeof(uint64_t)));
        h->zero_cap = zero_words;
    }
    bool aligned16 = true;
    if (!packed) {
        std::vector<const uint64_t*> tab(Kpad_tab);
        for (int n = 0; n < Kpad_tab; n++)
            tab[n] = n >= Kin ? h->d_zero : (ptrs_host ? ptrs_host[n] : strided + (size_t)n * mod_num * C);
        for (int n = 0; n < Kin; n++) aligned16 = aligned16 && (((uintptr_t)tab[n]) & 15) == 0;
        if (tab != h->tab_sent) {                           // a layer calls with the same sample buffers again and again
            uint64_t** slot = h->d_ptrs_slot(Kpad_tab);
            if (!slot) { set_error("PPMM: cannot allocate the row-pointer table"); return CKKS_E_NOMEM; }
            if ((rc = stage_to_device(h, slot, tab.data(), (size_t)Kpad_tab * sizeof(uint64_t*)))) return rc;
            h->tab_sent = tab;
        }
    }
    const int Mpad = (M + 127) / 128 * 128, Kpad = (Kin + 191) / 192 * 192;   // K padded to a multiple of three 64-deep MFMA steps (LDS ring of three slots)
    // per-call epilogue constants, kept behind the |A| maximum word; they depend on mod_num only
    uint64_t qmax = 0, qmin = ~0ull;
    for (int i = 0; i < mod_num; i++) { qmax = std::max(qmax, h->pq[h->np + i]); qmin = std::min(qmin, h->pq[h->np + i]); }
    uint64_t* d_cst = (uint64_t*)(h->d_absmax + 1);
    if (h->cst_mods != mod_num) {
        std::vector<uint64_t> cst(PPMM_CONST_WORDS, 0);
        const uint64_t qlast = h->pq[h->np + mod_num - 1];
        auto dbits = [](uint64_t x, uint64_t m) { double d = x > m / 2 ? -(double)(m - x) : (double)x; uint64_t b; memcpy(&b, &d, 8); return b; };
        for (int i = 0; i < mod_num; i++) {
            uint64_t qi = h->pq[h->np + i];
            if (i < mod_num - 1) {
                cst[i] = H::invmod(qlast % qi, qi);
                cst[PPMM_MAX_MODS + i] = H::shoup(cst[i], qi);
                cst[4 * PPMM_MAX_MODS + i] = dbits(cst[i], qi);
            }
            cst[2 * PPMM_MAX_MODS + i] = dbits(H::powmod(2, 32, qi), qi);
            cst[3 * PPMM_MAX_MODS + i] = dbits(H::powmod(2, 64, qi), qi);
        }
        if ((rc = stage_to_device(h, d_cst, cst.data(), PPMM_CONST_WORDS * sizeof(uint64_t)))) return rc;
        h->cst_mods = mod_num;
    }
    // digit counts.  d balanced digits in [-128, 127] reach from -0x80..80 up to +0x7f..7f (d bytes each), NOT up to 2^(8d-1) - 1:
    // the bytes of x + 0x80..80 must not carry into byte d.  DW digits must hold +-|A|max, DC digits every residue 0 .. qmax - 1.
    auto top = [](int d) { unsigned long long v = 0; for (int i = 0; i < d; i++) v = (v << 8) | 0x7f; return v; };
    int DC = 1; while (DC < 8 && qmax - 1 > top(DC)) DC++;
    const bool force_generic = h->ppmm_generic;                                   // test hook: exercise the generic kernel
    // what the matrix of a given |A|max runs on.  Residues in 5 digits (q < 2^39) with up to 4 plaintext digits, or in 7 digits
    // (q < 2^50) with up to 3; wider plaintext matrices (any int64) go through the same kernels in slices of three digits.
    struct Plan { int DW, slices, planes; bool mfma; };
    auto plan_for = [&](unsigned long long absmax) {
        Plan pl;
        pl.DW = 1; while (pl.DW < 8 && absmax > top(pl.DW)) pl.DW++;
        const bool one_launch = (DC <= 5 && pl.DW <= 4) || (DC <= 7 && qmax < (1ull << 50) && pl.DW <= 3);
        pl.slices = one_launch ? 1 : (pl.DW + 2) / 3;
        const bool width_ok = (DC <= 5 || (DC <= 7 && qmax < (1ull << 50))) && pl.slices <= 3;
        pl.mfma = !force_generic && aligned16 && (C % 64 == 0) && width_ok &&
                  (long)Kpad * (pl.slices == 1 && pl.DW == 4 ? 4 : 3) <= 16384 && absmax < qmin && qmin > (1ull << 25);
        // every plane the kernel instance reads is written (3 or 4: the instances are built for these widths), also those above the
        // measured digit count, which are zero for this matrix
        pl.planes = pl.slices > 1 ? 3 * pl.slices : pl.DW <= 3 ? 3 : 4;
        return pl;
    };
    // The plaintext matrix as the kernels take it (quantised; for the MFMA kernel split into digit planes).  By default it is made
    // anew in every call, in work space of the handle - the reference quantises W inside every call (PPMM_kernel.cuh:148), so
    // whatever the caller has written to W since the last call is what this call multiplies by.  For a matrix the caller has
    // declared static (pcmm_weights_static), or every matrix with pcmm_set_weight_cache(h, 1) - the caller's promise that W changes
    // only through this library's copies or with pcmm_weights_changed - the prepared form is kept under (device address, shape,
    // scaler) and found again here.
    pcmm_ctx::Weights* we = nullptr;
    const bool keep = weights_kept(h, W);
    if (keep)
        for (auto& w : h->weights)
            if (w.W == W && w.M == M && w.Kin == Kin && w.scaler == scaler) { we = &w; break; }
    if (we) {
        const Plan pl = plan_for(we->absmax);
        if (pl.mfma ? !we->d_Adig || we->planes != pl.planes : !we->d_A) { drop_weights(h, we); we = nullptr; }   // prepared for the other kernel
    }
    pcmm_ctx::Weights fresh;
    bool packed_early = false;
    if (!we) {
        const long count = (long)M * Kin;
        fresh.W = W; fresh.M = M; fresh.Kin = Kin; fresh.scaler = scaler;
        // work space of a call that keeps nothing: grown when a call needs more, reused in stream order otherwise (a call on another
        // stream than the last waits for the device first)
        auto work = [&](void** slot, size_t* cap, size_t need) -> hipError_t {
            if (need <= *cap) return hipSuccess;
            if (*slot) { (void)hipDeviceSynchronize(); (void)hipFree(*slot); *slot = nullptr; *cap = 0; }
            hipError_t e = hipMalloc(slot, need);
            if (e == hipSuccess) *cap = need;
            return e;
        };
        if (!keep && h->work_stream_known && h->work_stream != c->stream) (void)hipDeviceSynchronize();
        h->work_stream = c->stream; h->work_stream_known = true;
        hipError_t e = keep ? hipMalloc((void**)&fresh.d_A, (size_t)count * sizeof(long long))
                            : work((void**)&h->d_workA, &h->workA_cap, (size_t)count * sizeof(long long));
        if (e != hipSuccess) { set_error("PPMM: cannot allocate the quantised plaintext matrix"); return CKKS_E_NOMEM; }
        if (!keep) fresh.d_A = h->d_workA;
        auto release = [&]() { if (keep && fresh.d_A) (void)hipFree(fresh.d_A); };
        (void)hipMemsetAsync(h->d_absmax, 0, sizeof(unsigned long long), c->stream);
        hipLaunchKernelGGL(quantise_kernel, dim3((unsigned)((count + 256 * QUANT_PER_LANE - 1) / (256 * QUANT_PER_LANE))), dim3(256), 0, c->stream, W,
                           fresh.d_A, h->d_absmax, count, scaler);
        // The one host round trip of a matrix: its digit count selects the kernel instance.  The host waits for the copy alone (an event
        // behind it), and where the MFMA path is in reach the pack pass of the residues, which does not depend on the matrix, is
        // already queued behind the copy: the GPU works through it while the answer travels.
        hipError_t e2 = hipSuccess;
        if (!h->h_absmax) e2 = hipHostMalloc((void**)&h->h_absmax, sizeof(unsigned long long), hipHostMallocDefault);
        if (e2 == hipSuccess && !h->ev_absmax) e2 = hipEventCreateWithFlags(&h->ev_absmax, hipEventDisableTiming);
        if (e2 == hipSuccess) e2 = hipMemcpyAsync(h->h_absmax, h->d_absmax, sizeof(unsigned long long), hipMemcpyDeviceToHost, c->stream);
        if (e2 == hipSuccess) e2 = hipEventRecord(h->ev_absmax, c->stream);
        if (e2 != hipSuccess) { release(); return hip_fail(e2, "PPMM: |A| maximum"); }
        if (!packed && !force_generic && aligned16 && (C % 64 == 0) && (DC <= 5 || (DC <= 7 && qmax < (1ull << 50))) && (long)Kpad * 3 <= 16384 &&
            qmin > (1ull << 25)) {
            PpmmArgs pa;
            pa.A = nullptr; pa.Adig = nullptr; pa.mlwe = (const u64* const*)h->d_ptrs; pa.mlwe_base = nullptr; pa.mlwe_stride = (long)mod_num * C;
            pa.out = out; pa.pq = h->d_pq; pa.consts = d_cst; pa.C = C; pa.M = M; pa.Kin = Kin; pa.Mpad = Mpad; pa.Kpad = Kpad; pa.mod_num = mod_num;
            pa.np = h->np; pa.raw_all = 0;
            const size_t need = ppmm_bdig_bytes(pa, DC);
            bool room = need <= h->Bdig_cap;
            if (!room) {
                if (h->d_Bdig) { (void)hipDeviceSynchronize(); (void)hipFree(h->d_Bdig); h->d_Bdig = nullptr; h->Bdig_cap = 0; }
                if (hipMalloc((void**)&h->d_Bdig, need) == hipSuccess) { h->Bdig_cap = need; room = true; }
                else (void)hipGetLastError();                 // the later, checked allocation reports it
            }
            if (room) {
                h->packed_K = h->packed_mods = 0;             // the planes now hold this call's operands
                if ((rc = launch_ppmm_pack(c->stream, pa, DC, h->d_Bdig))) { release(); return rc; }
                packed_early = true;
            }
        }
        e2 = hipEventSynchronize(h->ev_absmax);
        if (e2 != hipSuccess) { release(); return hip_fail(e2, "PPMM: |A| maximum"); }
        fresh.absmax = *h->h_absmax;
        const Plan pl = plan_for(fresh.absmax);
        if (packed && !pl.mfma) { release(); set_error("PPMM on digit planes: the plaintext matrix or the primes are outside what the MFMA kernel takes"); return CKKS_E_INVALID; }
        fresh.bytes = (size_t)count * sizeof(long long);
        if (pl.mfma) {
            const size_t dbytes = (size_t)pl.planes * Mpad * Kpad;
            e = keep ? hipMalloc((void**)&fresh.d_Adig, dbytes) : work((void**)&h->d_workAdig, &h->workAdig_cap, dbytes);
            if (e != hipSuccess) { release(); set_error("PPMM: cannot allocate the plaintext digit planes"); return CKKS_E_NOMEM; }
            if (!keep) fresh.d_Adig = h->d_workAdig;
            const long total = (long)Mpad * Kpad;
            hipLaunchKernelGGL(digits_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, c->stream, fresh.d_A, fresh.d_Adig, M, Kin, Mpad, Kpad, pl.planes);
            fresh.planes = pl.planes;
            if (keep) {
                (void)hipFree(fresh.d_A);                   // waits for the kernel above; only the planes are kept
                fresh.d_A = nullptr;
            }
            fresh.bytes = dbytes;
        }
        we = keep ? keep_weights(h, fresh) : &fresh;
    }
    we->stamp = ++h->weights_clock;
    const Plan pl = plan_for(we->absmax);
    const unsigned long long absmax = we->absmax;
    const int DW = pl.DW, slices = pl.slices;
    const bool mfma_ok = pl.mfma;

    PpmmArgs a;
    a.A = we->d_A; a.Adig = we->d_Adig; a.mlwe = (const u64* const*)h->d_ptrs; a.mlwe_base = nullptr;
    a.mlwe_stride = (long)mod_num * C; a.out = out; a.pq = h->d_pq; a.consts = d_cst; a.C = C; a.M = M; a.Kin = Kin;
    a.Mpad = Mpad; a.Kpad = Kpad; a.mod_num = mod_num; a.np = h->np; a.raw_all = 0; a.no_tail = h->ppmm_no_tail ? 1 : 0;
    if (packed && !mfma_ok) { set_error("PPMM on digit planes: the plaintext matrix or the primes are outside what the MFMA kernel takes"); return CKKS_E_INVALID; }
    h->last_path = mfma_ok ? 1 : 0; h->last_DW = DW; h->last_DC = DC; h->last_absmax = absmax; h->last_slices = mfma_ok ? slices : 0;
    if (mfma_ok) {
        size_t need = ppmm_bdig_bytes(a, DC);
        if (packed && need > h->Bdig_cap) { set_error("PPMM on digit planes: planes not opened for this shape"); return CKKS_E_STATE; }
        if (need > h->Bdig_cap) {
            if (h->d_Bdig) { (void)hipDeviceSynchronize(); (void)hipFree(h->d_Bdig); h->d_Bdig = nullptr; h->Bdig_cap = 0; }
            hipError_t e = hipMalloc((void**)&h->d_Bdig, need);
            if (e != hipSuccess) { set_error("PPMM: cannot allocate the residue digit planes"); return CKKS_E_NOMEM; }
            h->Bdig_cap = need;
        }
        if (!packed) h->packed_K = h->packed_mods = 0;     // the planes now hold this call's operands
        if (slices == 1) {
            rc = launch_ppmm_mfma_impl(c->stream, a, DW, DC, h->d_Bdig, !packed && !packed_early);
            if (rc) return rc;
        } else {
            const size_t per_slice = (size_t)M * mod_num * C;
            if ((slices - 1) * per_slice > h->slices_cap) {
                if (h->d_slices) { (void)hipDeviceSynchronize(); (void)hipFree(h->d_slices); h->d_slices = nullptr; h->slices_cap = 0; }
                hipError_t e = hipMalloc((void**)&h->d_slices, (slices - 1) * per_slice * sizeof(uint64_t));
                if (e != hipSuccess) { set_error("PPMM: cannot allocate the buffers of the plaintext slices"); return CKKS_E_NOMEM; }
                h->slices_cap = (slices - 1) * per_slice;
            }
            PpmmArgs sa = a;
            sa.raw_all = 1;
            for (int sl = 0; sl < slices; sl++) {
                sa.Adig = we->d_Adig + (size_t)3 * sl * Mpad * Kpad;
                sa.out = sl == 0 ? out : h->d_slices + (size_t)(sl - 1) * per_slice;
                rc = launch_ppmm_mfma_impl(c->stream, sa, 3, DC, h->d_Bdig, !packed && !packed_early && sl == 0);      // the residue planes are packed once
                if (rc) return rc;
            }
            PpmmCombineArgs ca;
            ca.out = out; ca.more = h->d_slices; ca.pq = h->d_pq; ca.consts = d_cst; ca.C = C; ca.per_slice = (long)per_slice;
            ca.M = M; ca.mod_num = mod_num; ca.np = h->np; ca.slices = slices;
            for (int i = 0; i < mod_num; i++) {
                const uint64_t qi = h->pq[h->np + i];
                ca.w[0][i] = H::powmod(2, 24, qi);
                ca.w[1][i] = H::powmod(2, 48, qi);
            }
            hipLaunchKernelGGL(ppmm_combine_kernel, dim3((unsigned)((C + 255) / 256), M), dim3(256), 0, c->stream, ca);
        }
    } else {
        dim3 grid((unsigned)((C + 255) / 256), M), block(256);
        hipLaunchKernelGGL(ppmm_generic_kernel, grid, block, 0, c->stream, a);
    }
    CKKS_HIP_TRY(hipGetLastError());
    return CKKS_OK;
}

extern "C" int pcmm_info(const pcmm_ctx* h, const char* name, long* value) {
    if (!h || !name || !value) return CKKS_E_INVALID;
    std::string n(name);
    if (n == "last_path") *value = h->last_path; else if (n == "last_DW") *value = h->last_DW; else if (n == "last_DC") *value = h->last_DC;
    else if (n == "last_slices") *value = h->last_slices;
    else if (n == "last_absmax") *value = (long)h->last_absmax; else if (n == "N1") *value = h->N1; else if (n == "mlwe_rank") *value = h->rank;
    else { set_error("pcmm_info: unknown name " + n); return CKKS_E_INVALID; }
    return CKKS_OK;
}
// test / tuning switches of a ring-pack handle, by name (value 0: off, anything else: on)
extern "C" int pcmm_set_option(pcmm_ctx* h, const char* name, long value) {
    if (!h || !name) return CKKS_E_INVALID;
    const std::string n(name);
    if (n == "gather_plain") h->gather_plain = value != 0;          // rlweCipherDecompose with the one-lane-per-word gather
    else if (n == "ppmm_generic") h->ppmm_generic = value != 0;     // PPMM on the generic 128-bit kernel instead of the MFMA one
    else if (n == "ppmm_no_tail") h->ppmm_no_tail = value != 0;     // PPMM runs the remainder column panels whole instead of as jobs by prime
    else { set_error("pcmm_set_option: unknown name " + n); return CKKS_E_INVALID; }
    return CKKS_OK;
}
extern "C" int pcmm_set_weight_cache(pcmm_ctx* h, int enabled) {
    if (!h) return CKKS_E_INVALID;
    h->weights_cached = enabled != 0;
    if (!enabled)                                         // what is kept from now on: the matrices declared static
        for (size_t i = h->weights.size(); i-- > 0;)
            if (!weights_kept(h, h->weights[i].W)) drop_weights(h, &h->weights[i]);
    return CKKS_OK;
}
extern "C" int pcmm_weights_static(pcmm_ctx* h, const float* W, size_t bytes, int is_static) {
    if (!h || !W || !bytes) return CKKS_E_INVALID;
    std::lock_guard<std::mutex> lock(g_handles_mutex);
    const uintptr_t a = (uintptr_t)W, b = a + bytes;
    for (size_t i = h->static_ranges.size(); i-- > 0;)
        if (h->static_ranges[i].first < b && a < h->static_ranges[i].first + h->static_ranges[i].second)
            h->static_ranges.erase(h->static_ranges.begin() + (long)i);
    if (is_static) h->static_ranges.emplace_back(a, bytes);
    else if (!h->weights_cached)
        for (size_t i = h->weights.size(); i-- > 0;) {
            const uintptr_t wa = (uintptr_t)h->weights[i].W;
            if (wa >= a && wa < b) drop_weights(h, &h->weights[i]);
        }
    return CKKS_OK;
}
extern "C" int pcmm_weights_changed(pcmm_ctx* h, const float* W) {
    if (!h) return CKKS_E_INVALID;
    for (size_t i = h->weights.size(); i-- > 0;)
        if (!W || h->weights[i].W == W) drop_weights(h, &h->weights[i]);
    return CKKS_OK;
}
extern "C" int pcmm_ppmm(pcmm_ctx* h, const float* W, const uint64_t* const* mlwe_ptrs_host, uint64_t* out, int M, int Kin, int mod_num, double scaler) {
    return ppmm_common(h, W, mlwe_ptrs_host, nullptr, out, M, Kin, mod_num, scaler);
}
extern "C" int pcmm_ppmm_strided(pcmm_ctx* h, const float* W, const uint64_t* mlwe, uint64_t* out, int M, int Kin, int mod_num, double scaler) {
    return ppmm_common(h, W, nullptr, mlwe, out, M, Kin, mod_num, scaler);
}

// ---- gather straight into the operand digit planes, and the contraction on them ----
extern "C" int pcmm_packed_begin(pcmm_ctx* h, int Kin, int mod_num) {
    if (!h) return CKKS_E_INVALID;
    ckks_ctx* c = h->ctx;
    const long C = (long)(h->rank + 1) * h->N1;
    if (Kin <= 0 || Kin % 64 || mod_num < 1 || mod_num > h->nq || mod_num > 64 || C % 64 || h->N1 % 16) {
        set_error("pcmm_packed_begin: Kin must be a positive multiple of 64, mod_num within the ring-pack moduli, N1 a multiple of 16");
        return CKKS_E_INVALID;
    }
    for (int i = 0; i < mod_num; i++)
        if (h->pq[h->np + i] - 1 > 0x7f7f7f7f7full) { set_error("pcmm_packed_begin: the digit planes hold residues up to 0x7f7f7f7f7f (primes just below 2^39)"); return CKKS_E_INVALID; }
    const int Kpad = (Kin + 191) / 192 * 192;
    const size_t need = (size_t)mod_num * Kpad * C * 5;
    if (need > h->Bdig_cap) {
        if (h->d_Bdig) { (void)hipDeviceSynchronize(); (void)hipFree(h->d_Bdig); h->d_Bdig = nullptr; h->Bdig_cap = 0; }
        hipError_t e = hipMalloc((void**)&h->d_Bdig, need);
        if (e != hipSuccess) { set_error("pcmm_packed_begin: cannot allocate the residue digit planes"); return CKKS_E_NOMEM; }
        h->Bdig_cap = need;
    }
    // K steps of the padding hold zero digits
    if (Kpad > Kin) {
        const size_t step = (size_t)C * 64 * 5;
        for (int im = 0; im < mod_num; im++)
            CKKS_HIP_TRY(hipMemsetAsync(h->d_Bdig + ((size_t)im * (Kpad / 64) + Kin / 64) * step, 0, (size_t)(Kpad - Kin) / 64 * step, c->stream));
    }
    h->packed_K = Kin; h->packed_mods = mod_num;
    return CKKS_OK;
}

extern "C" int pcmm_rlwe_decompose_packed(pcmm_ctx* h, uint64_t* rlwe, int sample_offset, int mlwe_num, int take, int l) {
    if (!h || !rlwe) return CKKS_E_INVALID;
    ckks_ctx* c = h->ctx;
    const int k = h->rank;
    if (h->packed_K == 0) { set_error("rlweCipherDecompose to digit planes: planes not opened (pcmm_packed_begin)"); return CKKS_E_STATE; }
    if (mlwe_num > k) { set_error("rlweCipherDecompose extract number must be <= mlwe_rank"); return CKKS_E_INVALID; }   // PCMM_Scheme.cuh:103-106
    if (mlwe_num <= 0 || k % mlwe_num || take <= 0 || take > mlwe_num || take % 64 || sample_offset < 0 || sample_offset % 64 ||
        sample_offset + take > h->packed_K || l < 0 || l > c->L || l + 1 != h->packed_mods || (long)h->N1 * k != c->N) {
        set_error("rlweCipherDecompose to digit planes: samples come in multiples of 64 that divide the rank, inside the opened shape, at its level");
        return CKKS_E_INVALID;
    }
    const size_t lds = (size_t)17 * (k + 1) * sizeof(u64);
    static const bool big_lds = hipFuncSetAttribute(reinterpret_cast<const void*>(rlwe_gather_digits_kernel),
                                                    hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024) == hipSuccess;
    if (lds > (big_lds ? 96 * 1024 : 64 * 1024)) { set_error("rlweCipherDecompose to digit planes: rank too large for the LDS window"); return CKKS_E_INVALID; }
    int rc;
    const int K = c->K;
    if ((rc = launch_ntt(c, rlwe, 0, K, 2, l + 1, c->L + 1, 0, 1, true))) return rc;              // PCMM_Scheme.cuh:113
    GatherDigitsArgs a;
    a.rlwe = rlwe; a.bdig = h->d_Bdig; a.primes = c->d_primes; a.N = c->N; a.N1 = h->N1; a.rank = k; a.mlwe_num = mlwe_num; a.L = c->L;
    a.p_num = c->p_num; a.kstep0 = sample_offset / 64; a.ksteps = (h->packed_K + 191) / 192 * 3; a.c_tiles = (int)((long)(k + 1) * h->N1 / 64);
    hipLaunchKernelGGL(rlwe_gather_digits_kernel, dim3(h->N1 / 16, l + 1, take / 64), dim3(256), lds, c->stream, a);
    CKKS_HIP_TRY(hipGetLastError());
    return launch_ntt(c, rlwe, 0, K, 2, l + 1, c->L + 1, 0, 1, false);                            // :122
}

extern "C" int pcmm_ppmm_packed(pcmm_ctx* h, const float* W, uint64_t* out, int M, double scaler) {
    if (!h) return CKKS_E_INVALID;
    if (h->packed_K == 0) { set_error("PPMM on digit planes: planes not opened (pcmm_packed_begin)"); return CKKS_E_STATE; }
    return ppmm_common(h, W, nullptr, nullptr, out, M, h->packed_K, h->packed_mods, scaler, true);
}
