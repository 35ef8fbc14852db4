// RNS basis conversion, key-switch inner products, ModDown and rescale for gfx950.
//
// Replaces BasisConv.cuh (modUpPQtoT_23 / modUpQjtoT_23 / modUpTtoPQl_23 / modDownPQltoQl_23),
// ExternalProduct.cuh:7-97 (external_product_T) and Scheme_23.cuh:321-385 (rescale).  One generic kernel performs
// every exact conversion "nsrc source primes -> ntgt target primes" described by a ConvBlock; the arithmetic per
// coefficient is the reference's (BasisConv.cuh:18-58):
//     y_j  = (x_j + add_j) * (D/d_j)^-1 mod d_j                      (Shoup)
//     v    = (int) sum_j (double) y_j / (double) d_j                 (IEEE double, summed in index order)
//     out_k = Barrett( sum_j y_j * ((D/d_j) mod r_k)  -  v * (D mod r_k) ) [ + r_k - sub_k, one conditional subtract ]
// All of these kernels stream every limb once; they are HBM bound (read nsrc + write ntgt limbs per block).
#include "context.hpp"
#include "f64_exact.hpp"

namespace ckks {

struct ConvArgs {
    const u64* in;
    u64* out;
    const ConvBlock* blocks;
    const PrimeConst* primes;
    long N, in_batch_stride, out_batch_stride;   // strides in words
    long out_block_stride;                        // added per block index (hybrid: one [P|Q] polynomial per digit)
    int centred;
};

constexpr int CONV_THREADS = 256;

template <int MAXS>
__global__ __launch_bounds__(CONV_THREADS) void conv_kernel(ConvArgs a) {
    const ConvBlock& __restrict__ b = a.blocks[blockIdx.y];
    const long x = (long)blockIdx.x * CONV_THREADS + threadIdx.x;
    const u64* in = a.in + (long)blockIdx.z * a.in_batch_stride;
    u64* out = a.out + (long)blockIdx.z * a.out_batch_stride + (long)blockIdx.y * a.out_block_stride;
    const int nsrc = b.nsrc;
    u64 y[MAXS];
    double vv = 0.0;
#pragma unroll
    for (int j = 0; j < MAXS; j++) {
        y[j] = 0;
        if (j < nsrc) {
            const u64 d = a.primes[b.src_prime[j]].q;
            u64 xin = in[(long)b.src_limb[j] * a.N + x];
            if (j < b.ncopy) out[(long)b.copy_limb[j] * a.N + x] = xin;
            xin += b.add_in[j];
            y[j] = mul_shoup(xin, b.hatinv[j], b.hatinv_s[j], d);
            vv += (double)y[j] / (double)d;
        }
    }
    const u64 v = (u64)(long)(int)vv;
    for (int k = 0; k < b.ntgt; k++) {
        const PrimeConst& pr = a.primes[b.tgt_prime[k]];
        u128w acc = {0, 0};
#pragma unroll
        for (int j = 0; j < MAXS; j++)
            if (j < nsrc) mac128(acc, y[j], b.hat[k][j]);
        sub128_64(acc, v * b.dmod[k]);
        u64 r = barrett128(acc, pr.q, pr.mu_hi, pr.mu_lo);
        if (a.centred) r = csub(r + pr.q - b.sub_out[k], pr.q);
        out[(long)b.tgt_limb[k] * a.N + x] = r;
    }
}

// ---- the same conversion in FP64 for bases whose primes are all below 2^41 ----
// On this part a 64 x 64 -> 128-bit integer product costs more than ten quarter-rate 32-bit multiplies, a double FMA is one
// full-rate instruction: with u128 accumulation the conversions are bound by integer multiplies, not by memory.  Here every
// value is an exact integer held in a double (|.| < 2^53 throughout) and a*w mod q is the two-product form used by the NTT, so
// the words written are the same.  y_j is brought to its canonical representative before it enters v and the sum, because the
// reference's v = (int) sum y_j / d_j and sum y_j * hat_j are functions of that representative.
// (the arithmetic and the per-coefficient sums are in f64_exact.hpp, where a host build checks their ranges)
__device__ __forceinline__ double u2d(u64 x) { return exact_u2d(x); }                        // exact for x < 2^52
__device__ __forceinline__ u64 d2u(double x) { return bits52(x); }                           // exact integer 0 <= x < 2^52
__device__ __forceinline__ double mulmod_d(double a, double w, double q, double qinv) { return mulmod_f64(a, w, q, qinv); }      // in (-0.51 q, 0.51 q)
__device__ __forceinline__ double canon_d(double r, double q, double qinv) { return canon_f64(r, q, qinv); }                     // any |r| < 2^52 -> [0, q)

// The targets of a block are shared out over CONV_TGT_PARTS workgroups (each recomputes the cheap y_j): a lane that walked
// through all 24+ targets alone left the launch with too few, too long lanes to cover the memory latency.
constexpr int CONV_TGT_PARTS = 4;
template <int MAXS>
__global__ __launch_bounds__(CONV_THREADS) void conv_kernel_f64(ConvArgs a) {
    const int blk = blockIdx.y / CONV_TGT_PARTS, part = blockIdx.y % CONV_TGT_PARTS;
    const ConvBlock& __restrict__ b = a.blocks[blk];
    const long x = (long)blockIdx.x * CONV_THREADS + threadIdx.x;
    const u64* in = a.in + (long)blockIdx.z * a.in_batch_stride;
    u64* out = a.out + (long)blockIdx.z * a.out_batch_stride + (long)blk * a.out_block_stride;
    const int nsrc = b.nsrc;
    double y[MAXS];
    double vv = 0.0;
#pragma unroll
    for (int j = 0; j < MAXS; j++) {
        y[j] = 0.0;
        if (j < nsrc) {
            const PrimeConst& ps = a.primes[b.src_prime[j]];
            const u64 xin = in[(long)b.src_limb[j] * a.N + x];
            if (j < b.ncopy && part == 0) out[(long)b.copy_limb[j] * a.N + x] = xin;
            y[j] = conv_f64_scale(xin, b.hatinv_d[j], ps.qd, ps.qinv_d);
            vv += y[j] / ps.qd;
        }
    }
    const double v = (double)(int)vv;
    const int per = (b.ntgt + CONV_TGT_PARTS - 1) / CONV_TGT_PARTS, k_end = min(b.ntgt, (part + 1) * per);
    for (int k = part * per; k < k_end; k++) {
        const PrimeConst& pr = a.primes[b.tgt_prime[k]];
        out[(long)b.tgt_limb[k] * a.N + x] = conv_f64_target<MAXS>(y, nsrc, b.hat_d[k], v, b.dmod_d[k], pr.qd, pr.qinv_d);
    }
}

// ---- sources of any width, targets below 2^50 (the reference's 60-bit T basis back into its 49-bit P and Q primes) ----
// The scaled residues y_j are formed in integers as in conv_kernel (they are residues of the source primes), so v is the same
// number.  The sums modulo the targets are the FP64 ones: y_j = yh 2^31 + yl with both parts below 2^31, each multiplied by its
// own constant ((D/d_j) and (D/d_j) 2^31 mod r_k, balanced) in the two-product form; every term lies within 0.51 r_k of zero and
// the running sum is balanced after every four sources, so all integers stay below 2^53.  A 64 x 64 -> 128-bit product costs
// more than ten quarter-rate 32-bit multiplies on this part, the two FP64 products ten full-rate instructions.
// The targets of a block are shared out over `parts` workgroups, each of which forms the y_j again: one part per eight targets
// (reading and scaling the sources is two thirds of a part's time, so the 8 x 8 blocks of the T basis run unsplit: 53 us against
// 71 us in two parts and 114 us in four).
template <int MAXS>
__global__ __launch_bounds__(CONV_THREADS) void conv_kernel_split(ConvArgs a, int parts) {
    const int blk = blockIdx.y / parts, part = blockIdx.y % parts;
    const ConvBlock& __restrict__ b = a.blocks[blk];
    const long x = (long)blockIdx.x * CONV_THREADS + threadIdx.x;
    const u64* in = a.in + (long)blockIdx.z * a.in_batch_stride;
    u64* out = a.out + (long)blockIdx.z * a.out_batch_stride + (long)blk * a.out_block_stride;
    const int nsrc = b.nsrc;
    double yl[MAXS], yh[MAXS];
    double vv = 0.0;
#pragma unroll
    for (int j = 0; j < MAXS; j++) {
        yl[j] = yh[j] = 0.0;
        if (j < nsrc) {
            const u64 d = a.primes[b.src_prime[j]].q;
            u64 xin = in[(long)b.src_limb[j] * a.N + x];
            if (j < b.ncopy && part == 0) out[(long)b.copy_limb[j] * a.N + x] = xin;
            xin += b.add_in[j];
            const u64 y = mul_shoup(xin, b.hatinv[j], b.hatinv_s[j], d);
            vv += (double)y / (double)d;
            conv_split_parts(y, yl[j], yh[j]);
        }
    }
    const double v = (double)(int)vv;
    const int per = (b.ntgt + parts - 1) / parts, k_end = min(b.ntgt, (part + 1) * per);
    for (int k = part * per; k < k_end; k++) {
        const PrimeConst& pr = a.primes[b.tgt_prime[k]];
        const double q = pr.qd, qinv = pr.qinv_d;
        double r = conv_split_target<MAXS>(yl, yh, nsrc, b.hat_d[k], b.hat31_d[k], v, b.dmod_d[k], q, qinv);
        if (a.centred) {
            r -= u2d(b.sub_out[k]);
            r = r < 0.0 ? r + q : r;
        }
        out[(long)b.tgt_limb[k] * a.N + x] = d2u(r);
    }
}

static int launch_conv(ckks_ctx* c, const ConvPlan& plan, u64* out, const u64* in, int batch, long in_bs, long out_bs,
                       long out_block_stride, int centred, int max_src) {
    if (plan.count == 0 || batch <= 0) return CKKS_OK;
    ConvArgs a;
    a.in = in; a.out = out; a.blocks = c->d_conv + plan.first; a.primes = c->d_primes;
    a.N = c->N; a.in_batch_stride = in_bs; a.out_batch_stride = out_bs; a.out_block_stride = out_block_stride;
    a.centred = centred;
    dim3 grid((unsigned)(c->N / CONV_THREADS), plan.count, batch), block(CONV_THREADS);
    if (plan.f64_ok && !centred && c->arith_mode == 0) {
        grid.y *= CONV_TGT_PARTS;
        if (max_src <= 4) hipLaunchKernelGGL(conv_kernel_f64<4>, grid, block, 0, c->stream, a);
        else if (max_src <= 8) hipLaunchKernelGGL(conv_kernel_f64<8>, grid, block, 0, c->stream, a);
        else hipLaunchKernelGGL(conv_kernel_f64<CONV_MAX_SRC>, grid, block, 0, c->stream, a);
        CKKS_HIP_TRY(hipGetLastError());
        return CKKS_OK;
    }
    if (plan.split_ok && c->arith_mode == 0 && !c->conv_int) {
        const int parts = plan.max_tgt <= 8 ? 1 : plan.max_tgt <= 16 ? 2 : 4;
        grid.y *= parts;
        if (max_src <= 4) hipLaunchKernelGGL(conv_kernel_split<4>, grid, block, 0, c->stream, a, parts);
        else if (max_src <= 8) hipLaunchKernelGGL(conv_kernel_split<8>, grid, block, 0, c->stream, a, parts);
        else hipLaunchKernelGGL(conv_kernel_split<CONV_MAX_SRC>, grid, block, 0, c->stream, a, parts);
        CKKS_HIP_TRY(hipGetLastError());
        return CKKS_OK;
    }
    if (max_src <= 4) hipLaunchKernelGGL(conv_kernel<4>, grid, block, 0, c->stream, a);
    else if (max_src <= 8) hipLaunchKernelGGL(conv_kernel<8>, grid, block, 0, c->stream, a);
    else hipLaunchKernelGGL(conv_kernel<CONV_MAX_SRC>, grid, block, 0, c->stream, a);
    CKKS_HIP_TRY(hipGetLastError());
    return CKKS_OK;
}

// ---- ModDown: out_i = (c_{q_i} - Conv_{P -> q_i}(c_P)) * P^-1 mod q_i, no v term (BasisConv.cuh:257-326) ----
struct ModDownArgs {
    const u64* in;
    u64* out;
    const PrimeConst* primes;
    const u64* pHatVecModq;       // [L+1][K]
    const u64* pHatInv;           // [K] values, [K] Shoup words
    const u64* PinvModq;          // [L+1] values, [L+1] Shoup words
    long N, in_batch_stride, out_batch_stride;
    int K, q_num;
};
template <int MAXK>
__global__ __launch_bounds__(CONV_THREADS) void moddown_kernel(ModDownArgs a) {
    const long x = (long)blockIdx.x * CONV_THREADS + threadIdx.x;
    const int iq = blockIdx.y;
    const u64* in = a.in + (long)blockIdx.z * a.in_batch_stride;
    const PrimeConst& pq = a.primes[a.K + iq];
    u64 r;
    if (a.K == 1) {
        r = in[x] % pq.q;                                             // BasisConv.cuh:274
    } else {
        u128w acc = {0, 0};
#pragma unroll
        for (int i = 0; i < MAXK; i++)
            if (i < a.K) {
                u64 rb = mul_shoup(in[(long)i * a.N + x], a.pHatInv[i], a.pHatInv[a.K + i], a.primes[i].q);
                mac128(acc, rb, a.pHatVecModq[(long)iq * a.K + i]);
            }
        r = barrett128(acc, pq.q, pq.mu_hi, pq.mu_lo);
    }
    u64 v = pq.q - r + in[(long)(a.K + iq) * a.N + x];
    a.out[(long)blockIdx.z * a.out_batch_stride + (long)iq * a.N + x] = mul_shoup(v, a.PinvModq[iq], a.PinvModq[a.q_num + iq], pq.q);
}
constexpr int MODDOWN_TGTS = 4;        // output primes per lane: the special-prime residues are read and scaled once for all of them
template <int MAXK>
__global__ __launch_bounds__(CONV_THREADS) void moddown_kernel_f64(ModDownArgs a, int q_count) {
    const long x = (long)blockIdx.x * CONV_THREADS + threadIdx.x;
    const u64* in = a.in + (long)blockIdx.z * a.in_batch_stride;
    double rb[MAXK];
#pragma unroll
    for (int i = 0; i < MAXK; i++) {
        rb[i] = 0.0;
        if (i < a.K) {
            const PrimeConst& pp = a.primes[i];
            // the canonical representative of rb enters the sums (there is no v term to absorb another one)
            rb[i] = a.K == 1 ? u2d(in[x])
                             : canon_d(mulmod_d(u2d(in[(long)i * a.N + x]), u2d(a.pHatInv[i]), pp.qd, pp.qinv_d), pp.qd, pp.qinv_d);
        }
    }
    const int iq_end = min(q_count, (int)(blockIdx.y + 1) * MODDOWN_TGTS);
    for (int iq = blockIdx.y * MODDOWN_TGTS; iq < iq_end; iq++) {
        const PrimeConst& pq = a.primes[a.K + iq];
        double r;
        if (a.K == 1) {
            r = canon_d(rb[0], pq.qd, pq.qinv_d);                         // in[x] % q
        } else {
            double acc = 0.0;
#pragma unroll
            for (int i = 0; i < MAXK; i++)
                if (i < a.K) acc += mulmod_d(rb[i], u2d(a.pHatVecModq[(long)iq * a.K + i]), pq.qd, pq.qinv_d);
            r = canon_d(acc, pq.qd, pq.qinv_d);
        }
        const double v = pq.qd - r + u2d(in[(long)(a.K + iq) * a.N + x]);
        a.out[(long)blockIdx.z * a.out_batch_stride + (long)iq * a.N + x] =
            d2u(canon_d(mulmod_d(v, u2d(a.PinvModq[iq]), pq.qd, pq.qinv_d), pq.qd, pq.qinv_d));
    }
}
static int launch_moddown(ckks_ctx* c, u64* out, const u64* in, int l, int batch, long in_bs, long out_bs) {
    ModDownArgs a;
    a.in = in; a.out = out; a.primes = c->d_primes; a.pHatVecModq = c->d_pHatVecModq; a.pHatInv = c->d_pHatInvVecModp;
    a.PinvModq = c->d_PinvModq; a.N = c->N; a.in_batch_stride = in_bs; a.out_batch_stride = out_bs; a.K = c->K; a.q_num = c->q_num;
    dim3 grid((unsigned)(c->N / CONV_THREADS), l + 1, batch), block(CONV_THREADS);
    bool f64 = c->arith_mode == 0;
    for (int i = 0; i < c->K + l + 1 && f64; i++) f64 = c->f64_ok[i] != 0;
    if (f64) {
        grid.y = (unsigned)((l + 1 + MODDOWN_TGTS - 1) / MODDOWN_TGTS);
        if (c->K <= 4) hipLaunchKernelGGL(moddown_kernel_f64<4>, grid, block, 0, c->stream, a, l + 1);
        else if (c->K <= 8) hipLaunchKernelGGL(moddown_kernel_f64<8>, grid, block, 0, c->stream, a, l + 1);
        else hipLaunchKernelGGL(moddown_kernel_f64<16>, grid, block, 0, c->stream, a, l + 1);
        CKKS_HIP_TRY(hipGetLastError());
        return CKKS_OK;
    }
    if (c->K <= 4) hipLaunchKernelGGL(moddown_kernel<4>, grid, block, 0, c->stream, a);
    else if (c->K <= 8) hipLaunchKernelGGL(moddown_kernel<8>, grid, block, 0, c->stream, a);
    else hipLaunchKernelGGL(moddown_kernel<16>, grid, block, 0, c->stream, a);
    CKKS_HIP_TRY(hipGetLastError());
    return CKKS_OK;
}

// ---- inner product over digits: out[z][o] = sum_d c[d][o % c_mod] * key[z][d][o]  (ExternalProduct.cuh:56-83) ----
struct InnerArgs {
    const u64* c;
    const u64* key;
    u64* out;
    const PrimeConst* primes;
    long N;
    int ndigits, c_mod, prime0;
    long c_digit_stride, key_digit_stride, key_z_stride, out_z_stride;   // in limbs
};
__global__ __launch_bounds__(CONV_THREADS) void inner_product_kernel(InnerArgs a) {
    const long x = (long)blockIdx.x * CONV_THREADS + threadIdx.x;
    const int o = blockIdx.y;
    const int k = o % a.c_mod;
    const PrimeConst& pr = a.primes[a.prime0 + k];
    u128w acc1 = {0, 0}, acc2 = {0, 0};
    for (int d = 0; d < a.ndigits; d++) {
        u64 ra = a.c[((long)d * a.c_digit_stride + k) * a.N + x];
        long kidx = ((long)d * a.key_digit_stride + o) * a.N + x;
        mac128(acc1, ra, a.key[kidx]);
        mac128(acc2, ra, a.key[a.key_z_stride * a.N + kidx]);
    }
    a.out[(long)o * a.N + x] = barrett128(acc1, pr.q, pr.mu_hi, pr.mu_lo);
    a.out[(a.out_z_stride + o) * a.N + x] = barrett128(acc2, pr.q, pr.mu_hi, pr.mu_lo);
}

// One switching key against `batch` digit sets (external_product_T_kernel_swk_reuse, ExternalProduct.cuh:103-149): every key word is
// read once and multiplied into the accumulators of all the sets.  Set `it` lies c_set_stride limbs behind set it - 1; its two
// result polynomials are polynomials 2 it and 2 it + 1 of the output (out_z_stride limbs each).
constexpr int REUSE_MAX_BATCH = 8;                 // the reference's accumulator array holds eight sets
__global__ __launch_bounds__(CONV_THREADS) void inner_product_reuse_kernel(InnerArgs a, int batch, long c_set_stride) {
    const long x = (long)blockIdx.x * CONV_THREADS + threadIdx.x;
    const int o = blockIdx.y;
    const int k = o % a.c_mod;
    const PrimeConst& pr = a.primes[a.prime0 + k];
    u128w acc1[REUSE_MAX_BATCH], acc2[REUSE_MAX_BATCH];
#pragma unroll
    for (int it = 0; it < REUSE_MAX_BATCH; it++) acc1[it] = acc2[it] = u128w{0, 0};
    for (int d = 0; d < a.ndigits; d++) {
        const long kidx = ((long)d * a.key_digit_stride + o) * a.N + x;
        const u64 k1 = a.key[kidx], k2 = a.key[a.key_z_stride * a.N + kidx];
        const u64* cp = a.c + ((long)d * a.c_digit_stride + k) * a.N + x;
#pragma unroll
        for (int it = 0; it < REUSE_MAX_BATCH; it++)
            if (it < batch) {
                const u64 ra = cp[(long)it * c_set_stride * a.N];
                mac128(acc1[it], ra, k1);
                mac128(acc2[it], ra, k2);
            }
    }
#pragma unroll
    for (int it = 0; it < REUSE_MAX_BATCH; it++)
        if (it < batch) {
            a.out[((long)(2 * it) * a.out_z_stride + o) * a.N + x] = barrett128(acc1[it], pr.q, pr.mu_hi, pr.mu_lo);
            a.out[((long)(2 * it + 1) * a.out_z_stride + o) * a.N + x] = barrett128(acc2[it], pr.q, pr.mu_hi, pr.mu_lo);
        }
}

// ---- rescale (Scheme_23.cuh:321-367) ----
__global__ __launch_bounds__(CONV_THREADS) void mod_to_qi_kernel(u64* dst, const u64* src, const PrimeConst* primes, long N, int K, int q_num, int l) {
    const long x = (long)blockIdx.x * CONV_THREADS + threadIdx.x;
    const int i = blockIdx.y, z = blockIdx.z;
    const PrimeConst& pr = primes[K + i];
    u64 rb = src[((long)z * q_num + l) * N + x];
    dst[((long)z * q_num + i) * N + x] = barrett64(rb, pr.q, pr.mu_hi);
}
__global__ __launch_bounds__(CONV_THREADS) void rescale_kernel(u64* a, const u64* b, const PrimeConst* primes, const u64* inv, const u64* inv_s,
                                                               long N, int K, int q_num) {
    const long x = (long)blockIdx.x * CONV_THREADS + threadIdx.x;
    const int i = blockIdx.y, z = blockIdx.z;
    const u64 q = primes[K + i].q;
    const long idx = ((long)z * q_num + i) * N + x;
    u64 ra = csub(a[idx] + 2 * q - b[idx], q);
    a[idx] = mul_shoup(ra, inv[i], inv_s[i], q);
}

static bool level_ok(const ckks_ctx* c, int l) { return c && l >= 0 && l <= c->L; }

}  // namespace ckks

using namespace ckks;

extern "C" int ckks_modup_pq_to_t(ckks_ctx* c, uint64_t* out, const uint64_t* in, int l, int batch) {
    if (!level_ok(c, l) || !out || !in || c->t_num == 0 || c->gamma == 0) { set_error("modUpPQtoT_23: bad level or no T basis"); return CKKS_E_INVALID; }
    return launch_conv(c, c->plan_pq_to_t[l], out, in, batch, (long)(c->p_num + c->q_num) * c->N,
                       (long)c->Ri_blockNum * c->t_num * c->N, 0, 0, c->gamma);
}
extern "C" int ckks_modup_qj_to_t(ckks_ctx* c, uint64_t* out, const uint64_t* in, int l, int batch) {
    if (!level_ok(c, l) || !out || !in || c->t_num == 0 || c->p_num == 0) { set_error("modUpQjtoT_23: bad level or no T/P basis"); return CKKS_E_INVALID; }
    return launch_conv(c, c->plan_qj_to_t[l], out, in, batch, (long)c->q_num * c->N, (long)c->Qj_blockNum * c->t_num * c->N, 0, 0, c->p_num);
}
extern "C" int ckks_modup_t_to_pql(ckks_ctx* c, uint64_t* buf, const uint64_t* in, int l, int batch) {
    if (!level_ok(c, l) || !buf || !in || c->t_num == 0 || c->gamma == 0) { set_error("modUpTtoPQl_23: bad level or no T basis"); return CKKS_E_INVALID; }
    long bs = (long)c->Ri_blockNum * c->t_num * c->N;
    return launch_conv(c, c->plan_t_to_pq[l], buf, in, batch, bs, bs, 0, 1, c->t_num);
}
extern "C" int ckks_moddown_pql_to_ql(ckks_ctx* c, uint64_t* out, const uint64_t* buf, int l, int batch) {
    if (!level_ok(c, l) || !out || !buf || c->p_num == 0) { set_error("modDownPQltoQl_23: bad level or no P basis"); return CKKS_E_INVALID; }
    if (batch <= 0) return CKKS_OK;
    return launch_moddown(c, out, buf, l, batch, (long)c->Ri_blockNum * c->t_num * c->N, (long)c->q_num * c->N);
}
extern "C" int ckks_external_product_t(ckks_ctx* c, uint64_t* out, const uint64_t* cT, const uint64_t* swk, int l) {
    if (!level_ok(c, l) || !out || !cT || !swk || c->t_num == 0 || c->gamma == 0 || c->p_num == 0) { set_error("external_product_T: bad level or basis"); return CKKS_E_INVALID; }
    InnerArgs a;
    a.c = cT; a.key = swk; a.out = out; a.primes = c->d_primes; a.N = c->N;
    a.ndigits = (l + 1 + c->p_num - 1) / c->p_num;                       // cipher_blockNum, ExternalProduct.cuh:87
    if (a.ndigits > c->dnum) { set_error("external_product_T: the level needs more digits than the key holds (q_num is no multiple of p_num)"); return CKKS_E_INVALID; }
    a.c_mod = c->t_num; a.prime0 = c->p_num + c->q_num;
    a.c_digit_stride = c->t_num; a.key_digit_stride = (long)c->t_num * c->Ri_blockNum;
    a.key_z_stride = (long)c->Ri_blockNum * c->t_num * c->dnum; a.out_z_stride = (long)c->Ri_blockNum * c->t_num;
    int blockNum = (c->p_num + l + 1 + c->gamma - 1) / c->gamma;         // :88
    dim3 grid((unsigned)(c->N / CONV_THREADS), blockNum * c->t_num), block(CONV_THREADS);
    hipLaunchKernelGGL(inner_product_kernel, grid, block, 0, c->stream, a);
    CKKS_HIP_TRY(hipGetLastError());
    return CKKS_OK;
}
extern "C" int ckks_external_product_t_swk_reuse(ckks_ctx* c, uint64_t* out, const uint64_t* cT, const uint64_t* swk, int l, int batch_size) {
    if (!level_ok(c, l) || !out || !cT || !swk || c->t_num == 0 || c->gamma == 0 || c->p_num == 0) { set_error("external_product_T_swk_reuse: bad level or basis"); return CKKS_E_INVALID; }
    if (batch_size < 1 || batch_size > REUSE_MAX_BATCH) { set_error("external_product_T_swk_reuse: batch_size must be 1 .. 8 (the reference's accumulator array)"); return CKKS_E_INVALID; }
    InnerArgs a;
    a.c = cT; a.key = swk; a.out = out; a.primes = c->d_primes; a.N = c->N;
    a.ndigits = (l + 1 + c->p_num - 1) / c->p_num;                       // cipher_blockNum, ExternalProduct.cuh:153
    if (a.ndigits > c->dnum) { set_error("external_product_T_swk_reuse: the level needs more digits than the key holds (q_num is no multiple of p_num)"); return CKKS_E_INVALID; }
    a.c_mod = c->t_num; a.prime0 = c->p_num + c->q_num;
    a.c_digit_stride = c->t_num; a.key_digit_stride = (long)c->t_num * c->Ri_blockNum;
    a.key_z_stride = (long)c->Ri_blockNum * c->t_num * c->dnum; a.out_z_stride = (long)c->Ri_blockNum * c->t_num;
    const int blockNum = (c->p_num + l + 1 + c->gamma - 1) / c->gamma;   // :154
    dim3 grid((unsigned)(c->N / CONV_THREADS), blockNum * c->t_num), block(CONV_THREADS);
    hipLaunchKernelGGL(inner_product_reuse_kernel, grid, block, 0, c->stream, a, batch_size, (long)c->t_num * c->Qj_blockNum);   // :126
    CKKS_HIP_TRY(hipGetLastError());
    return CKKS_OK;
}
extern "C" int ckks_rescale(ckks_ctx* c, uint64_t* cipher, uint64_t* scratch, int l) {
    if (!c || !cipher || !scratch) return CKKS_E_INVALID;
    if (l < 1 || l > c->L) { set_error("rescaleAndEqual: ciphertext is on level 0"); return CKKS_E_STATE; }
    const int K = c->K, L = c->L;
    int rc = launch_ntt(c, cipher, l, K + l, 2, 1, L + 1, 0, 1, true);                            // Scheme_23.cuh:372
    if (rc) return rc;
    const u64* inv_l = (const u64*)c->d_qiInvModql + (size_t)l * (l - 1) / 2;
    bool fused = false;
    if ((rc = launch_rescale_fused(c, cipher, l, inv_l, &fused))) return rc;
    if (fused) return CKKS_OK;
    dim3 grid((unsigned)(c->N / CONV_THREADS), l, 2), block(CONV_THREADS);
    hipLaunchKernelGGL(mod_to_qi_kernel, grid, block, 0, c->stream, (u64*)scratch, (const u64*)cipher, c->d_primes, c->N, K, L + 1, l);
    rc = launch_ntt(c, scratch, 0, K, 2, l, L + 1, 0, 1, false);                                   // :376
    if (rc) return rc;
    const u64* inv = (const u64*)c->d_qiInvModql + (size_t)l * (l - 1) / 2;
    hipLaunchKernelGGL(rescale_kernel, grid, block, 0, c->stream, (u64*)cipher, (const u64*)scratch, c->d_primes, inv, inv + c->qiInv_count, c->N, K, L + 1);
    CKKS_HIP_TRY(hipGetLastError());
    return CKKS_OK;
}
extern "C" int ckks_keyswitch_23(ckks_ctx* c, uint64_t* out, uint64_t* d2, const uint64_t* swk, int l, uint64_t* up, uint64_t* ext, uint64_t* buf) {
    bool added;
    return ckks::keyswitch_23_add(c, out, d2, swk, l, up, ext, buf, nullptr, 0, &added);
}
int ckks::keyswitch_23_add(ckks_ctx* c, uint64_t* out, uint64_t* d2, const uint64_t* swk, int l, uint64_t* up, uint64_t* ext, uint64_t* buf,
                           const uint64_t* addend, long addend_poly_stride, bool* added) {
    *added = false;
    if (!c || !out || !d2 || !up || !ext || !buf) return CKKS_E_INVALID;
    if (!swk) { set_error("rotKey_23 not exists"); return CKKS_E_STATE; }                           // KeySwitch_23.cuh:198-201
    if (!level_ok(c, l) || c->t_num == 0 || c->gamma == 0 || c->p_num == 0) { set_error("keyswitch_23: bad level or basis"); return CKKS_E_INVALID; }
    const int K = c->K, L = c->L, T = c->t_num, RB = c->Ri_blockNum;
    const int swk_blockNum = (K + l + 1 + c->gamma - 1) / c->gamma, cipher_blockNum = (l + 1 + K - 1) / K;
    int rc;
    if ((rc = launch_ntt(c, d2, 0, K, 1, l + 1, L + 1, 0, 1, true))) return rc;                     // :219
    if ((rc = ckks_modup_qj_to_t(c, up, d2, l, 1))) return rc;                                      // :221
    if ((rc = launch_ntt(c, up, 0, K + L + 1, cipher_blockNum, T, T, 0, 1, false))) return rc;      // :223
    bool ext_fused = false;
    if ((rc = launch_ext_product_inverse_fused(c, ext, up, swk, l, &ext_fused))) return rc;       // :225 and :226 in two launches
    if (!ext_fused) {
        if ((rc = ckks_external_product_t(c, ext, up, swk, l))) return rc;                          // :225
        if ((rc = launch_ntt(c, ext, 0, K + L + 1, swk_blockNum, T, T, (long)RB * T, 2, true))) return rc;   // :226
    }
    if ((rc = ckks_modup_t_to_pql(c, buf, ext, l, 2))) return rc;                                   // :228
    bool fused = false;
    if ((rc = launch_ks_moddown_fused(c, out, buf, (long)RB * T * c->N, l, L + 1, false, &fused, addend, addend_poly_stride))) return rc;  // :229 and :231 in two launches
    if (fused) { *added = addend != nullptr; return CKKS_OK; }
    if ((rc = ckks_moddown_pql_to_ql(c, out, buf, l, 2))) return rc;                                // :229
    return launch_ntt(c, out, 0, K, 2, l + 1, L + 1, 0, 1, false);                                  // :231
}

// ---- textbook hybrid key switch over [P | Q_l] ----
extern "C" int ckks_hybrid_modup(ckks_ctx* c, uint64_t* digits, const uint64_t* in, int l) {
    if (!level_ok(c, l) || !digits || !in || c->p_num == 0) { set_error("hybrid_modup: bad level or no P basis"); return CKKS_E_INVALID; }
    return launch_conv(c, c->plan_hybrid[l], digits, in, 1, 0, 0, (long)(c->p_num + c->q_num) * c->N, 0, c->p_num);
}
extern "C" int ckks_hybrid_inner_product(ckks_ctx* c, uint64_t* ip, const uint64_t* digits, const uint64_t* evk, int l) {
    if (!level_ok(c, l) || !ip || !digits || !evk || c->p_num == 0) { set_error("hybrid_inner_product: bad level or no P basis"); return CKKS_E_INVALID; }
    const int W = c->p_num + c->q_num, dnum = (c->q_num + c->p_num - 1) / c->p_num;
    InnerArgs a;
    a.c = digits; a.key = evk; a.out = ip; a.primes = c->d_primes; a.N = c->N;
    a.ndigits = (l + 1 + c->p_num - 1) / c->p_num;
    a.c_mod = W; a.prime0 = 0; a.c_digit_stride = W; a.key_digit_stride = W; a.key_z_stride = (long)dnum * W; a.out_z_stride = W;
    dim3 grid((unsigned)(c->N / CONV_THREADS), c->p_num + l + 1), block(CONV_THREADS);
    hipLaunchKernelGGL(inner_product_kernel, grid, block, 0, c->stream, a);
    CKKS_HIP_TRY(hipGetLastError());
    return CKKS_OK;
}
extern "C" int ckks_hybrid_moddown(ckks_ctx* c, uint64_t* out, const uint64_t* in, int l) {
    if (!level_ok(c, l) || !out || !in || c->p_num == 0) { set_error("hybrid_moddown: bad level or no P basis"); return CKKS_E_INVALID; }
    return launch_moddown(c, out, in, l, 2, (long)(c->p_num + c->q_num) * c->N, (long)c->q_num * c->N);
}
extern "C" int ckks_hybrid_keyswitch(ckks_ctx* c, uint64_t* out, uint64_t* in_ntt, const uint64_t* evk, int l, uint64_t* scratch) {
    if (!level_ok(c, l) || !out || !in_ntt || !evk || !scratch || c->p_num == 0) { set_error("hybrid_keyswitch: bad argument"); return CKKS_E_INVALID; }
    const int P = c->p_num, Q = c->q_num, W = P + Q, dn = (l + 1 + P - 1) / P;
    uint64_t* dig = scratch;
    uint64_t* ip = scratch + (size_t)dn * W * c->N;
    int rc;
    bool fused = false;
    // Where it applies (N = 2^16, primes below 2^39): five launches up to the sums in the coefficient domain, the digit area of the
    // scratch serving as work space, the input left as it is; the sums' special-prime limbs come out scaled for the ModDown below.
    bool finished = false;
    if ((rc = launch_hybrid_front_fused(c, in_ntt, dig, ip, evk, l, &fused, out, Q, &finished))) return rc;
    if (finished) return CKKS_OK;
    if (!fused) {
        if ((rc = launch_ntt(c, in_ntt, 0, P, 1, l + 1, Q, 0, 1, true))) return rc;
        if ((rc = ckks_hybrid_modup(c, dig, in_ntt, l))) return rc;
        if ((rc = launch_ntt(c, dig, 0, 0, dn, P + l + 1, W, 0, 1, false))) return rc;
        if ((rc = ckks_hybrid_inner_product(c, ip, dig, evk, l))) return rc;
        if ((rc = launch_ntt(c, ip, 0, 0, 2, P + l + 1, W, 0, 1, true))) return rc;
    }
    const bool scaled = fused;
    if ((rc = launch_ks_moddown_fused(c, out, ip, (long)W * c->N, l, Q, scaled, &fused))) return rc;
    if (fused) return CKKS_OK;
    if (scaled) { set_error("hybrid_keyswitch: internal: the two one-launch steps apply under the same conditions"); return CKKS_E_UNAVAILABLE; }
    if ((rc = ckks_hybrid_moddown(c, out, ip, l))) return rc;
    return launch_ntt(c, out, 0, P, 2, l + 1, Q, 0, 1, false);
}
