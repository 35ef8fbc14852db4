// Hoisted rotations of the slot <-> coefficient transforms for gfx950: the baby-step / giant-step evaluation of a plaintext
// matrix on a ciphertext with every rotation taken in the T basis, where it is an index permutation of NTT-domain limbs.
//
// Reference: EncodingMatrix::Giant_Rotate_And_Mult_PlaintT and ::Baby_Rotate with their kernels
// (Bootstrapping_C2S_S2C_impl.cuh:7-228), the level loop of EvalCoeffsToSlots / EvalSlotsToCoeffs around them (:254-382, 531-625),
// cipher_mul_P_batch (poly_arithmetic.cuh:863-887), cipher_add_T_batch_device (:143-153, 409-413) and
// Scheme_23::rescaleAndEqual_noNTT (Scheme_23.cuh:321-337, 427-440).
//
// Memory behaviour.  The rotation by 5^r reads slot pi(x) = bitrev(((5^r (2 bitrev(x) + 1) mod 2N) - 1) / 2) for output slot x.
// For the 64 consecutive x of a wave, pi keeps the upper bits common and permutes the low six, so every gather of a wave is one
// aligned 512-byte segment: keys, digits and P*b are read at full line efficiency without staging.  The reference passes its
// key / plaintext pointer tables through device memory with a blocking copy per call; here they travel as kernel arguments.
#include <hip/hip_runtime.h>
#include <string>

#include "context.hpp"

using namespace ckks;

namespace {

constexpr int THREADS = 256;
constexpr int MAX_GS = 16, MAX_BS = 8, MAX_LIMBS = 64;

__device__ __forceinline__ long hoist_perm(u64 pow, long x, int logN, u64 mask) {
    u64 e = 2 * (u64)(__brev((unsigned)x) >> (32 - logN)) + 1;
    e = (((pow * e) & mask) - 1) >> 1;
    return (long)(__brev((unsigned)e) >> (32 - logN));
}

// Sums of up to 16 products of operands below 2^60 without carries: the operands are split at bit 30 and the four partial
// products, each below 2^60, are summed in four 64-bit words (16 x (2^30 - 1)^2 < 2^64), one 32 x 32 + 64-bit multiply-add each;
// the 128-bit value is put together once per sum.  A 64 x 64 -> 128-bit multiply-add in 32-bit pieces with carry chains costs
// about three times as many instructions, and these kernels are bound by them.
struct Sum60 {
    u64 s00, s01, s10, s11;
};
__device__ __forceinline__ void mac60(Sum60& s, u64 a, u64 b) {
    const unsigned a0 = (unsigned)a & 0x3fffffffu, a1 = (unsigned)(a >> 30);
    const unsigned b0 = (unsigned)b & 0x3fffffffu, b1 = (unsigned)(b >> 30);
    s.s00 += (u64)a0 * b0;
    s.s01 += (u64)a0 * b1;
    s.s10 += (u64)a1 * b0;
    s.s11 += (u64)a1 * b1;
}
__device__ __forceinline__ u128w fold60(const Sum60& s, u64 extra) {       // s00 + (s01 + s10) 2^30 + s11 2^60 + extra
    u128w r{s.s00, 0};
    const u64 m = s.s01 + s.s10;
    const u64 mc = m < s.s01;                              // bit 64 of the middle sum
    u64 lo = r.lo + (m << 30);
    r.hi = (m >> 34) + (mc << 30) + (lo < r.lo);
    r.lo = lo;
    lo = r.lo + (s.s11 << 60);
    r.hi += (s.s11 >> 4) + (lo < r.lo);
    r.lo = lo;
    lo = r.lo + extra;
    r.hi += (lo < r.lo);
    r.lo = lo;
    return r;
}
// FAST: every T prime below 2^60 and at most 16 digits (so at most 16 terms per sum): the carry-free sums above
template <bool FAST>
struct Acc;
template <>
struct Acc<true> {
    Sum60 s{0, 0, 0, 0};
    __device__ __forceinline__ void mac(u64 a, u64 b) { mac60(s, a, b); }
    __device__ __forceinline__ u128w value(u64 extra) const { return fold60(s, extra); }
};
template <>
struct Acc<false> {
    u128w s{0, 0};
    __device__ __forceinline__ void mac(u64 a, u64 b) { mac128(s, a, b); }
    __device__ __forceinline__ u128w value(u64 extra) const {
        u128w r = s;
        r.lo += extra;
        r.hi += (r.lo < extra);
        return r;
    }
};

// Workgroup id -> (256-slot chunk, T prime, block).  The digits of a, P b and the plaintexts of a (chunk, prime) are the same for
// every block; workgroups whose ids agree modulo 8 share an XCD and its L2 and start in id order, so the blocks of one (chunk,
// prime) get consecutive places in one XCD's sequence and read those operands from the L2 instead of from memory again (counters:
// 13.2 GB fetched for 7.4 GB of distinct operands with a plain 3-D grid).
struct TileIndex {
    int chunk, k, blk;
};
__device__ __forceinline__ TileIndex tile_index(unsigned id, int chunks, int T, int blocks) {
    TileIndex t;
    if ((chunks & 7) == 0) {
        const unsigned xcd = id & 7, j = id >> 3, per = (unsigned)chunks >> 3;
        t.blk = (int)(j % (unsigned)blocks);
        const unsigned r = j / (unsigned)blocks;
        t.chunk = (int)((r % per) * 8 + xcd);
        t.k = (int)(r / per);
    } else {
        t.chunk = (int)(id % (unsigned)chunks);
        t.k = (int)((id / (unsigned)chunks) % (unsigned)T);
        t.blk = (int)(id / ((unsigned)chunks * (unsigned)T));
    }
    return t;
}

struct GiantArgs {
    u64* out;                       // [bs][a | b][Ri_blockNum][t_num] limbs
    const u64* pqT;                 // P * (a, b) in T: [a | b][Ri_blockNum][t_num]
    const u64* up;                  // digits of a in T: [digit][t_num]
    const PrimeConst* primes;
    const u64* key[MAX_GS];         // null: the pair itself
    u64 pow[MAX_GS];
    const u64* plain[MAX_BS * MAX_GS];
    int acc_num[MAX_BS];
    long N;
    int logN, T, RB, dnum, digits, prime0, bs, gs, blocks;
};

// one lane per (block, T prime, slot); per rotation of the giant step the rotated pair is formed once and multiplied into the
// accumulators of all baby steps
template <int BS, bool FAST>
__global__ __launch_bounds__(THREADS) void giant_rotate_mult_kernel(GiantArgs a) {
    const TileIndex ti = tile_index(blockIdx.x, (int)(a.N / THREADS), a.T, a.blocks);
    const long x = (long)ti.chunk * THREADS + threadIdx.x;
    const int k = ti.k, blk = ti.blk;
    const PrimeConst p = a.primes[a.prime0 + k];
    const long N = a.N;
    const u64 mask = 2 * (u64)N - 1;
    const size_t half = (size_t)a.RB * a.T * N;
    const size_t limb = ((size_t)blk * a.T + k) * N;
    Acc<false> acc_a[BS], acc_b[BS];         // 128-bit sums here: the carry-free form would double their registers
    for (int j = 0; j < a.gs; j++) {
        const u64* key = a.key[j];
        u64 ea, eb;
        if (!key) {
            ea = a.pqT[limb + x];
            eb = a.pqT[limb + x + half];
        } else {
            const long px = hoist_perm(a.pow[j], x, a.logN, mask);
            Acc<FAST> s1, s2;
            for (int i = 0; i < a.digits; i++) {
                const u64 d = a.up[((size_t)i * a.T + k) * N + px];
                const size_t kidx = ((size_t)i * a.T * a.RB + (size_t)blk * a.T + k) * N + px;
                s1.mac(d, key[kidx]);
                s2.mac(d, key[half * a.dnum + kidx]);
            }
            const u64 b0 = a.pqT[limb + px + half];
            ea = barrett128(s1.value(0), p.q, p.mu_hi, p.mu_lo);
            eb = barrett128(s2.value(b0), p.q, p.mu_hi, p.mu_lo);
        }
#pragma unroll
        for (int i = 0; i < BS; i++)
            if (i < a.bs && j < a.acc_num[i]) {
                const u64 mx = a.plain[i * a.gs + j][(size_t)k * N + x];
                acc_a[i].mac(ea, mx);
                acc_b[i].mac(eb, mx);
            }
    }
#pragma unroll
    for (int i = 0; i < BS; i++)
        if (i < a.bs) {
            a.out[limb + x + (size_t)(2 * i) * half] = barrett128(acc_a[i].value(0), p.q, p.mu_hi, p.mu_lo);
            a.out[limb + x + (size_t)(2 * i + 1) * half] = barrett128(acc_b[i].value(0), p.q, p.mu_hi, p.mu_lo);
        }
}

struct BabyArgs {
    u64* out;                       // [a | b][Ri_blockNum][t_num], accumulated in place
    const u64* up;
    const u64* in;                  // the pair that is rotated; only its b half is read
    const PrimeConst* primes;
    const u64* key[MAX_GS];
    u64 pow[MAX_GS];
    long N;
    int logN, T, RB, dnum, digits, prime0, rot_num, blocks;
};
template <bool FAST>
__global__ __launch_bounds__(THREADS) void baby_rotate_kernel(BabyArgs a) {
    const TileIndex ti = tile_index(blockIdx.x, (int)(a.N / THREADS), a.T, a.blocks);
    const long x = (long)ti.chunk * THREADS + threadIdx.x;
    const int k = ti.k, blk = ti.blk;
    const PrimeConst p = a.primes[a.prime0 + k];
    const long N = a.N;
    const u64 mask = 2 * (u64)N - 1;
    const size_t half = (size_t)a.RB * a.T * N;
    const size_t limb = ((size_t)blk * a.T + k) * N;
    u64 oa = a.out[limb + x], ob = a.out[limb + x + half];
    bool any = false;
    for (int r = 0; r < a.rot_num; r++) {
        const u64* key = a.key[r];
        if (!key) continue;
        any = true;
        const long px = hoist_perm(a.pow[r], x, a.logN, mask);
        Acc<FAST> s1, s2;
        for (int i = 0; i < a.digits; i++) {
            const u64 d = a.up[((size_t)i * a.T + k) * N + px];
            const size_t kidx = ((size_t)i * a.T * a.RB + (size_t)blk * a.T + k) * N + px;
            s1.mac(d, key[kidx]);
            s2.mac(d, key[half * a.dnum + kidx]);
        }
        const u64 b0 = a.in[limb + px + half];
        u128w v1 = s1.value(oa), v2 = s2.value(b0);
        v2.lo += ob;
        v2.hi += (v2.lo < ob);
        oa = barrett128(v1, p.q, p.mu_hi, p.mu_lo);
        ob = barrett128(v2, p.q, p.mu_hi, p.mu_lo);
    }
    if (any) {
        a.out[limb + x] = oa;
        a.out[limb + x + half] = ob;
    }
}

struct MulPArgs {
    u64* out;
    const u64* cipher;
    const PrimeConst* primes;
    u64 pmod[MAX_LIMBS];
    long N;
    int K, L;
};
// limb K + i of the pair over [P | Q] = cipher limb i times P mod q_i; grid y runs over K + l + 1 limbs, the first K are zeroed
__global__ __launch_bounds__(THREADS) void cipher_mul_p_kernel(MulPArgs a) {
    const long x = (long)blockIdx.x * THREADS + threadIdx.x;
    const int limb = blockIdx.y, z = blockIdx.z;
    u64* dst = a.out + ((size_t)z * (a.K + a.L + 1) + limb) * a.N + x;
    if (limb < a.K) { *dst = 0; return; }
    const int i = limb - a.K;
    const PrimeConst p = a.primes[a.K + i];
    u128w acc{0, 0};
    mac128(acc, a.cipher[((size_t)z * (a.L + 1) + i) * a.N + x], a.pmod[i]);
    *dst = barrett128(acc, p.q, p.mu_hi, p.mu_lo);
}

__global__ __launch_bounds__(THREADS) void cipher_add_t_kernel(u64* a, const u64* b, const PrimeConst* primes, long N, int T, int prime0) {
    const long x = (long)blockIdx.x * THREADS + threadIdx.x;
    const int k = blockIdx.y, z = blockIdx.z;
    const size_t i = ((size_t)z * T + k) * N + x;
    a[i] = csub(a[i] + b[i], primes[prime0 + k].q);
}

__global__ __launch_bounds__(THREADS) void rescale_coeff_kernel(u64* a, const PrimeConst* primes, const u64* inv, const u64* inv_s, long N, int K, int q_num,
                                                                int l) {
    const long x = (long)blockIdx.x * THREADS + threadIdx.x;
    const int i = blockIdx.y, z = blockIdx.z;
    const u64 q = primes[K + i].q;
    const size_t idx = ((size_t)z * q_num + i) * N + x;
    const u64 ra = csub(a[idx] + 2 * q - a[((size_t)z * q_num + l) * N + x], q);
    a[idx] = mul_shoup(ra, inv[i], inv_s[i], q);
}

// the carry-free sums need every operand below 2^60 and at most 16 terms per sum
bool carry_free_ok(const ckks_ctx* c, int digits) {
    if (digits > 16 || c->arith_mode == 1) return false;
    for (int k = 0; k < c->t_num; k++)
        if (c->pqt[(size_t)c->p_num + c->q_num + k] >= (1ull << 60)) return false;
    return true;
}

int need_t_basis(const ckks_ctx* c, int l, const char* who) {
    if (!c) { set_error(std::string(who) + ": null context"); return CKKS_E_INVALID; }
    if (c->t_num == 0 || c->gamma == 0 || c->p_num == 0) { set_error(std::string(who) + ": needs the P and T bases"); return CKKS_E_INVALID; }
    if (l < 0 || l > c->L) { set_error(std::string(who) + ": level out of range"); return CKKS_E_INVALID; }
    return CKKS_OK;
}

}  // namespace

extern "C" int ckks_cipher_mul_p(ckks_ctx* c, uint64_t* out, const uint64_t* cipher, int l) {
    if (!c || !out || !cipher || l < 0 || l > c->L || c->p_num == 0 || l + 1 > MAX_LIMBS) { set_error("cipher_mul_P: bad argument or no P basis"); return CKKS_E_INVALID; }
    MulPArgs a;
    a.out = (u64*)out; a.cipher = (const u64*)cipher; a.primes = c->d_primes; a.N = c->N; a.K = c->K; a.L = c->L;
    for (int i = 0; i < MAX_LIMBS; i++) a.pmod[i] = i <= l ? c->PModqt[i] : 0;
    hipLaunchKernelGGL(cipher_mul_p_kernel, dim3((unsigned)(c->N / THREADS), c->K + l + 1, 2), dim3(THREADS), 0, c->stream, a);
    CKKS_HIP_TRY(hipGetLastError());
    return CKKS_OK;
}

extern "C" int ckks_cipher_add_t(ckks_ctx* c, uint64_t* a, const uint64_t* b, int blocks) {
    if (!c || !a || !b || blocks < 0 || c->t_num == 0) { set_error("cipher_add_T: bad argument or no T basis"); return CKKS_E_INVALID; }
    if (blocks == 0) return CKKS_OK;
    hipLaunchKernelGGL(cipher_add_t_kernel, dim3((unsigned)(c->N / THREADS), c->t_num, blocks), dim3(THREADS), 0, c->stream, (u64*)a, (const u64*)b,
                       c->d_primes, c->N, c->t_num, c->p_num + c->q_num);
    CKKS_HIP_TRY(hipGetLastError());
    return CKKS_OK;
}

extern "C" int ckks_rescale_coeff(ckks_ctx* c, uint64_t* cipher, int l) {
    if (!c || !cipher || l < 1 || l > c->L) { set_error("rescaleAndEqual_noNTT: bad argument or level 0"); return CKKS_E_INVALID; }
    const u64* inv = (const u64*)c->d_qiInvModql + (size_t)l * (l - 1) / 2;
    hipLaunchKernelGGL(rescale_coeff_kernel, dim3((unsigned)(c->N / THREADS), l, 2), dim3(THREADS), 0, c->stream, (u64*)cipher, c->d_primes, inv,
                       inv + c->qiInv_count, c->N, c->K, c->L + 1, l);
    CKKS_HIP_TRY(hipGetLastError());
    return CKKS_OK;
}

extern "C" int ckks_giant_rotate_mult_plain_t(ckks_ctx* c, uint64_t* bs_cipher_T, const uint64_t* PQ_to_T, const uint64_t* modUp_QjtoT,
                                              const uint64_t* const* rotKeys_host, const int* rotSlots_host, const uint64_t* const* plaintextT_host,
                                              const int* accNum_host, int bs, int gs, int l) {
    int rc = need_t_basis(c, l, "Giant_Rotate_And_Mult_PlaintT");
    if (rc != CKKS_OK) return rc;
    if (!bs_cipher_T || !PQ_to_T || !modUp_QjtoT || !rotKeys_host || !rotSlots_host || !plaintextT_host || !accNum_host) {
        set_error("Giant_Rotate_And_Mult_PlaintT: null argument");
        return CKKS_E_INVALID;
    }
    if (bs < 1 || bs > MAX_BS || gs < 1 || gs > MAX_GS) { set_error("Giant_Rotate_And_Mult_PlaintT: 1 <= bs <= 8 and 1 <= gs <= 16"); return CKKS_E_INVALID; }
    GiantArgs a;
    a.out = (u64*)bs_cipher_T; a.pqT = (const u64*)PQ_to_T; a.up = (const u64*)modUp_QjtoT; a.primes = c->d_primes;
    a.N = c->N; a.logN = c->logN; a.T = c->t_num; a.RB = c->Ri_blockNum; a.dnum = c->dnum;
    a.digits = (l + 1 + c->p_num - 1) / c->p_num; a.prime0 = c->p_num + c->q_num; a.bs = bs; a.gs = gs;
    if (a.digits > c->dnum) { set_error("hoisted rotations: the level needs more digits than the keys hold (q_num is no multiple of p_num)"); return CKKS_E_INVALID; }
    for (int j = 0; j < MAX_GS; j++) {
        a.key[j] = j < gs ? (const u64*)rotKeys_host[j] : nullptr;
        a.pow[j] = 1;
        if (j < gs && rotKeys_host[j]) {
            if (rotSlots_host[j] < 0) { set_error("Giant_Rotate_And_Mult_PlaintT: a key without its rotation"); return CKKS_E_INVALID; }
            if ((rc = ckks_rot_group(c, rotSlots_host[j], &a.pow[j]))) return rc;
        }
    }
    for (int i = 0; i < MAX_BS; i++) {
        a.acc_num[i] = i < bs ? accNum_host[i] : 0;
        if (a.acc_num[i] < 0 || a.acc_num[i] > gs) { set_error("Giant_Rotate_And_Mult_PlaintT: accNum outside 0..gs"); return CKKS_E_INVALID; }
    }
    for (int i = 0; i < MAX_BS * MAX_GS; i++) a.plain[i] = nullptr;
    for (int i = 0; i < bs; i++)
        for (int j = 0; j < a.acc_num[i]; j++) {
            a.plain[i * gs + j] = (const u64*)plaintextT_host[i * gs + j];
            if (!a.plain[i * gs + j]) { set_error("Giant_Rotate_And_Mult_PlaintT: a plaintext inside accNum is null"); return CKKS_E_INVALID; }
        }
    const int blockNum = (c->p_num + l + 1 + c->gamma - 1) / c->gamma;
    a.blocks = blockNum;
    const dim3 grid((unsigned)(c->N / THREADS) * (unsigned)c->t_num * (unsigned)blockNum), block(THREADS);
    if (carry_free_ok(c, a.digits)) {
        if (bs == 1) hipLaunchKernelGGL((giant_rotate_mult_kernel<1, true>), grid, block, 0, c->stream, a);
        else if (bs == 2) hipLaunchKernelGGL((giant_rotate_mult_kernel<2, true>), grid, block, 0, c->stream, a);
        else if (bs <= 4) hipLaunchKernelGGL((giant_rotate_mult_kernel<4, true>), grid, block, 0, c->stream, a);
        else hipLaunchKernelGGL((giant_rotate_mult_kernel<8, true>), grid, block, 0, c->stream, a);
    } else {
        if (bs == 1) hipLaunchKernelGGL((giant_rotate_mult_kernel<1, false>), grid, block, 0, c->stream, a);
        else if (bs == 2) hipLaunchKernelGGL((giant_rotate_mult_kernel<2, false>), grid, block, 0, c->stream, a);
        else if (bs <= 4) hipLaunchKernelGGL((giant_rotate_mult_kernel<4, false>), grid, block, 0, c->stream, a);
        else hipLaunchKernelGGL((giant_rotate_mult_kernel<8, false>), grid, block, 0, c->stream, a);
    }
    CKKS_HIP_TRY(hipGetLastError());
    return CKKS_OK;
}

extern "C" int ckks_baby_rotate(ckks_ctx* c, uint64_t* output, const uint64_t* modUp_QjtoT, const uint64_t* input, int rotNum,
                                const uint64_t* const* rotKeys_host, const int* rotSlots_host, int l) {
    int rc = need_t_basis(c, l, "Baby_Rotate");
    if (rc != CKKS_OK) return rc;
    if (!output || !modUp_QjtoT || !input || !rotKeys_host || !rotSlots_host) { set_error("Baby_Rotate: null argument"); return CKKS_E_INVALID; }
    if (rotNum < 0 || rotNum > MAX_GS) { set_error("Baby_Rotate: at most 16 rotations per call"); return CKKS_E_INVALID; }
    if (output == input) { set_error("Baby_Rotate: output and input must be different buffers"); return CKKS_E_INVALID; }
    BabyArgs a;
    a.out = (u64*)output; a.up = (const u64*)modUp_QjtoT; a.in = (const u64*)input; a.primes = c->d_primes;
    a.N = c->N; a.logN = c->logN; a.T = c->t_num; a.RB = c->Ri_blockNum; a.dnum = c->dnum;
    a.digits = (l + 1 + c->p_num - 1) / c->p_num; a.prime0 = c->p_num + c->q_num; a.rot_num = rotNum;
    if (a.digits > c->dnum) { set_error("hoisted rotations: the level needs more digits than the keys hold (q_num is no multiple of p_num)"); return CKKS_E_INVALID; }
    bool any = false;
    for (int r = 0; r < MAX_GS; r++) {
        a.key[r] = r < rotNum ? (const u64*)rotKeys_host[r] : nullptr;
        a.pow[r] = 1;
        if (a.key[r]) {
            if (rotSlots_host[r] < 0) { set_error("Baby_Rotate: a key without its rotation"); return CKKS_E_INVALID; }
            if ((rc = ckks_rot_group(c, rotSlots_host[r], &a.pow[r]))) return rc;
            any = true;
        }
    }
    if (!any) return CKKS_OK;
    const int blockNum = (c->p_num + l + 1 + c->gamma - 1) / c->gamma;
    a.blocks = blockNum;
    const dim3 grid((unsigned)(c->N / THREADS) * (unsigned)c->t_num * (unsigned)blockNum);
    if (carry_free_ok(c, a.digits)) hipLaunchKernelGGL(baby_rotate_kernel<true>, grid, dim3(THREADS), 0, c->stream, a);
    else hipLaunchKernelGGL(baby_rotate_kernel<false>, grid, dim3(THREADS), 0, c->stream, a);
    CKKS_HIP_TRY(hipGetLastError());
    return CKKS_OK;
}

extern "C" int ckks_bsgs_scratch_words(const ckks_ctx* c, int bs, size_t* words) {
    if (!c || !words || bs < 1 || bs > MAX_BS || c->t_num == 0) { set_error("bsgs_scratch_words: bad argument or no T basis"); return CKKS_E_INVALID; }
    const size_t N = (size_t)c->N, half = (size_t)c->Ri_blockNum * c->t_num * N;
    *words = N * c->t_num * c->Qj_blockNum + 2 * (size_t)(c->K + c->L + 1) * N + 2 * half * (size_t)(bs + 3);
    return CKKS_OK;
}

extern "C" int ckks_bsgs_level_23(ckks_ctx* c, uint64_t* cipher, int l, const uint64_t* const* plaintextT_host, const int* accNum_host,
                                  const int* rot_in_host, const uint64_t* const* rot_in_keys_host, const int* rot_out_host,
                                  const uint64_t* const* rot_out_keys_host, int bs, int gs, uint64_t* scratch) {
    int rc = need_t_basis(c, l, "bsgs_level_23");
    if (rc != CKKS_OK) return rc;
    if (!cipher || !plaintextT_host || !accNum_host || !rot_in_host || !rot_in_keys_host || !rot_out_host || !rot_out_keys_host || !scratch) {
        set_error("bsgs_level_23: null argument");
        return CKKS_E_INVALID;
    }
    if (bs < 1 || bs > MAX_BS || gs < 1 || gs > MAX_GS) { set_error("bsgs_level_23: 1 <= bs <= 8 and 1 <= gs <= 16"); return CKKS_E_INVALID; }
    for (int j = 0; j < gs; j++)
        if (rot_in_host[j] != 0 && !rot_in_keys_host[j]) { set_error("rotKey_23 not exists"); return CKKS_E_STATE; }
    for (int i = 1; i < bs; i++)
        if (rot_out_host[i] != 0 && !rot_out_keys_host[i]) { set_error("rotKey_23 not exists"); return CKKS_E_STATE; }
    const size_t N = (size_t)c->N;
    const int K = c->K, L = c->L, T = c->t_num, RB = c->Ri_blockNum;
    const int cipher_blockNum = (l + 1 + K - 1) / K, blockNum = (K + l + 1 + c->gamma - 1) / c->gamma;
    const size_t half = (size_t)RB * T * N;
    uint64_t* up = scratch;
    uint64_t* pq = up + N * T * c->Qj_blockNum;
    uint64_t* pqT = pq + 2 * (size_t)(K + L + 1) * N;
    uint64_t* gsT = pqT + 2 * half;
    uint64_t* back = gsT + 2 * half;
    uint64_t* bsT = back + 2 * half;
    if ((rc = ckks_modup_qj_to_t(c, up, cipher, l, 1))) return rc;                                                  // :262
    if ((rc = launch_ntt(c, up, 0, K + L + 1, cipher_blockNum, T, T, 0, 1, false))) return rc;                      // :263
    if ((rc = ckks_cipher_mul_p(c, pq, cipher, l))) return rc;                                                      // :267
    if ((rc = ckks_modup_pq_to_t(c, pqT, pq, l, 2))) return rc;                                                     // :270
    if ((rc = launch_ntt(c, pqT, 0, K + L + 1, blockNum, T, T, (long)RB * T, 2, false))) return rc;                 // :272
    const uint64_t* keys[MAX_GS];
    int slots[MAX_GS];
    for (int j = 0; j < gs; j++) { keys[j] = rot_in_host[j] != 0 ? rot_in_keys_host[j] : nullptr; slots[j] = rot_in_host[j] != 0 ? rot_in_host[j] : -1; }
    if ((rc = ckks_giant_rotate_mult_plain_t(c, bsT, pqT, up, keys, slots, plaintextT_host, accNum_host, bs, gs, l))) return rc;   // :308
    for (int i = 1; i < bs; i++) {                                                                                  // :326-356
        uint64_t* part = bsT + (size_t)i * 2 * half;
        if (rot_out_host[i] == 0) {
            if ((rc = ckks_cipher_add_t(c, bsT, part, RB * 2))) return rc;
            continue;
        }
        CKKS_HIP_TRY(hipMemcpyAsync(gsT, part, 2 * half * sizeof(uint64_t), hipMemcpyDeviceToDevice, c->stream));
        if ((rc = launch_ntt(c, part, 0, K + L + 1, blockNum, T, T, (long)RB * T, 2, true))) return rc;
        if ((rc = ckks_modup_t_to_pql(c, back, part, l, 1))) return rc;
        if ((rc = ckks_moddown_pql_to_ql(c, cipher, back, l, 1))) return rc;
        if ((rc = ckks_modup_qj_to_t(c, up, cipher, l, 1))) return rc;
        if ((rc = launch_ntt(c, up, 0, K + L + 1, cipher_blockNum, T, T, 0, 1, false))) return rc;
        const uint64_t* key1[1] = {rot_out_keys_host[i]};
        const int slot1[1] = {rot_out_host[i]};
        if ((rc = ckks_baby_rotate(c, bsT, up, gsT, 1, key1, slot1, l))) return rc;
    }
    if ((rc = launch_ntt(c, bsT, 0, K + L + 1, blockNum, T, T, (long)RB * T, 2, true))) return rc;                  // :359
    if ((rc = ckks_modup_t_to_pql(c, back, bsT, l, 2))) return rc;                                                  // :361
    return ckks_moddown_pql_to_ql(c, cipher, back, l, 2);                                                           // :363
}
