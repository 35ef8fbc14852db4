// Context construction: prime bookkeeping, twiddle and base-conversion tables, upload to the device.
// Replaces Context_23::Context_23 / preComputeOnCPU / copyMemoryToGPU (Context_23.cuh:12-701).  Primes are given
// by the caller instead of being switched on logN (Params.cuh), and every table lives in the handle instead of in
// process-global __constant__ symbols.
#include <algorithm>
#include <cstring>
#include <mutex>

#include "context.hpp"
#include "host_math.hpp"

namespace H = ckks_host;

namespace ckks {
static thread_local std::string g_err;
void set_error(const std::string& s) { g_err = s; }
int hip_fail(hipError_t e, const char* what) {
    g_err = std::string(what) + ": " + hipGetErrorString(e);
    return CKKS_E_HIP;
}
}  // namespace ckks

extern "C" const char* ckks_last_error(void) { return ckks::g_err.c_str(); }
extern "C" const char* ckks_version(void) { return "ckks_llm_amd 0.1 (gfx950)"; }

static int ceil_div(int a, int b) { return (a + b - 1) / b; }

template <class T>
static int upload(T** dptr, const std::vector<T>& v) {
    *dptr = nullptr;
    if (v.empty()) return CKKS_OK;
    CKKS_HIP_TRY(hipMalloc((void**)dptr, v.size() * sizeof(T)));
    CKKS_HIP_TRY(hipMemcpy(*dptr, v.data(), v.size() * sizeof(T), hipMemcpyHostToDevice));
    return CKKS_OK;
}

// floor(T/2) mod m with T = prod t_i odd: ((T mod 2m) - 1) / 2 mod m  (NTL arithmetic in Context_23.cuh:96-130)
static u64 half_product_mod(const std::vector<u64>& t, u64 m) {
    u64 m2 = 2 * m, r = 1;
    for (u64 x : t) r = H::mulmod(r, x % m2, m2);
    return ((r - 1) / 2) % m;
}

static double balanced_double(u64 x, u64 q) { return x > q / 2 ? -(double)(q - x) : (double)x; }

// builds the exact-conversion block "source primes src (pqt indices) -> target primes tgt"
static void fill_conv_block(ckks::ConvBlock& b, const std::vector<u64>& pqt, const std::vector<int>& src,
                            const std::vector<int>& src_limb, const std::vector<int>& tgt, const std::vector<int>& tgt_limb) {
    std::memset(&b, 0, sizeof(b));
    b.nsrc = (int)src.size();
    b.ntgt = (int)tgt.size();
    std::vector<u64> sp;
    for (int i : src) sp.push_back(pqt[i]);
    for (int j = 0; j < b.nsrc; j++) {
        b.src_prime[j] = (short)src[j];
        b.src_limb[j] = (short)src_limb[j];
        u64 hat = H::prod_mod(sp, 0, b.nsrc, j, sp[j]);
        b.hatinv[j] = H::invmod(hat, sp[j]);
        b.hatinv_s[j] = H::shoup(b.hatinv[j], sp[j]);
    }
    for (int k = 0; k < b.ntgt; k++) {
        u64 r = pqt[tgt[k]];
        b.tgt_prime[k] = (short)tgt[k];
        b.tgt_limb[k] = (short)tgt_limb[k];
        for (int j = 0; j < b.nsrc; j++) b.hat[k][j] = H::prod_mod(sp, 0, b.nsrc, j, r);
        b.dmod[k] = H::prod_mod(sp, 0, b.nsrc, -1, r);
    }
    // FP64 tables for the conversion kernel's double-precision path (all primes of the block below 2^41)
    b.f64_ok = 1;
    for (int i : src) if (pqt[i] >= (1ull << 41)) b.f64_ok = 0;
    for (int i : tgt) if (pqt[i] >= (1ull << 41)) b.f64_ok = 0;
    b.split_ok = 1;
    for (int i : tgt) if (pqt[i] >= (1ull << 50)) b.split_ok = 0;
    if (b.f64_ok)
        for (int j = 0; j < b.nsrc; j++) b.hatinv_d[j] = balanced_double(b.hatinv[j], sp[j]);
    if (b.f64_ok || b.split_ok) {
        for (int k = 0; k < b.ntgt; k++) {
            const u64 r = pqt[tgt[k]];
            for (int j = 0; j < b.nsrc; j++) {
                b.hat_d[k][j] = balanced_double(b.hat[k][j], r);
                b.hat31_d[k][j] = balanced_double(H::mulmod(b.hat[k][j], (1ull << 31) % r, r), r);
            }
            b.dmod_d[k] = balanced_double(b.dmod[k], r);
        }
    }
}

extern "C" int ckks_ctx_create(ckks_ctx** out, int logN, const uint64_t* p, int p_num, const uint64_t* q, int q_num,
                               const uint64_t* t, int t_num, int gamma) {
    if (!out) return CKKS_E_INVALID;
    *out = nullptr;
    if (logN < 8 || logN > 16 || q_num < 1 || p_num < 0 || t_num < 0 || gamma < 0 || (t_num > 0 && gamma < 1) ||
        (q_num > 0 && !q) || (p_num > 0 && !p) || (t_num > 0 && !t)) {
        ckks::set_error("ckks_ctx_create: need 8 <= logN <= 16, q_num >= 1, gamma >= 1 when t_num > 0");
        return CKKS_E_INVALID;
    }
    if (gamma > ckks::CONV_MAX_SRC || p_num > ckks::CONV_MAX_SRC || t_num > ckks::CONV_MAX_SRC ||
        p_num + q_num > 2 * ckks::CONV_MAX_TGT) {
        ckks::set_error("ckks_ctx_create: basis too large (gamma, p_num, t_num <= 16)");
        return CKKS_E_INVALID;
    }
    const long N = 1L << logN;
    std::vector<u64> pqt;
    for (int i = 0; i < p_num; i++) pqt.push_back(p[i]);
    for (int i = 0; i < q_num; i++) pqt.push_back(q[i]);
    for (int i = 0; i < t_num; i++) pqt.push_back(t[i]);
    for (u64 m : pqt) {
        if (m < 3 || (m & 1) == 0 || m >= (1ull << 62) || (m - 1) % (2 * (u64)N) != 0) {
            ckks::set_error("ckks_ctx_create: every modulus must be an odd prime < 2^62 with m = 1 mod 2N");
            return CKKS_E_INVALID;
        }
    }
    ckks_ctx* c = new ckks_ctx();
    c->logN = logN; c->N = N; c->p_num = p_num; c->q_num = q_num; c->t_num = t_num; c->gamma = gamma;
    c->L = q_num - 1; c->K = p_num;
    c->dnum = p_num ? q_num / p_num : 0;                                   // Context_23.cuh:29
    c->Ri_blockNum = gamma ? ceil_div(p_num + q_num, gamma) : 0;           // :32
    c->Qj_blockNum = p_num ? ceil_div(q_num, p_num) : 0;                   // :33
    c->pqt = pqt;
    c->nprimes = (int)pqt.size();
    const int tot = c->nprimes, K = p_num, L = c->L, PQ = p_num + q_num;
    std::vector<u64> pV(pqt.begin(), pqt.begin() + K), qV(pqt.begin() + K, pqt.begin() + PQ), tV(pqt.begin() + PQ, pqt.end());

    // ---- per-prime constants and twiddle tables ----
    c->mu_hi.resize(tot); c->mu_lo.resize(tot); c->psi.resize(tot); c->psiinv.resize(tot);
    c->n_inv.resize(tot); c->n_inv_shoup.resize(tot); c->halfTmodpqti.resize(tot); c->f64_ok.resize(tot);
    c->psi_table.resize((size_t)tot * N); c->psiinv_table.resize((size_t)tot * N);
    std::vector<ckks::PrimeConst> pc(tot);
    std::vector<ulonglong2> twf((size_t)tot * N), twi((size_t)tot * N);
    std::vector<double> twdf((size_t)tot * N, 0.0), twdi((size_t)tot * N, 0.0);
    for (int i = 0; i < tot; i++) {
        const u64 m = pqt[i];
        H::barrett_mu(m, c->mu_hi[i], c->mu_lo[i]);
        u64 psi = H::mth_root(2 * (u64)N, m);
        if (psi == 0 || H::powmod(psi, (u64)N, m) != m - 1) {
            delete c;
            ckks::set_error("ckks_ctx_create: no primitive 2N-th root found (modulus not prime?)");
            return CKKS_E_INVALID;
        }
        c->psi[i] = psi;
        c->psiinv[i] = H::invmod(psi, m);
        c->n_inv[i] = H::invmod((u64)N % m, m);
        c->n_inv_shoup[i] = H::shoup(c->n_inv[i], m);
        c->halfTmodpqti[i] = t_num ? half_product_mod(tV, m) : 0;
        c->f64_ok[i] = m < (1ull << 41);
        // powers in natural order, scattered to bit-reversed positions (table convention of Utils.cuh:190-201)
        u64* pt = &c->psi_table[(size_t)i * N];
        u64* it = &c->psiinv_table[(size_t)i * N];
        u64 pw = 1, ipw = 1;
        for (long k = 0; k < N; k++) {
            uint32_t r = H::bitrev((uint32_t)k, logN);
            pt[r] = pw; it[r] = ipw;
            pw = H::mulmod(pw, psi, m);
            ipw = H::mulmod(ipw, c->psiinv[i], m);
        }
        it[1] = H::mulmod(it[1], c->n_inv[i], m);                          // Utils.cuh:200
        for (long k = 0; k < N; k++) {
            twf[(size_t)i * N + k] = make_ulonglong2(pt[k], H::shoup(pt[k], m));
            twi[(size_t)i * N + k] = make_ulonglong2(it[k], H::shoup(it[k], m));
            if (m < (1ull << 50)) {                                            // FP64 back ends: below 2^41, and the wide one below 2^50
                twdf[(size_t)i * N + k] = balanced_double(pt[k], m);
                twdi[(size_t)i * N + k] = balanced_double(it[k], m);
            }
        }
        ckks::PrimeConst& P = pc[i];
        P.q = m; P.mu_hi = c->mu_hi[i]; P.mu_lo = c->mu_lo[i];
        P.n_inv = c->n_inv[i]; P.n_inv_s = c->n_inv_shoup[i];
        P.w1n = it[1]; P.w1n_s = H::shoup(it[1], m);
        P.qd = (double)m; P.qinv_d = 1.0 / (double)m;
        P.n_inv_d = balanced_double(c->n_inv[i], m); P.w1n_d = balanced_double(it[1], m);
        P.f64_ok = c->f64_ok[i]; P.pad = 0;
    }

    // ---- reference-named constant tables (host copies; layouts as uploaded at Context_23.cuh:528-701) ----
    for (int l = 0; l <= L; l++)
        for (int i = 0; i < K; i++) c->pHatVecModq.push_back(H::prod_mod(pV, 0, K, i, qV[l]));         // :162-176
    std::vector<u64> pHatInv_s;
    for (int i = 0; i < K; i++) {                                                                       // :178-190
        u64 v = H::invmod(H::prod_mod(pV, 0, K, i, pV[i]), pV[i]);
        c->pHatInvVecModp.push_back(v);
        pHatInv_s.push_back(H::shoup(v, pV[i]));
    }
    std::vector<u64> PinvModq_s;
    for (int i = 0; i <= L; i++) {                                                                      // :397-410
        u64 v = H::prod_mod(pV, 0, K, -1, qV[i]);
        c->PModqt.push_back(v);
        u64 w = H::invmod(v, qV[i]);
        c->PinvModq.push_back(w);
        PinvModq_s.push_back(H::shoup(w, qV[i]));
    }
    for (int i = 0; i < t_num; i++) c->PModqt.push_back(H::prod_mod(pV, 0, K, -1, tV[i]));              // :412-421
    std::vector<u64> qiInv_s;
    for (int l = 1; l <= L; l++)                                                                        // :425-436
        for (int j = 0; j < l; j++) {
            u64 v = H::invmod(qV[l] % qV[j], qV[j]);
            c->qiInvModql.push_back(v);
            qiInv_s.push_back(H::shoup(v, qV[j]));
        }
    if (gamma > 0 && t_num > 0) {                                                                       // :232-283
        c->RiHatInv.assign((size_t)c->Ri_blockNum * gamma, 0);
        c->RiHatModT.assign((size_t)c->Ri_blockNum * t_num * gamma, 0);
        c->Rimodti.assign((size_t)t_num * c->Ri_blockNum, 0);
        for (int i = 0; i < c->Ri_blockNum; i++) {
            int lo = i * gamma, hi = std::min(lo + gamma, PQ);
            for (int j = lo; j < hi; j++)
                c->RiHatInv[(size_t)i * gamma + (j - lo)] = H::invmod(H::prod_mod(pqt, lo, hi, j, pqt[j]), pqt[j]);
            for (int k = 0; k < t_num; k++) {
                for (int j = lo; j < hi; j++)
                    c->RiHatModT[(size_t)i * t_num * gamma + (size_t)k * gamma + (j - lo)] = H::prod_mod(pqt, lo, hi, j, tV[k]);
                c->Rimodti[(size_t)k * c->Ri_blockNum + i] = H::prod_mod(pqt, lo, hi, -1, tV[k]);
            }
        }
    }
    if (p_num > 0 && t_num > 0) {                                                                       // :286-351
        const int B = c->Qj_blockNum;
        c->QjHatInv.assign((size_t)(L + 1) * B * p_num, 0);
        c->QjHatModT.assign((size_t)(L + 1) * B * t_num * p_num, 0);
        c->Qjmodti.assign((size_t)(L + 1) * B * t_num, 0);
        for (int l = 0; l <= L; l++)
            for (int i = 0; i < ceil_div(l + 1, p_num); i++) {
                int lo = i * p_num, hi = std::min(lo + p_num, l + 1);
                for (int j = lo; j < hi; j++)
                    c->QjHatInv[(size_t)l * B * p_num + (size_t)i * p_num + (j - lo)] = H::invmod(H::prod_mod(qV, lo, hi, j, qV[j]), qV[j]);
                for (int k = 0; k < t_num; k++) {
                    for (int j = lo; j < hi; j++)
                        c->QjHatModT[(size_t)l * B * t_num * p_num + (size_t)i * t_num * p_num + (size_t)k * p_num + (j - lo)] =
                            H::prod_mod(qV, lo, hi, j, tV[k]);
                    c->Qjmodti[(size_t)l * B * t_num + (size_t)i * t_num + k] = H::prod_mod(qV, lo, hi, -1, tV[k]);
                }
            }
    }
    for (int i = 0; i < t_num; i++) c->THatInv.push_back(H::invmod(H::prod_mod(tV, 0, t_num, i, tV[i]), tV[i]));   // :354-367
    for (int i = 0; i < PQ && t_num > 0; i++) {                                                        // :369-393
        for (int j = 0; j < t_num; j++) c->THatModRi.push_back(H::prod_mod(tV, 0, t_num, j, pqt[i]));
        c->Tmodpqi.push_back(H::prod_mod(tV, 0, t_num, -1, pqt[i]));
    }

    // ---- conversion plans: one ConvBlock per (map, level, block) ----
    std::vector<ckks::ConvBlock> blocks;
    auto iota = [](int lo, int hi) { std::vector<int> v; for (int i = lo; i < hi; i++) v.push_back(i); return v; };
    c->plan_pq_to_t.resize(L + 1); c->plan_qj_to_t.resize(L + 1); c->plan_t_to_pq.resize(L + 1); c->plan_hybrid.resize(L + 1);
    c->plan_hybrid_all.resize(L + 1);
    for (int l = 0; l <= L; l++) {
        if (gamma > 0 && t_num > 0) {
            // [P|Q] gamma-block -> T (BasisConv.cuh:7-79).  The constants are those of the WHOLE block of [P|Q_L]
            // even when level l cuts the block short (reference behaviour: tables are level independent).
            int nb = ceil_div(p_num + l + 1, gamma);
            c->plan_pq_to_t[l].first = (int)blocks.size(); c->plan_pq_to_t[l].count = nb;
            for (int b = 0; b < nb; b++) {
                int lo = b * gamma, hi_full = std::min(lo + gamma, PQ), hi = std::min(lo + gamma, p_num + l + 1);
                std::vector<int> tg, tl;
                for (int k = 0; k < t_num; k++) { tg.push_back(PQ + k); tl.push_back(b * t_num + k); }
                ckks::ConvBlock blk;
                fill_conv_block(blk, pqt, iota(lo, hi_full), iota(lo, hi_full), tg, tl);
                blk.nsrc = hi - lo;      // residues actually summed (BasisConv.cuh:21)
                blocks.push_back(blk);
            }
            // T -> gamma-block of [P|Q_l], centred (BasisConv.cuh:183-254)
            c->plan_t_to_pq[l].first = (int)blocks.size(); c->plan_t_to_pq[l].count = nb;
            for (int b = 0; b < nb; b++) {
                int lo = b * gamma, hi = std::min(lo + gamma, p_num + l + 1);
                std::vector<int> sl;
                for (int k = 0; k < t_num; k++) sl.push_back(b * t_num + k);
                ckks::ConvBlock blk;
                fill_conv_block(blk, pqt, iota(PQ, PQ + t_num), sl, iota(lo, hi), iota(lo, hi));
                for (int k = 0; k < t_num; k++) blk.add_in[k] = c->halfTmodpqti[PQ + k];
                for (int k = 0; k < hi - lo; k++) blk.sub_out[k] = c->halfTmodpqti[lo + k];
                blocks.push_back(blk);
            }
        }
        if (p_num > 0 && t_num > 0) {
            // digit of p_num Q-primes -> T (BasisConv.cuh:84-179)
            int nb = ceil_div(l + 1, p_num);
            c->plan_qj_to_t[l].first = (int)blocks.size(); c->plan_qj_to_t[l].count = nb;
            for (int b = 0; b < nb; b++) {
                int lo = b * p_num, hi = std::min(lo + p_num, l + 1);
                std::vector<int> tg, tl;
                for (int k = 0; k < t_num; k++) { tg.push_back(PQ + k); tl.push_back(b * t_num + k); }
                ckks::ConvBlock blk;
                fill_conv_block(blk, pqt, iota(p_num + lo, p_num + hi), iota(lo, hi), tg, tl);
                blocks.push_back(blk);
            }
        }
        if (p_num > 0) {
            // textbook hybrid: digit of p_num Q-primes -> every other prime of [P | Q_l]; the digit's own limbs are copied
            int nb = ceil_div(l + 1, p_num);
            c->plan_hybrid[l].first = (int)blocks.size(); c->plan_hybrid[l].count = nb;
            for (int b = 0; b < nb; b++) {
                int lo = b * p_num, hi = std::min(lo + p_num, l + 1);
                std::vector<int> tg;
                for (int r = 0; r < p_num + l + 1; r++)
                    if (r < p_num + lo || r >= p_num + hi) tg.push_back(r);
                if ((int)tg.size() > ckks::CONV_MAX_TGT) {
                    delete c;
                    ckks::set_error("ckks_ctx_create: p_num + q_num too large for the hybrid conversion plan");
                    return CKKS_E_INVALID;
                }
                ckks::ConvBlock blk;
                fill_conv_block(blk, pqt, iota(p_num + lo, p_num + hi), iota(lo, hi), tg, tg);
                blk.ncopy = hi - lo;
                for (int j = 0; j < hi - lo; j++) { blk.copy_prime[j] = (short)(lo + j); blk.copy_limb[j] = (short)(p_num + lo + j); }
                blocks.push_back(blk);
            }
            // the same digits with EVERY prime of [P | Q_l] as a target, target k = prime k (for a prime of the digit itself the
            // constants reduce to "the residue back": (D/d_j) mod d_j0 = 0 for j != j0, D mod d_j0 = 0), for the key switch whose
            // ModUp runs inside the first pass of the digits' forward transform
            if (p_num + l + 1 <= ckks::CONV_MAX_TGT) {
                c->plan_hybrid_all[l].first = (int)blocks.size(); c->plan_hybrid_all[l].count = nb;
                for (int b = 0; b < nb; b++) {
                    int lo = b * p_num, hi = std::min(lo + p_num, l + 1);
                    ckks::ConvBlock blk;
                    fill_conv_block(blk, pqt, iota(p_num + lo, p_num + hi), iota(lo, hi), iota(0, p_num + l + 1), iota(0, p_num + l + 1));
                    blocks.push_back(blk);
                }
            }
        }
    }

    for (auto* plans : {&c->plan_pq_to_t, &c->plan_qj_to_t, &c->plan_t_to_pq, &c->plan_hybrid, &c->plan_hybrid_all})
        for (ckks::ConvPlan& pl : *plans) {
            pl.f64_ok = pl.count > 0;
            for (int b = 0; b < pl.count; b++) pl.f64_ok = pl.f64_ok && blocks[pl.first + b].f64_ok;
            pl.split_ok = pl.count > 0;
            for (int b = 0; b < pl.count; b++) pl.split_ok = pl.split_ok && blocks[pl.first + b].split_ok;
            for (int b = 0; b < pl.count; b++) pl.max_tgt = std::max(pl.max_tgt, blocks[pl.first + b].ntgt);
        }

    // ---- upload ----
    int rc = CKKS_OK;
    auto up = [&](int r) { if (rc == CKKS_OK) rc = r; };
    up(upload(&c->d_primes, pc));
    {
        // The same constants with N^-1 (and the last inverse twiddle, which carries N^-1) of every special prime p_i multiplied by
        // (P/p_i)^-1 mod p_i: an inverse transform run with this table leaves, on the special-prime limbs, the scaled residues that
        // ModDown starts from (BasisConv.cuh:283-289) instead of the plain coefficients.  FP64 back end only.
        std::vector<ckks::PrimeConst> pm = pc;
        for (int i = 0; i < K; i++) {
            pm[i].n_inv_d = balanced_double(H::mulmod(pc[i].n_inv, c->pHatInvVecModp[i], pV[i]), pV[i]);
            pm[i].w1n_d = balanced_double(H::mulmod(pc[i].w1n, c->pHatInvVecModp[i], pV[i]), pV[i]);
        }
        up(upload(&c->d_primes_moddown, pm));
    }
    if (p_num > 0) {
        // One table per level l with N^-1 (and the last inverse twiddle) of every prime q_i, i <= l, multiplied by (D/q_i)^-1 mod q_i,
        // D = the product of the primes of q_i's digit at that level: an inverse transform run with it leaves the scaled residues
        // y_i that the exact conversion starts from (BasisConv.cuh:18-24).  FP64 back end only.
        std::vector<ckks::PrimeConst> pu;
        for (int l = 0; l <= L; l++) {
            std::vector<ckks::PrimeConst> t = pc;
            for (int b = 0; b < c->plan_hybrid[l].count; b++) {
                const ckks::ConvBlock& blk = blocks[c->plan_hybrid[l].first + b];
                for (int j = 0; j < blk.nsrc; j++) {
                    const int i = blk.src_prime[j];
                    t[i].n_inv_d = balanced_double(H::mulmod(pc[i].n_inv, blk.hatinv[j], pqt[i]), pqt[i]);
                    t[i].w1n_d = balanced_double(H::mulmod(pc[i].w1n, blk.hatinv[j], pqt[i]), pqt[i]);
                }
            }
            pu.insert(pu.end(), t.begin(), t.end());
        }
        up(upload(&c->d_primes_modup, pu));
    }
    up(upload(&c->d_tw_fwd, twf));
    up(upload(&c->d_tw_inv, twi));
    up(upload(&c->d_twd_fwd, twdf));
    up(upload(&c->d_twd_inv, twdi));
    up(upload(&c->d_conv, blocks));
    up(upload(&c->d_pHatVecModq, c->pHatVecModq));
    {
        std::vector<u64> v = c->pHatInvVecModp; v.insert(v.end(), pHatInv_s.begin(), pHatInv_s.end());
        up(upload(&c->d_pHatInvVecModp, v));
        std::vector<u64> w = c->PinvModq; w.insert(w.end(), PinvModq_s.begin(), PinvModq_s.end());
        up(upload(&c->d_PinvModq, w));
        c->qiInv_count = c->qiInvModql.size();
        std::vector<u64> z = c->qiInvModql; z.insert(z.end(), qiInv_s.begin(), qiInv_s.end());
        up(upload(&c->d_qiInvModql, z));
    }
    if (rc == CKKS_OK) {
        int dev = 0, cus = 0;
        if (hipGetDevice(&dev) == hipSuccess && hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && cus > 0) c->cu_count = cus;
        c->device = dev;
        if (rc == CKKS_OK) rc = ckks::ntt_noalloc_init(nullptr);
        if (rc == CKKS_OK && c->logN == 16) rc = ckks::ntt_pair_init(c);
    }
    if (rc == CKKS_OK && hipEventCreate(&c->ev0) != hipSuccess) rc = CKKS_E_HIP;
    if (rc == CKKS_OK && hipEventCreate(&c->ev1) != hipSuccess) rc = CKKS_E_HIP;
    if (rc == CKKS_OK && hipEventCreate(&c->ev_mid) != hipSuccess) rc = CKKS_E_HIP;
    if (rc != CKKS_OK) { ckks_ctx_destroy(c); return rc; }
    *out = c;
    return CKKS_OK;
}

extern "C" int ckks_ctx_destroy(ckks_ctx* c) {
    if (!c) return CKKS_OK;
    (void)hipDeviceSynchronize();
    void* ptrs[] = {c->d_primes, c->d_primes_moddown, c->d_primes_modup, c->d_tw_fwd, c->d_tw_inv, c->d_twd_fwd, c->d_twd_inv, c->d_conv, c->d_pHatVecModq,
                    c->d_pHatInvVecModp, c->d_PinvModq, c->d_qiInvModql, c->d_ntt_chain, c->d_ntt_mid};
    for (void* p : ptrs) if (p) (void)hipFree(p);
    if (c->d_ntt_pair) (void)hipFree(c->d_ntt_pair);
    if (c->h_pair_fail) (void)hipHostFree(c->h_pair_fail);
    for (auto& e : c->decode_tabs) (void)hipFree(e.dev);
    for (hipEvent_t e : c->ev_marks) if (e) (void)hipEventDestroy(e);
    if (c->ev0) (void)hipEventDestroy(c->ev0);
    if (c->ev1) (void)hipEventDestroy(c->ev1);
    if (c->ev_mid) (void)hipEventDestroy(c->ev_mid);
    delete c;
    return CKKS_OK;
}

extern "C" int ckks_set_stream(ckks_ctx* c, void* s) {
    if (!c) return CKKS_E_INVALID;
    c->stream = (hipStream_t)s;
    return CKKS_OK;
}

extern "C" int ckks_ctx_info(const ckks_ctx* c, const char* name, long* value) {
    if (!c || !name || !value) return CKKS_E_INVALID;
    std::string n(name);
    if (n == "N") *value = c->N; else if (n == "logN") *value = c->logN;
    else if (n == "p_num") *value = c->p_num; else if (n == "q_num") *value = c->q_num; else if (n == "t_num") *value = c->t_num;
    else if (n == "gamma") *value = c->gamma; else if (n == "dnum") *value = c->dnum;
    else if (n == "Ri_blockNum") *value = c->Ri_blockNum; else if (n == "Qj_blockNum") *value = c->Qj_blockNum;
    else if (n == "arith_mode") *value = c->arith_mode; else if (n == "ntt_mode") *value = c->ntt_mode;
    else if (n == "ntt_mid_bytes") *value = (long)c->ntt_mid_cap;      // size of the inter-pass buffer the ordinary entry points have grown so far
    else if (n == "ntt_resident_round") *value = c->logN == 16 ? ckks::ntt_resident_round(c) : 0;      // limbs per round of the resident transform (0: it never applies)
    else if (n == "ntt_chain_deferred_tiles") return ckks::ntt_chain_deferred(const_cast<ckks_ctx*>(c), value);
    else if (n == "ntt_pair_deferred_tiles") return ckks::ntt_pair_deferred(const_cast<ckks_ctx*>(c), value);
    else if (n == "ntt_pair_stolen_tiles") return ckks::ntt_pair_deferred(const_cast<ckks_ctx*>(c), value, true);
    else if (n == "ntt_pair_resident_blocks") *value = c->pair_resident_blocks[ckks::PAIR_KIND_F64];      // of the FP64 transform kernel
    else if (n == "ntt_pair_resident_blocks_int") *value = c->pair_resident_blocks[ckks::PAIR_KIND_INT];
    else if (n == "ntt_extra_forms") *value = ckks::ntt_extra_forms();
    else { ckks::set_error("ckks_ctx_info: unknown name " + n); return CKKS_E_INVALID; }
    return CKKS_OK;
}

// test / tuning hook: 0 = automatic back end choice, 1 = force the integer back end
extern "C" int ckks_ctx_set_arith_mode(ckks_ctx* c, int mode) {
    if (!c || mode < 0 || mode > 1) return CKKS_E_INVALID;
    c->arith_mode = mode;
    return CKKS_OK;
}

// test / tuning hook: 0 = automatic, 1 = two launches per transform, 2 = chained one-launch transform wherever that kernel exists
// (N >= 2^15), 3 = one workgroup per limb wherever that kernel exists (N >= 2^15), 4 = paired one-launch transform at every batch
// size (N = 2^16; the automatic mode takes it for small batches), 5 = the same with the tiles of a limb spread over all XCDs
// (the automatic mode's choice between 41 and 128 limbs), 6 = the resident transform wherever it applies (N = 2^16, primes below
// 2^36, at least one limb per compute unit; the automatic mode takes it there too)
extern "C" int ckks_ctx_set_ntt_mode(ckks_ctx* c, int mode) {
    if (!c || mode < 0 || mode > 6) return CKKS_E_INVALID;
    c->ntt_mode = mode;
    return CKKS_OK;
}

// test / tuning switches of a context, by name
extern "C" int ckks_ctx_set_option(ckks_ctx* c, const char* name, long value) {
    if (!c || !name) return CKKS_E_INVALID;
    const std::string n(name);
    if (n == "ks_split") c->ks_split = value != 0;
    else if (n == "ks_back_split") c->ks_back_split = value != 0;
    else if (n == "conv_int") c->conv_int = value != 0;
    else if (n == "ntt_no_reverse") c->ntt_no_reverse = value != 0;
    else if (n == "pair_no_steal") c->pair_no_steal = value != 0;
    else if (n == "ntt_chunk") { if (value < 0 || value > 65535) return CKKS_E_INVALID; c->ntt_chunk = (int)value; }
    else { ckks::set_error("ckks_ctx_set_option: unknown name " + n); return CKKS_E_INVALID; }
    return CKKS_OK;
}

// test / tuning hook of the chained transform: skew = how many limbs a chain's first pass runs ahead of its second pass (0: default),
// spin_max = polls a second-pass workgroup spends on its limb's completion word before it leaves its tile to the finishing launch
// (-1: default; 0 sends every tile there, which is how the tests reach that path)
extern "C" int ckks_ctx_set_ntt_chain(ckks_ctx* c, int skew, int spin_max) {
    if (!c || skew < 0 || skew > 64 || spin_max < -1) return CKKS_E_INVALID;
    c->chain_skew = skew;
    c->chain_spin = spin_max;
    return CKKS_OK;
}

// Waits for the context's stream and reports what HIP has to say about the launches so far.
extern "C" int ckks_ctx_check(ckks_ctx* c) {
    if (!c) return CKKS_E_INVALID;
    CKKS_HIP_TRY(hipStreamSynchronize(c->stream));
    CKKS_HIP_TRY(hipGetLastError());
    if (ckks::ntt_pair_failed(c)) { ckks::set_error("NTT: a one-launch transform gave up waiting for its first pass; its output is incomplete"); return CKKS_E_UNAVAILABLE; }
    return CKKS_OK;
}

extern "C" int ckks_ctx_table(const ckks_ctx* c, const char* name, uint64_t* host_out, size_t cap, size_t* count) {
    if (!c || !name) return CKKS_E_INVALID;
    std::string n(name);
    const std::vector<uint64_t>* v = nullptr;
    std::vector<uint64_t> tmp;
    if (n == "pqt") v = &c->pqt; else if (n == "mu_hi") v = &c->mu_hi; else if (n == "mu_lo") v = &c->mu_lo;
    else if (n == "psi") v = &c->psi; else if (n == "psiinv") v = &c->psiinv; else if (n == "n_inv") v = &c->n_inv;
    else if (n == "n_inv_shoup") v = &c->n_inv_shoup; else if (n == "halfTmodpqti") v = &c->halfTmodpqti;
    else if (n == "psi_table") v = &c->psi_table; else if (n == "psiinv_table") v = &c->psiinv_table;
    else if (n == "pHatVecModq") v = &c->pHatVecModq; else if (n == "pHatInvVecModp") v = &c->pHatInvVecModp;
    else if (n == "PModqt") v = &c->PModqt; else if (n == "PinvModq") v = &c->PinvModq;
    else if (n == "RiHatInv") v = &c->RiHatInv; else if (n == "RiHatModT") v = &c->RiHatModT; else if (n == "Rimodti") v = &c->Rimodti;
    else if (n == "QjHatInv") v = &c->QjHatInv; else if (n == "QjHatModT") v = &c->QjHatModT; else if (n == "Qjmodti") v = &c->Qjmodti;
    else if (n == "THatInv") v = &c->THatInv; else if (n == "THatModRi") v = &c->THatModRi; else if (n == "Tmodpqi") v = &c->Tmodpqi;
    else if (n == "qiInvModql") v = &c->qiInvModql;
    else if (n == "psi_shoup_table" || n == "psiinv_shoup_table") {
        const std::vector<uint64_t>& src = n == "psi_shoup_table" ? c->psi_table : c->psiinv_table;
        tmp.resize(src.size());
        for (size_t i = 0; i < src.size(); i++) tmp[i] = H::shoup(src[i], c->pqt[i / c->N]);
        v = &tmp;
    }
    if (!v) { ckks::set_error("ckks_ctx_table: unknown table " + n); return CKKS_E_INVALID; }
    if (count) *count = v->size();
    if (host_out) {
        if (cap < v->size()) { ckks::set_error("ckks_ctx_table: buffer too small"); return CKKS_E_INVALID; }
        std::memcpy(host_out, v->data(), v->size() * sizeof(uint64_t));
    }
    return CKKS_OK;
}

// ---- plumbing ----
extern "C" int ckks_malloc(void** p, size_t bytes) {
    if (!p) return CKKS_E_INVALID;
    hipError_t e = hipMalloc(p, bytes);
    if (e == hipErrorOutOfMemory) { ckks::set_error("ckks_malloc: out of device memory"); return CKKS_E_NOMEM; }
    if (e != hipSuccess) return ckks::hip_fail(e, "hipMalloc");
    return CKKS_OK;
}
// Freeing or overwriting device memory through these calls also drops what the ring-pack handles had prepared from it (the digit
// planes of a weight matrix are keyed by its address).
extern "C" int ckks_free(void* p) {
    if (!p) return CKKS_OK;
    hipDeviceptr_t base = nullptr;
    size_t size = 0;
    if (hipMemGetAddressRange(&base, &size, (hipDeviceptr_t)p) == hipSuccess && size) pcmm_forget_weights(base, size, true);
    else { (void)hipGetLastError(); pcmm_forget_weights(p, 1, true); }
    CKKS_HIP_TRY(hipFree(p));
    return CKKS_OK;
}
extern "C" int ckks_memcpy_h2d(void* d, const void* s, size_t n) { pcmm_forget_weights(d, n); CKKS_HIP_TRY(hipMemcpy(d, s, n, hipMemcpyHostToDevice)); return CKKS_OK; }
extern "C" int ckks_memcpy_d2h(void* d, const void* s, size_t n) { CKKS_HIP_TRY(hipMemcpy(d, s, n, hipMemcpyDeviceToHost)); return CKKS_OK; }
extern "C" int ckks_memcpy_d2d(void* d, const void* s, size_t n) { pcmm_forget_weights(d, n); CKKS_HIP_TRY(hipMemcpy(d, s, n, hipMemcpyDeviceToDevice)); return CKKS_OK; }
extern "C" int ckks_memset(void* d, int v, size_t n) { pcmm_forget_weights(d, n); CKKS_HIP_TRY(hipMemset(d, v, n)); return CKKS_OK; }
extern "C" int ckks_sync(void) { CKKS_HIP_TRY(hipDeviceSynchronize()); return CKKS_OK; }
extern "C" int ckks_device_count(int* n) { if (!n) return CKKS_E_INVALID; CKKS_HIP_TRY(hipGetDeviceCount(n)); return CKKS_OK; }
extern "C" int ckks_timer_start(ckks_ctx* c) { if (!c) return CKKS_E_INVALID; CKKS_HIP_TRY(hipEventRecord(c->ev0, c->stream)); return CKKS_OK; }
extern "C" int ckks_timer_stop(ckks_ctx* c, float* ms) {
    if (!c || !ms) return CKKS_E_INVALID;
    CKKS_HIP_TRY(hipEventRecord(c->ev1, c->stream));
    CKKS_HIP_TRY(hipEventSynchronize(c->ev1));
    CKKS_HIP_TRY(hipEventElapsedTime(ms, c->ev0, c->ev1));
    return CKKS_OK;
}

// Marks on the context's stream, read back in pairs: a caller that queues many launches back to back puts a mark between them
// (an event record; nothing waits) and asks for the intervals once the work is done.
constexpr int TIMER_MAX_MARKS = 4096;
extern "C" int ckks_timer_mark(ckks_ctx* c, int slot) {
    if (!c || slot < 0 || slot >= TIMER_MAX_MARKS) { ckks::set_error("timer_mark: slot outside 0 .. 4095"); return CKKS_E_INVALID; }
    if ((size_t)slot >= c->ev_marks.size()) c->ev_marks.resize((size_t)slot + 1, nullptr);
    if (!c->ev_marks[slot]) CKKS_HIP_TRY(hipEventCreate(&c->ev_marks[slot]));
    CKKS_HIP_TRY(hipEventRecord(c->ev_marks[slot], c->stream));
    return CKKS_OK;
}
extern "C" int ckks_timer_between(ckks_ctx* c, int slot_a, int slot_b, float* ms) {
    if (!c || !ms || slot_a < 0 || slot_b < 0 || (size_t)slot_a >= c->ev_marks.size() || (size_t)slot_b >= c->ev_marks.size() ||
        !c->ev_marks[slot_a] || !c->ev_marks[slot_b]) { ckks::set_error("timer_between: a slot that was never marked"); return CKKS_E_INVALID; }
    CKKS_HIP_TRY(hipEventSynchronize(c->ev_marks[slot_b]));
    CKKS_HIP_TRY(hipEventElapsedTime(ms, c->ev_marks[slot_a], c->ev_marks[slot_b]));
    return CKKS_OK;
}

// Per-kernel timing of one transform: the two passes are separate launches; HIP events are recorded on the
// context's stream before, between and after them.
extern "C" int ckks_ntt_timed(ckks_ctx* c, uint64_t* dev, int sp, int sm, int pn, int mn, int pml, int inverse,
                              float* first_pass_ms, float* second_pass_ms) {
    if (!c || !first_pass_ms || !second_pass_ms) return CKKS_E_INVALID;
    CKKS_HIP_TRY(hipEventRecord(c->ev0, c->stream));
    c->ev_mid_armed = true;
    int rc = ckks::launch_ntt(c, dev, sp, sm, pn, mn, pml, 0, 1, inverse != 0);
    c->ev_mid_armed = false;
    if (rc) return rc;
    CKKS_HIP_TRY(hipEventRecord(c->ev1, c->stream));
    CKKS_HIP_TRY(hipEventSynchronize(c->ev1));
    CKKS_HIP_TRY(hipEventElapsedTime(first_pass_ms, c->ev0, c->ev_mid));
    CKKS_HIP_TRY(hipEventElapsedTime(second_pass_ms, c->ev_mid, c->ev1));
    return CKKS_OK;
}

// ---- NTT entry points ----
extern "C" int ckks_ntt_fwd(ckks_ctx* c, uint64_t* dev, int sp, int sm, int pn, int mn, int pml) {
    return ckks::launch_ntt(c, dev, sp, sm, pn, mn, pml, 0, 1, false);
}
extern "C" int ckks_ntt_inv(ckks_ctx* c, uint64_t* dev, int sp, int sm, int pn, int mn, int pml) {
    return ckks::launch_ntt(c, dev, sp, sm, pn, mn, pml, 0, 1, true);
}
extern "C" int ckks_ntt_noalloc(ckks_ctx* c, uint64_t* dev, int sp, int sm, int pn, int mn, int pml, int inverse) {
    return ckks::launch_ntt_noalloc(c, dev, sp, sm, pn, mn, pml, inverse != 0);
}
extern "C" int ckks_ntt_chain_slot(unsigned slot, unsigned tiles, unsigned skew, unsigned* second, unsigned* k, unsigned* tile) {
    if (!second || !k || !tile || !tiles) return CKKS_E_INVALID;
    ckks::ntt_chain_slot(slot, tiles, skew, second, k, tile);
    return CKKS_OK;
}
extern "C" unsigned ckks_ntt_chain_slots(unsigned kmax, unsigned tiles, unsigned skew) { return ckks::ntt_chain_slots(kmax, tiles, skew); }
extern "C" int ckks_ntt_noalloc_max_limbs(void) { return ckks::ntt_noalloc_max_limbs(); }
extern "C" int ckks_ntt_fwd_ext(ckks_ctx* c, uint64_t* dev, int sp, int sm, int pn, int mn, int pml, int cmn, int bs) {
    return ckks::launch_ntt(c, dev, sp, sm, pn, mn, pml, cmn, bs, false);
}
extern "C" int ckks_ntt_inv_ext(ckks_ctx* c, uint64_t* dev, int sp, int sm, int pn, int mn, int pml, int cmn, int bs) {
    return ckks::launch_ntt(c, dev, sp, sm, pn, mn, pml, cmn, bs, true);
}
