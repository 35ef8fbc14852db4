// CPU oracle for the CKKS hot path.  TEST INFRASTRUCTURE ONLY: see ckks_oracle.h.
// Plain C++17, unsigned __int128 for wide arithmetic, optional OpenMP over limbs / rows.
// Every routine cites the file:line of haozetao/ckks_llm it restates.
#include "ckks_oracle.h"

#include <cmath>
#include <cstring>
#include <set>
#include <string>
#include <vector>
#ifdef _OPENMP
#include <omp.h>
#endif

typedef unsigned __int128 u128;
typedef uint64_t u64;

// ------------------------------------------------------------------------------------------------
// scalar modmath
// ------------------------------------------------------------------------------------------------
// Utils.cuh:33-38
u64 orc_mulmod(u64 a, u64 b, u64 q) { return (u64)(((u128)a * b) % q); }
// Utils.cuh:14-31
u64 orc_powmod(u64 a, u64 e, u64 q) {
    u64 r = 1;
    while (e) {
        if (e & 1) r = orc_mulmod(r, a, q);
        a = orc_mulmod(a, a, q);
        e >>= 1;
    }
    return r;
}
// Utils.cuh:48-53 (Fermat inverse; q prime)
u64 orc_invmod(u64 a, u64 q) { return orc_powmod(a % q, q - 2, q); }
// Utils.cuh:40-45
u64 orc_xshoup(u64 x, u64 q) { return (u64)((((u128)x) << 64) / q); }

// uint128.cuh:143-147
static inline u64 csub_q(u64 a, u64 q) {
    u64 t = a - q;
    return t + (t >> 63) * q;
}
// uint128.cuh:169-179
u64 orc_mulmod_shoup(u64 a, u64 b, u64 b_shoup, u64 q) {
    u64 hi = (u64)(((u128)a * b_shoup) >> 64);
    u64 r = a * b - hi * q;
    return csub_q(r, q);
}
// Context_23.cuh:67-70 : mu = floor(2^128 / q) split in two words (q odd, so floor((2^128-1)/q) is the same number)
void orc_barrett_mu(u64 q, u64* mu_hi, u64* mu_lo) {
    u128 mu = (~(u128)0) / q;
    *mu_hi = (u64)(mu >> 64);
    *mu_lo = (u64)mu;
}
// uint128.cuh:182-212 : the quotient estimate drops the low word of a.lo*mu.lo exactly as the PTX does
u64 orc_barrett128(u64 a_hi, u64 a_lo, u64 q, u64 mu_hi, u64 mu_lo) {
    u64 tmp = (u64)(((u128)a_lo * mu_lo) >> 64);
    u128 s = (u128)a_lo * mu_hi + tmp;       // mad.lo.cc / madc.hi
    u64 tmp2 = (u64)s;
    u64 res = (u64)(s >> 64);
    u128 s2 = (u128)a_hi * mu_lo + tmp2;     // second cross product
    res += (u64)(s2 >> 64);                  // madc.hi with carry-in folded in s2
    res += a_hi * mu_hi;                     // mad.lo
    u64 r = a_lo - res * q;
    return csub_q(r, q);
}
// uint128.cuh:214-225
u64 orc_barrett64(u64 a, u64 q, u64 mu_hi) {
    u64 s = (u64)(((u128)mu_hi * a) >> 64);
    return csub_q(a - s * q, q);
}

// ------------------------------------------------------------------------------------------------
// roots of unity and tables
// ------------------------------------------------------------------------------------------------
// Utils.cuh:63-77.  The loop bound is the reference's: i < sqrt(n) on the shrinking n, strict,
// evaluated in double; a remaining cofactor > 2 is recorded as a "factor" even when it is a square.
static void find_prime_factors(std::set<u64>& s, u64 number) {
    while (number % 2 == 0) { s.insert(2); number /= 2; }
    for (u64 i = 3; (double)i < std::sqrt((double)number); i++) {
        while (number % i == 0) { s.insert(i); number /= i; }
    }
    if (number > 2) s.insert(number);
}
// Utils.cuh:79-96
u64 orc_find_primitive_root(u64 q) {
    std::set<u64> s;
    u64 phi = q - 1;
    find_prime_factors(s, phi);
    for (u64 r = 2; r <= phi; r++) {
        bool bad = false;
        for (u64 f : s) if (orc_powmod(r, phi / f, q) == 1) { bad = true; break; }
        if (!bad) return r;
    }
    return (u64)-1;
}
// Utils.cuh:98-109
u64 orc_find_mth_root(u64 M, u64 q) {
    u64 g = orc_find_primitive_root(q);
    if ((q - 1) % M != 0) return (u64)-1;
    return orc_powmod(g, (q - 1) / M, q);
}
// Utils.cuh:125-132
uint32_t orc_bitrev(uint32_t x, int bits) {
    uint32_t r = 0;
    for (int i = 0; i < bits; i++) { r = (r << 1) | (x & 1); x >>= 1; }
    return r;
}
static int ilog2(u64 n) { int l = 0; while ((1ull << l) < n) l++; return l; }

// Utils.cuh:190-210 : psi[bitrev(i)] = psi^i, psiinv[bitrev(i)] = psi^-i, psiinv[1] *= n^-1, Shoup companions.
void orc_fill_psi_tables(u64 psi, u64 q, uint32_t n, u64* psi_tab, u64* psiinv_tab, u64* psi_shoup, u64* psiinv_shoup) {
    int lg = ilog2(n);
    u64 psiinv = orc_invmod(psi, q);
    u64 ninv = orc_invmod(n, q);
    psi_tab[0] = psiinv_tab[0] = 1;
    for (uint32_t i = 1; i < n; i++) {
        uint32_t prev = orc_bitrev(i - 1, lg), next = orc_bitrev(i, lg);
        psi_tab[next] = orc_mulmod(psi, psi_tab[prev], q);
        psiinv_tab[next] = orc_mulmod(psiinv, psiinv_tab[prev], q);
    }
    psiinv_tab[1] = orc_mulmod(psiinv_tab[1], ninv, q);
    if (psi_shoup) for (uint32_t i = 0; i < n; i++) psi_shoup[i] = orc_xshoup(psi_tab[i], q);
    if (psiinv_shoup) for (uint32_t i = 0; i < n; i++) psiinv_shoup[i] = orc_xshoup(psiinv_tab[i], q);
}

// Forward negacyclic NTT, natural -> bit-reversed order, canonical output.
// Loop shape: python/ntt.ipynb cell 2 (low_NTT); stage/twiddle rule psi[m+i]: ntt_60bit.cuh:320-346, :583-679.
void orc_ntt_limb(u64* a, uint32_t n, u64 q, const u64* psi_tab) {
    uint32_t t = n;
    for (uint32_t m = 1; m < n; m <<= 1) {
        t >>= 1;
        for (uint32_t i = 0; i < m; i++) {
            u64 w = psi_tab[m + i];
            uint32_t j1 = 2 * i * t, j2 = j1 + t;
            for (uint32_t j = j1; j < j2; j++) {
                u64 U = a[j], V = orc_mulmod(a[j + t], w, q);
                u64 s = U + V; if (s >= q) s -= q;
                u64 d = U >= V ? U - V : U + q - V;
                a[j] = s; a[j + t] = d;
            }
        }
    }
}
// Inverse (Gentleman-Sande), bit-reversed -> natural order, scaled by n^-1, canonical output.
// python/ntt.ipynb cell 2 (low_INNT); the reference folds n^-1 into psiinv[1] (Utils.cuh:200) for the (U-V) branch
// of the last stage and multiplies the (U+V) branch by n_inv explicitly (ntt_60bit.cuh:890-893).
void orc_intt_limb(u64* a, uint32_t n, u64 q, const u64* psiinv_tab, u64 n_inv) {
    uint32_t t = 1;
    for (uint32_t m = n; m > 1; m >>= 1) {
        uint32_t h = m >> 1, j1 = 0;
        for (uint32_t i = 0; i < h; i++) {
            u64 w = psiinv_tab[h + i];
            for (uint32_t j = j1; j < j1 + t; j++) {
                u64 U = a[j], V = a[j + t];
                u64 s = U + V; if (s >= q) s -= q;
                u64 d = U >= V ? U - V : U + q - V;
                a[j] = (h == 1) ? orc_mulmod(s, n_inv, q) : s;
                a[j + t] = orc_mulmod(d, w, q);
            }
            j1 += 2 * t;
        }
        t <<= 1;
    }
}

// Same transforms with the Shoup companions (uint128.cuh:169-179) instead of a 128-bit remainder; used by the
// batched entry points so the oracle doubles as a timed CPU baseline.  Checked against the plain loops in tests.
static void ntt_limb_shoup(u64* a, uint32_t n, u64 q, const u64* w, const u64* ws) {
    uint32_t t = n;
    for (uint32_t m = 1; m < n; m <<= 1) {
        t >>= 1;
        for (uint32_t i = 0; i < m; i++) {
            u64 W = w[m + i], Ws = ws[m + i];
            u64* x = a + 2 * (size_t)i * t; u64* y = x + t;
            for (uint32_t j = 0; j < t; j++) {
                u64 U = x[j], V = orc_mulmod_shoup(y[j], W, Ws, q);
                u64 s = U + V; s = s >= q ? s - q : s;
                u64 d = U >= V ? U - V : U + q - V;
                x[j] = s; y[j] = d;
            }
        }
    }
}
static void intt_limb_shoup(u64* a, uint32_t n, u64 q, const u64* w, const u64* ws, u64 n_inv, u64 n_inv_s) {
    uint32_t t = 1;
    for (uint32_t m = n; m > 1; m >>= 1) {
        uint32_t h = m >> 1;
        for (uint32_t i = 0; i < h; i++) {
            u64 W = w[h + i], Ws = ws[h + i];
            u64* x = a + 2 * (size_t)i * t; u64* y = x + t;
            for (uint32_t j = 0; j < t; j++) {
                u64 U = x[j], V = y[j];
                u64 s = U + V; s = s >= q ? s - q : s;
                u64 d = U >= V ? U - V : U + q - V;
                x[j] = (h == 1) ? orc_mulmod_shoup(s, n_inv, n_inv_s, q) : s;
                y[j] = orc_mulmod_shoup(d, W, Ws, q);
            }
        }
        t <<= 1;
    }
}
// Utils.cuh:255-285
void orc_negacyclic_mul(const u64* a, const u64* b, u64* c, uint32_t n, u64 q) {
    std::vector<u64> w(2 * (size_t)n, 0);
    for (uint32_t i = 0; i < n; i++)
        for (uint32_t j = 0; j < n; j++)
            w[i + j] = (u64)(((u128)a[i] * b[j] + w[i + j]) % q);
    for (uint32_t i = 0; i < n; i++) {
        u64 lo = w[i], hi = w[i + n];
        if (lo < hi) lo += q;
        c[i] = (lo - hi) % q;
    }
}

// ------------------------------------------------------------------------------------------------
// context
// ------------------------------------------------------------------------------------------------
struct orc_ctx {
    int logN = 0, p_num = 0, q_num = 0, t_num = 0, gamma = 0, L = 0, K = 0, dnum = 0;
    int Ri_blockNum = 0, Qj_blockNum = 0;
    long N = 0;
    std::vector<u64> pqt, mu_hi, mu_lo, psi, psiinv_root, n_inv, n_inv_shoup, halfTmodpqti;
    std::vector<u64> psi_table, psiinv_table, psi_shoup_table, psiinv_shoup_table;   // [prime][N]
    // P -> q  (ModDown)
    std::vector<u64> pHatVecModq;                          // [l<=L][K]
    std::vector<u64> pHatInvVecModp, pHatInvVecModp_shoup; // [K]
    std::vector<u64> PModqt, PModqt_shoup, PinvModq, PinvModq_shoup;
    // Ri -> T
    std::vector<u64> RiHatInv, RiHatInv_shoup;             // [Ri_blockNum][gamma]
    std::vector<u64> RiHatModT;                            // [Ri_blockNum][t_num][gamma]
    std::vector<u64> Rimodti;                              // [t_num][Ri_blockNum]
    // Qj -> T
    std::vector<u64> QjHatInv, QjHatInv_shoup;             // [L+1][Qj_blockNum][p_num]
    std::vector<u64> QjHatModT;                            // [L+1][Qj_blockNum][t_num][p_num]
    std::vector<u64> Qjmodti;                              // [L+1][Qj_blockNum][t_num]
    // T -> PQ
    std::vector<u64> THatInv, THatInv_shoup;               // [t_num]
    std::vector<u64> THatModRi;                            // [K+L+1][t_num]
    std::vector<u64> Tmodpqi;                              // [K+L+1]
    // rescale
    std::vector<u64> qiInvModql, qiInvModql_shoup;         // triangular, row l-1 at offset l(l-1)/2
    // generic exact-conversion tables for the textbook hybrid switch: per level, per digit
    const u64* psi_tab(int prime) const { return &psi_table[(size_t)prime * N]; }
    const u64* psiinv_tab(int prime) const { return &psiinv_table[(size_t)prime * N]; }
};

static int ceil_div(int a, int b) { return (a + b - 1) / b; }

// big-integer-free helpers: product of a list of primes modulo m
static u64 prod_mod(const std::vector<u64>& v, int lo, int hi, int skip, u64 m) {
    u64 r = 1;
    for (int i = lo; i < hi; i++) { if (i == skip) continue; r = orc_mulmod(r, v[i] % m, m); }
    return r;
}

// floor(T/2) mod m for T = prod t_i, without big integers: T is odd, so floor(T/2) = (T-1)/2 and
// (T-1)/2 mod m = ((T mod 2m) - 1)/2 mod m  (Context_23.cuh:96-130 computes it with NTL::ZZ).
static u64 half_prod_mod(const std::vector<u64>& t, u64 m) {
    const u64 m2 = 2 * m;                      // m < 2^62 for every modulus this code handles
    u64 r = 1;
    for (u64 x : t) r = (u64)(((u128)r * (x % m2)) % m2);
    return ((r - 1) / 2) % m;                  // r = T mod 2m is odd
}

orc_ctx* orc_ctx_create(int logN, const u64* p, int p_num, const u64* q, int q_num, const u64* t, int t_num, int gamma) {
    orc_ctx* c = new orc_ctx();
    c->logN = logN; c->N = 1L << logN;
    c->p_num = p_num; c->q_num = q_num; c->t_num = t_num; c->gamma = gamma;
    c->L = q_num - 1; c->K = p_num;
    c->dnum = p_num ? q_num / p_num : 0;                                      // Context_23.cuh:29
    c->Ri_blockNum = gamma ? ceil_div(p_num + q_num, gamma) : 0;              // :32
    c->Qj_blockNum = p_num ? ceil_div(q_num, p_num) : 0;                      // :33
    const long N = c->N; const int K = p_num, L = c->L;
    for (int i = 0; i < p_num; i++) c->pqt.push_back(p[i]);
    for (int i = 0; i < q_num; i++) c->pqt.push_back(q[i]);
    for (int i = 0; i < t_num; i++) c->pqt.push_back(t[i]);
    const int tot = (int)c->pqt.size();
    std::vector<u64> pV(p, p + p_num), qV(q, q + q_num), tV(t, t + t_num);
    c->mu_hi.resize(tot); c->mu_lo.resize(tot); c->psi.resize(tot); c->psiinv_root.resize(tot);
    c->n_inv.resize(tot); c->n_inv_shoup.resize(tot);
    for (int i = 0; i < tot; i++) {
        u64 m = c->pqt[i];
        orc_barrett_mu(m, &c->mu_hi[i], &c->mu_lo[i]);
        c->psi[i] = orc_find_mth_root(2 * (u64)N, m);                         // Context_23.cuh:75,91,108
        c->psiinv_root[i] = orc_invmod(c->psi[i], m);                         // :134-141
        c->n_inv[i] = orc_invmod((u64)N, m);                                  // :144-151
        c->n_inv_shoup[i] = orc_xshoup(c->n_inv[i], m);                       // :153-160
        c->halfTmodpqti.push_back(t_num ? half_prod_mod(tV, m) : 0);          // :126-130
    }
    c->psi_table.resize((size_t)tot * N); c->psiinv_table.resize((size_t)tot * N);
    c->psi_shoup_table.resize((size_t)tot * N); c->psiinv_shoup_table.resize((size_t)tot * N);
#pragma omp parallel for schedule(dynamic)
    for (int i = 0; i < tot; i++)                                             // Context_23.cuh:481-495
        orc_fill_psi_tables(c->psi[i], c->pqt[i], (uint32_t)N, &c->psi_table[(size_t)i * N], &c->psiinv_table[(size_t)i * N],
                            &c->psi_shoup_table[(size_t)i * N], &c->psiinv_shoup_table[(size_t)i * N]);

    // ---- P x Q_l -> Q_l : Context_23.cuh:162-190 ----
    for (int l = 0; l <= L; l++)
        for (int i = 0; i < K; i++) c->pHatVecModq.push_back(prod_mod(pV, 0, K, i, qV[l]));
    for (int i = 0; i < K; i++) {
        u64 v = orc_invmod(prod_mod(pV, 0, K, i, pV[i]), pV[i]);
        c->pHatInvVecModp.push_back(v); c->pHatInvVecModp_shoup.push_back(orc_xshoup(v, pV[i]));
    }
    // ---- Ri -> T : Context_23.cuh:232-283 ----
    const int PQ = p_num + q_num;
    if (gamma > 0 && t_num > 0) {
        c->RiHatInv.assign((size_t)c->Ri_blockNum * gamma, 0); c->RiHatInv_shoup.assign((size_t)c->Ri_blockNum * gamma, 0);
        c->RiHatModT.assign((size_t)c->Ri_blockNum * t_num * gamma, 0);
        c->Rimodti.assign((size_t)t_num * c->Ri_blockNum, 0);
        for (int i = 0; i < c->Ri_blockNum; i++) {
            int lo = i * gamma, hi = std::min(lo + gamma, PQ);
            for (int j = lo; j < hi; j++) {
                u64 v = orc_invmod(prod_mod(c->pqt, lo, hi, j, c->pqt[j]), c->pqt[j]);
                c->RiHatInv[(size_t)i * gamma + (j - lo)] = v;
                c->RiHatInv_shoup[(size_t)i * gamma + (j - lo)] = orc_xshoup(v, c->pqt[j]);
            }
            for (int k = 0; k < t_num; k++) {
                for (int j = lo; j < hi; j++)
                    c->RiHatModT[(size_t)i * t_num * gamma + (size_t)k * gamma + (j - lo)] = prod_mod(c->pqt, lo, hi, j, tV[k]);
                c->Rimodti[(size_t)k * c->Ri_blockNum + i] = prod_mod(c->pqt, lo, hi, -1, tV[k]);
            }
        }
    }
    // ---- Qj -> T : Context_23.cuh:286-351 ----
    if (p_num > 0 && t_num > 0) {
        const int B = c->Qj_blockNum;
        c->QjHatInv.assign((size_t)(L + 1) * B * p_num, 0); c->QjHatInv_shoup.assign((size_t)(L + 1) * B * p_num, 0);
        c->QjHatModT.assign((size_t)(L + 1) * B * t_num * p_num, 0);
        c->Qjmodti.assign((size_t)(L + 1) * B * t_num, 0);
        for (int l = 0; l <= L; l++) {
            int nb = ceil_div(l + 1, p_num);
            for (int i = 0; i < nb; i++) {
                int lo = i * p_num, hi = std::min(lo + p_num, l + 1);
                for (int j = lo; j < hi; j++) {
                    u64 v = orc_invmod(prod_mod(qV, lo, hi, j, qV[j]), qV[j]);
                    size_t o = (size_t)l * B * p_num + (size_t)i * p_num + (j - lo);
                    c->QjHatInv[o] = v; c->QjHatInv_shoup[o] = orc_xshoup(v, qV[j]);
                }
                for (int k = 0; k < t_num; k++) {
                    for (int j = lo; j < hi; j++)
                        c->QjHatModT[(size_t)l * B * t_num * p_num + (size_t)i * t_num * p_num + (size_t)k * p_num + (j - lo)] =
                            prod_mod(qV, lo, hi, j, tV[k]);
                    c->Qjmodti[(size_t)l * B * t_num + (size_t)i * t_num + k] = prod_mod(qV, lo, hi, -1, tV[k]);
                }
            }
        }
    }
    // ---- T -> PQ : Context_23.cuh:354-393 ----
    for (int i = 0; i < t_num; i++) {
        u64 v = orc_invmod(prod_mod(tV, 0, t_num, i, tV[i]), tV[i]);
        c->THatInv.push_back(v); c->THatInv_shoup.push_back(orc_xshoup(v, tV[i]));
    }
    for (int i = 0; i < PQ; i++) {
        for (int j = 0; j < t_num; j++) c->THatModRi.push_back(prod_mod(tV, 0, t_num, j, c->pqt[i]));
        c->Tmodpqi.push_back(prod_mod(tV, 0, t_num, -1, c->pqt[i]));
    }
    // ---- P mod q,t ; P^-1 mod q : Context_23.cuh:397-421 ----
    for (int i = 0; i <= L; i++) {
        u64 v = prod_mod(pV, 0, K, -1, qV[i]);
        c->PModqt.push_back(v); c->PModqt_shoup.push_back(orc_xshoup(v, qV[i]));
        u64 w = orc_invmod(v, qV[i]);
        c->PinvModq.push_back(w); c->PinvModq_shoup.push_back(orc_xshoup(w, qV[i]));
    }
    for (int i = 0; i < t_num; i++) {
        u64 v = prod_mod(pV, 0, K, -1, tV[i]);
        c->PModqt.push_back(v); c->PModqt_shoup.push_back(orc_xshoup(v, tV[i]));
    }
    // ---- rescale : Context_23.cuh:425-436, device layout :557-563 (row l-1 at offset l(l-1)/2) ----
    for (int l = 1; l <= L; l++)
        for (int j = 0; j < l; j++) {
            u64 v = orc_invmod(qV[l], qV[j]);
            c->qiInvModql.push_back(v); c->qiInvModql_shoup.push_back(orc_xshoup(v, qV[j]));
        }
    return c;
}
void orc_ctx_destroy(orc_ctx* c) { delete c; }

int orc_ctx_info(const orc_ctx* c, const char* name) {
    std::string n(name);
    if (n == "logN") return c->logN;
    if (n == "p_num") return c->p_num;
    if (n == "q_num") return c->q_num;
    if (n == "t_num") return c->t_num;
    if (n == "gamma") return c->gamma;
    if (n == "dnum") return c->dnum;
    if (n == "Ri_blockNum") return c->Ri_blockNum;
    if (n == "Qj_blockNum") return c->Qj_blockNum;
    return -1;
}
long orc_ctx_get(const orc_ctx* c, const char* name, u64* out, long cap) {
    std::string n(name);
    const std::vector<u64>* v = nullptr;
    if (n == "pqt") v = &c->pqt; else if (n == "mu_hi") v = &c->mu_hi; else if (n == "mu_lo") v = &c->mu_lo;
    else if (n == "psi") v = &c->psi; else if (n == "psiinv") v = &c->psiinv_root;
    else if (n == "n_inv") v = &c->n_inv; else if (n == "n_inv_shoup") v = &c->n_inv_shoup;
    else if (n == "halfTmodpqti") v = &c->halfTmodpqti;
    else if (n == "psi_table") v = &c->psi_table; else if (n == "psiinv_table") v = &c->psiinv_table;
    else if (n == "psi_shoup_table") v = &c->psi_shoup_table; else if (n == "psiinv_shoup_table") v = &c->psiinv_shoup_table;
    else if (n == "pHatVecModq") v = &c->pHatVecModq; else if (n == "pHatInvVecModp") v = &c->pHatInvVecModp;
    else if (n == "PModqt") v = &c->PModqt; else if (n == "PinvModq") v = &c->PinvModq;
    else if (n == "RiHatInv") v = &c->RiHatInv; else if (n == "RiHatModT") v = &c->RiHatModT; else if (n == "Rimodti") v = &c->Rimodti;
    else if (n == "QjHatInv") v = &c->QjHatInv; else if (n == "QjHatModT") v = &c->QjHatModT; else if (n == "Qjmodti") v = &c->Qjmodti;
    else if (n == "THatInv") v = &c->THatInv; else if (n == "THatModRi") v = &c->THatModRi; else if (n == "Tmodpqi") v = &c->Tmodpqi;
    else if (n == "qiInvModql") v = &c->qiInvModql;
    if (!v) return -1;
    long cnt = (long)v->size();
    if (out) { if (cap < cnt) return -1; std::memcpy(out, v->data(), cnt * sizeof(u64)); }
    return cnt;
}

// ------------------------------------------------------------------------------------------------
// batched NTT with the reference's addressing (Context_23.cuh:847-930; ntt_60bit.cuh:446-455, :913-934)
// ------------------------------------------------------------------------------------------------
static int ntt_batch(const orc_ctx* c, u64* a, int start_poly_idx, int start_mod_idx, int poly_num, int mod_num,
                     int poly_mod_len, long batch_stride_limbs, int batch, bool inverse) {
    const long N = c->N;
    if (start_mod_idx < 0 || start_mod_idx + mod_num > (int)c->pqt.size()) return -1;
    const long total = (long)batch * poly_num * mod_num;
#pragma omp parallel for schedule(static)
    for (long w = 0; w < total; w++) {
        int j = (int)(w % mod_num); long r = w / mod_num;
        int y = (int)(r % poly_num); int z = (int)(r / poly_num);
        u64* limb = a + ((long)z * batch_stride_limbs + (long)y * poly_mod_len + start_poly_idx + j) * N;
        int prime = start_mod_idx + j;
        if (inverse) intt_limb_shoup(limb, (uint32_t)N, c->pqt[prime], c->psiinv_tab(prime), &c->psiinv_shoup_table[(size_t)prime * N],
                                     c->n_inv[prime], c->n_inv_shoup[prime]);
        else ntt_limb_shoup(limb, (uint32_t)N, c->pqt[prime], c->psi_tab(prime), &c->psi_shoup_table[(size_t)prime * N]);
    }
    return 0;
}
int orc_ntt_fwd(const orc_ctx* c, u64* a, int sp, int sm, int pn, int mn, int pml) { return ntt_batch(c, a, sp, sm, pn, mn, pml, 0, 1, false); }
int orc_ntt_inv(const orc_ctx* c, u64* a, int sp, int sm, int pn, int mn, int pml) { return ntt_batch(c, a, sp, sm, pn, mn, pml, 0, 1, true); }
int orc_ntt_fwd_ext(const orc_ctx* c, u64* a, int sp, int sm, int pn, int mn, int pml, int cmn, int bs) { return ntt_batch(c, a, sp, sm, pn, mn, pml, cmn, bs, false); }
int orc_ntt_inv_ext(const orc_ctx* c, u64* a, int sp, int sm, int pn, int mn, int pml, int cmn, int bs) { return ntt_batch(c, a, sp, sm, pn, mn, pml, cmn, bs, true); }

// ------------------------------------------------------------------------------------------------
// basis conversion
// ------------------------------------------------------------------------------------------------
static inline u128 sub128_64(u128 a, u64 b) { return a - (u128)b; }          // uint128.cuh:273-283 (wraps mod 2^128)
static inline u64 barrett_idx(const orc_ctx* c, u128 acc, int prime) {
    return orc_barrett128((u64)(acc >> 64), (u64)acc, c->pqt[prime], c->mu_hi[prime], c->mu_lo[prime]);
}

// BasisConv.cuh:7-79
int orc_modup_pq_to_t(const orc_ctx* c, u64* out, const u64* in, int l, int batch) {
    const long N = c->N; const int g = c->gamma, P = c->p_num, Q = c->q_num, T = c->t_num;
    if (g <= 0 || T <= 0 || l < 0 || l > c->L) return -1;
    const int blockNum = ceil_div(P + l + 1, g);
    for (int b = 0; b < batch; b++)
#pragma omp parallel for collapse(2) schedule(static)
        for (int blk = 0; blk < blockNum; blk++)
            for (long x = 0; x < N; x++) {
                u64 rb[64]; double vv = 0; int cnt = 0;
                for (int i = 0; i < g && i + blk * g < P + l + 1; i++, cnt++) {
                    int pi = i + blk * g; u64 ri = c->pqt[pi];
                    u64 ra = in[((long)pi + (long)b * (P + Q)) * N + x];
                    rb[i] = orc_mulmod_shoup(ra, c->RiHatInv[(size_t)blk * g + i], c->RiHatInv_shoup[(size_t)blk * g + i], ri);
                    vv += (double)rb[i] / (double)ri;                          // :33
                }
                int vf = (int)vv;                                              // :36
                for (int k = 0; k < T; k++) {
                    u128 acc = 0;
                    for (int j = 0; j < cnt; j++) acc += (u128)rb[j] * c->RiHatModT[(size_t)blk * T * g + (size_t)k * g + j];
                    acc = sub128_64(acc, (u64)vf * c->Rimodti[(size_t)k * c->Ri_blockNum + blk]);   // :54
                    long oidx = (long)b * c->Ri_blockNum * T + (long)blk * T + k;                    // :52
                    out[oidx * N + x] = barrett_idx(c, acc, P + Q + k);
                }
            }
    return 0;
}

// BasisConv.cuh:84-179.  The reference indexes Qjmodti with the batch index folded in (:142,:153), which for
// batch > 0 walks into the next level's table; every caller uses the table of level l, and so does this restatement.
int orc_modup_qj_to_t(const orc_ctx* c, u64* out, const u64* in, int l, int batch) {
    const long N = c->N; const int P = c->p_num, Q = c->q_num, T = c->t_num, B = c->Qj_blockNum;
    if (P <= 0 || T <= 0 || l < 0 || l > c->L) return -1;
    const int blockNum = ceil_div(l + 1, P);
    const u64* hatinv = &c->QjHatInv[(size_t)l * B * P]; const u64* hatinv_s = &c->QjHatInv_shoup[(size_t)l * B * P];
    const u64* hatT = &c->QjHatModT[(size_t)l * B * T * P]; const u64* qjmodt = &c->Qjmodti[(size_t)l * B * T];
    for (int b = 0; b < batch; b++)
#pragma omp parallel for collapse(2) schedule(static)
        for (int blk = 0; blk < blockNum; blk++)
            for (long x = 0; x < N; x++) {
                u64 rb[64]; double vv = 0; int cnt = 0;
                for (int j = 0; j < P && j + blk * P < l + 1; j++, cnt++) {
                    int iq = j + blk * P; u64 qi = c->pqt[P + iq];
                    u64 ra = in[(long)b * Q * N + (long)iq * N + x];
                    rb[j] = orc_mulmod_shoup(ra, hatinv[iq], hatinv_s[iq], qi);
                    vv += (double)rb[j] / (double)qi;                          // :113-114
                }
                int vf = (int)vv;                                              // :152
                for (int k = 0; k < T; k++) {
                    u128 acc = 0;
                    for (int j = 0; j < cnt; j++) acc += (u128)rb[j] * hatT[(size_t)blk * T * P + (size_t)k * P + j];
                    acc = sub128_64(acc, (u64)vf * qjmodt[(size_t)blk * T + k]);
                    long oidx = (long)b * B * T + (long)blk * T + k;
                    out[oidx * N + x] = barrett_idx(c, acc, P + Q + k);
                }
            }
    return 0;
}

// BasisConv.cuh:183-254
int orc_modup_t_to_pql(const orc_ctx* c, u64* buf, const u64* in, int l, int batch) {
    const long N = c->N; const int g = c->gamma, P = c->p_num, Q = c->q_num, T = c->t_num, RB = c->Ri_blockNum;
    if (g <= 0 || T <= 0 || l < 0 || l > c->L) return -1;
    const int blockNum = ceil_div(P + l + 1, g);
    for (int b = 0; b < batch; b++)
#pragma omp parallel for collapse(2) schedule(static)
        for (int blk = 0; blk < blockNum; blk++)
            for (long x = 0; x < N; x++) {
                u64 rb[64]; double vv = 0;
                for (int i = 0; i < T; i++) {
                    u64 t = c->pqt[P + Q + i];
                    u64 ra = in[(long)b * RB * T * N + ((long)blk * T + i) * N + x];
                    ra = ra + c->halfTmodpqti[P + Q + i];                      // :203
                    rb[i] = orc_mulmod_shoup(ra, c->THatInv[i], c->THatInv_shoup[i], t);
                    vv += (double)rb[i] / (double)t;                           // :209-210
                }
                int vf = (int)vv;
                for (int j = 0; j < g && j + blk * g < P + l + 1; j++) {
                    int ipq = j + blk * g; u64 ri = c->pqt[ipq];
                    u128 acc = 0;
                    for (int i = 0; i < T; i++) acc += (u128)rb[i] * c->THatModRi[(size_t)ipq * T + i];
                    acc = sub128_64(acc, (u64)vf * c->Tmodpqi[ipq]);           // :232
                    u64 r = barrett_idx(c, acc, ipq);
                    r = r + ri - c->halfTmodpqti[ipq];                         // :236
                    r = csub_q(r, ri);
                    buf[(long)b * RB * T * N + (long)ipq * N + x] = r;         // :239
                }
            }
    return 0;
}

// BasisConv.cuh:257-347
int orc_moddown_pql_to_ql(const orc_ctx* c, u64* out, const u64* buf, int l, int batch) {
    const long N = c->N; const int P = c->p_num, Q = c->q_num, T = c->t_num, RB = c->Ri_blockNum;
    if (P <= 0 || l < 0 || l > c->L) return -1;
    const long in_stride = (long)RB * T * N;
    for (int b = 0; b < batch; b++)
#pragma omp parallel for collapse(2) schedule(static)
        for (int iq = 0; iq <= l; iq++)
            for (long x = 0; x < N; x++) {
                u64 qi = c->pqt[P + iq];
                u64 r;
                if (P == 1) {                                                  // :261-283
                    r = buf[b * in_stride + x] % qi;
                } else {                                                       // :286-326
                    u128 acc = 0;
                    for (int i = 0; i < P; i++) {
                        u64 ra = buf[b * in_stride + (long)i * N + x];
                        u64 rb = orc_mulmod_shoup(ra, c->pHatInvVecModp[i], c->pHatInvVecModp_shoup[i], c->pqt[i]);
                        acc += (u128)rb * c->pHatVecModq[(size_t)iq * P + i];
                    }
                    r = barrett_idx(c, acc, P + iq);
                }
                u64 v = qi - r + buf[b * in_stride + (long)(P + iq) * N + x];
                out[(long)b * Q * N + (long)iq * N + x] = orc_mulmod_shoup(v, c->PinvModq[iq], c->PinvModq_shoup[iq], qi);
            }
    return 0;
}

// ExternalProduct.cuh:7-97
int orc_external_product_t(const orc_ctx* c, u64* out, const u64* cT, const u64* swk, int l) {
    const long N = c->N; const int g = c->gamma, P = c->p_num, Q = c->q_num, T = c->t_num, RB = c->Ri_blockNum, dnum = c->dnum;
    if (g <= 0 || T <= 0 || P <= 0 || l < 0 || l > c->L) return -1;
    const int cipher_blockNum = ceil_div(l + 1, P), blockNum = ceil_div(P + l + 1, g);
    if (cipher_blockNum > dnum) return -1;               // q_num is no multiple of p_num: the key holds q_num / p_num digits only
#pragma omp parallel for collapse(2) schedule(static)
    for (int blk = 0; blk < blockNum; blk++)
        for (int k = 0; k < T; k++)
            for (long x = 0; x < N; x++) {
                u128 acc1 = 0, acc2 = 0;
                for (int i = 0; i < cipher_blockNum; i++) {
                    u64 ra = cT[((long)i * T + k) * N + x];
                    long kidx = ((long)i * T * RB + (long)blk * T + k) * N + x;
                    acc1 += (u128)ra * swk[kidx];
                    acc2 += (u128)ra * swk[(long)RB * T * dnum * N + kidx];
                }
                long oidx = x + (long)blk * T * N + (long)k * N;
                out[oidx] = barrett_idx(c, acc1, P + Q + k);
                out[(long)RB * T * N + oidx] = barrett_idx(c, acc2, P + Q + k);
            }
    return 0;
}

// ExternalProduct.cuh:103-162: one key, batch_size digit sets; set `iter` of cT starts t_num * Qj_blockNum limbs behind the one
// before (:126), its pair goes to polynomials 2 iter and 2 iter + 1 of out (:134, :155).  The reference holds eight accumulators.
int orc_external_product_t_swk_reuse(const orc_ctx* c, u64* out, const u64* cT, const u64* swk, int l, int batch_size) {
    const long N = c->N; const int g = c->gamma, P = c->p_num, Q = c->q_num, T = c->t_num, RB = c->Ri_blockNum, QB = c->Qj_blockNum, dnum = c->dnum;
    if (g <= 0 || T <= 0 || P <= 0 || l < 0 || l > c->L || batch_size < 1 || batch_size > 8) return -1;
    const int cipher_blockNum = ceil_div(l + 1, P), blockNum = ceil_div(P + l + 1, g);
    if (cipher_blockNum > dnum) return -1;
#pragma omp parallel for collapse(2) schedule(static)
    for (int blk = 0; blk < blockNum; blk++)
        for (int k = 0; k < T; k++)
            for (long x = 0; x < N; x++) {
                const long oidx = x + (long)blk * T * N + (long)k * N;
                for (int half = 0; half < 2; half++)
                    for (int iter = 0; iter < batch_size; iter++) {
                        u128 acc = 0;
                        for (int i = 0; i < cipher_blockNum; i++) {
                            const u64 ra = cT[((long)i * T + k) * N + x + (long)iter * T * QB * N];
                            const u64 rb = swk[(long)half * RB * T * dnum * N + ((long)i * T * RB + (long)blk * T + k) * N + x];
                            acc += (u128)ra * rb;
                        }
                        out[(long)RB * T * N * (iter * 2 + half) + oidx] = barrett_idx(c, acc, P + Q + k);
                    }
            }
    return 0;
}

// Scheme_23.cuh:321-385
int orc_rescale(const orc_ctx* c, u64* cipher, int l) {
    const long N = c->N; const int K = c->K, L = c->L;
    if (l < 1 || l > L) return -1;
    orc_ntt_inv(c, cipher, l, K + l, 2, 1, L + 1);                              // :372
    std::vector<u64> rb((size_t)2 * (L + 1) * N, 0);
    for (int z = 0; z < 2; z++)
        for (int i = 0; i < l; i++) {
            u64 q = c->pqt[K + i], mu_hi = c->mu_hi[K + i];
            for (long x = 0; x < N; x++)                                       // mod_to_qi :356-367
                rb[((size_t)z * (L + 1) + i) * N + x] = orc_barrett64(cipher[((size_t)z * (L + 1) + l) * N + x], q, mu_hi);
        }
    orc_ntt_fwd(c, rb.data(), 0, K, 2, l, L + 1);                               // :376
    const u64* inv = &c->qiInvModql[(size_t)l * (l - 1) / 2]; const u64* inv_s = &c->qiInvModql_shoup[(size_t)l * (l - 1) / 2];
    for (int z = 0; z < 2; z++)
        for (int i = 0; i < l; i++) {
            u64 q = c->pqt[K + i];
            for (long x = 0; x < N; x++) {                                     // :339-354
                size_t idx = ((size_t)z * (L + 1) + i) * N + x;
                u64 ra = cipher[idx] + 2 * q - rb[idx];
                ra = csub_q(ra, q);
                cipher[idx] = orc_mulmod_shoup(ra, inv[i], inv_s[i], q);
            }
        }
    return 0;
}

// KeySwitch_23.cuh:219-231
int orc_keyswitch_23(const orc_ctx* c, u64* out, const u64* d2, const u64* swk, int l) {
    const long N = c->N; const int K = c->K, L = c->L, T = c->t_num, RB = c->Ri_blockNum, g = c->gamma;
    if (g <= 0 || T <= 0 || K <= 0 || l < 0 || l > L) return -1;
    const int swk_blockNum = ceil_div(K + l + 1, g), cipher_blockNum = ceil_div(l + 1, K);
    std::vector<u64> axax(d2, d2 + (size_t)(L + 1) * N);
    std::vector<u64> up((size_t)N * T * c->Qj_blockNum, 0), ext((size_t)N * T * RB * 2, 0), buf((size_t)N * T * RB * 2, 0);
    orc_ntt_inv(c, axax.data(), 0, K, 1, l + 1, L + 1);                         // :219
    orc_modup_qj_to_t(c, up.data(), axax.data(), l, 1);                        // :221
    orc_ntt_fwd(c, up.data(), 0, K + L + 1, cipher_blockNum, T, T);             // :223
    orc_external_product_t(c, ext.data(), up.data(), swk, l);                  // :225
    orc_ntt_inv_ext(c, ext.data(), 0, K + L + 1, swk_blockNum, T, T, RB * T, 2);// :226
    orc_modup_t_to_pql(c, buf.data(), ext.data(), l, 2);                       // :228
    orc_moddown_pql_to_ql(c, out, buf.data(), l, 2);                           // :229
    orc_ntt_fwd(c, out, 0, K, 2, l + 1, L + 1);                                 // :231
    return 0;
}

// ------------------------------------------------------------------------------------------------
// textbook hybrid key switch over [P | Q_l], alpha = p_num primes per digit.
// The reference has no such routine (its switch goes through the auxiliary basis T); this one applies the
// reference's exact-conversion recipe (BasisConv.cuh:18-58: y_j = x_j * (D^_j)^-1 mod d_j,
// v = trunc(sum (double)y_j/(double)d_j), out = sum y_j * (D^_j mod r) - v * (D mod r)) to a digit D of
// alpha consecutive Q primes and every other prime r of [P | Q_l], and its ModDown (BasisConv.cuh:286-326).
// ------------------------------------------------------------------------------------------------
int orc_hybrid_modup(const orc_ctx* c, u64* digits_out, const u64* in, int l) {
    const long N = c->N; const int P = c->p_num, Q = c->q_num;
    if (P <= 0 || l < 0 || l > c->L) return -1;
    const int dn = ceil_div(l + 1, P), W = P + Q;
    for (int d = 0; d < dn; d++) {
        int lo = d * P, hi = std::min(lo + P, l + 1), cnt = hi - lo;
        std::vector<u64> hatinv(cnt), hatinv_s(cnt);
        for (int j = lo; j < hi; j++) {
            u64 qj = c->pqt[P + j];
            hatinv[j - lo] = orc_invmod(prod_mod(c->pqt, P + lo, P + hi, P + j, qj), qj);
            hatinv_s[j - lo] = orc_xshoup(hatinv[j - lo], qj);
        }
        std::vector<int> targets;
        for (int r = 0; r < P + l + 1; r++) if (r < P + lo || r >= P + hi) targets.push_back(r);
        std::vector<u64> hat((size_t)targets.size() * cnt), Dmod(targets.size());
        for (size_t ti = 0; ti < targets.size(); ti++) {
            u64 r = c->pqt[targets[ti]];
            for (int j = lo; j < hi; j++) hat[ti * cnt + (j - lo)] = prod_mod(c->pqt, P + lo, P + hi, P + j, r);
            Dmod[ti] = prod_mod(c->pqt, P + lo, P + hi, -1, r);
        }
        u64* o = digits_out + (long)d * W * N;
#pragma omp parallel for schedule(static)
        for (long x = 0; x < N; x++) {
            u64 y[64]; double vv = 0;
            for (int j = lo; j < hi; j++) {
                u64 qj = c->pqt[P + j], xin = in[(long)j * N + x];
                o[(long)(P + j) * N + x] = xin;
                y[j - lo] = orc_mulmod_shoup(xin, hatinv[j - lo], hatinv_s[j - lo], qj);
                vv += (double)y[j - lo] / (double)qj;
            }
            int vf = (int)vv;
            for (size_t ti = 0; ti < targets.size(); ti++) {
                u128 acc = 0;
                for (int j = 0; j < cnt; j++) acc += (u128)y[j] * hat[ti * cnt + j];
                acc = sub128_64(acc, (u64)vf * Dmod[ti]);
                o[(long)targets[ti] * N + x] = barrett_idx(c, acc, targets[ti]);
            }
        }
    }
    return 0;
}
// evk: [2 (a,b)][dnum][P+Q] limbs (NTT domain); digits: [dn][P+Q] limbs (NTT domain); out: [2][P+Q] limbs.
int orc_hybrid_inner_product(const orc_ctx* c, u64* out, const u64* digits, const u64* evk, int l) {
    const long N = c->N; const int P = c->p_num, Q = c->q_num, W = P + Q;
    if (P <= 0 || l < 0 || l > c->L) return -1;
    const int dn = ceil_div(l + 1, P), dnum = ceil_div(Q, P);
#pragma omp parallel for collapse(2) schedule(static)
    for (int z = 0; z < 2; z++)
        for (int r = 0; r < P + l + 1; r++)
            for (long x = 0; x < N; x++) {
                u128 acc = 0;
                for (int d = 0; d < dn; d++)
                    acc += (u128)digits[((long)d * W + r) * N + x] * evk[(((long)z * dnum + d) * W + r) * N + x];
                out[((long)z * W + r) * N + x] = barrett_idx(c, acc, r);
            }
    return 0;
}
// in: [2][P+Q] limbs (coefficient domain) -> out: [2][Q] limbs; arithmetic of BasisConv.cuh:286-326.
int orc_hybrid_moddown(const orc_ctx* c, u64* out, const u64* in, int l) {
    const long N = c->N; const int P = c->p_num, Q = c->q_num, W = P + Q;
    if (P <= 0 || l < 0 || l > c->L) return -1;
#pragma omp parallel for collapse(2) schedule(static)
    for (int z = 0; z < 2; z++)
        for (int iq = 0; iq <= l; iq++) {
            u64 qi = c->pqt[P + iq];
            for (long x = 0; x < N; x++) {
                u128 acc = 0;
                for (int i = 0; i < P; i++) {
                    u64 rb = orc_mulmod_shoup(in[((long)z * W + i) * N + x], c->pHatInvVecModp[i], c->pHatInvVecModp_shoup[i], c->pqt[i]);
                    acc += (u128)rb * c->pHatVecModq[(size_t)iq * P + i];
                }
                u64 r = barrett_idx(c, acc, P + iq);
                u64 v = qi - r + in[((long)z * W + P + iq) * N + x];
                out[((long)z * Q + iq) * N + x] = orc_mulmod_shoup(v, c->PinvModq[iq], c->PinvModq_shoup[iq], qi);
            }
        }
    return 0;
}
// in_ntt: Q limbs (NTT domain); out: [2][Q] limbs (NTT domain).
int orc_hybrid_keyswitch(const orc_ctx* c, u64* out, const u64* in_ntt, const u64* evk, int l) {
    const long N = c->N; const int P = c->p_num, Q = c->q_num, W = P + Q;
    if (P <= 0 || l < 0 || l > c->L) return -1;
    const int dn = ceil_div(l + 1, P);
    std::vector<u64> in(in_ntt, in_ntt + (size_t)Q * N), dig((size_t)dn * W * N, 0), ip((size_t)2 * W * N, 0);
    orc_ntt_inv(c, in.data(), 0, P, 1, l + 1, Q);
    orc_hybrid_modup(c, dig.data(), in.data(), l);
    orc_ntt_fwd(c, dig.data(), 0, 0, dn, P + l + 1, W);
    orc_hybrid_inner_product(c, ip.data(), dig.data(), evk, l);
    orc_ntt_inv(c, ip.data(), 0, 0, 2, P + l + 1, W);
    orc_hybrid_moddown(c, out, ip.data(), l);
    orc_ntt_fwd(c, out, 0, P, 2, l + 1, Q);
    return 0;
}

// ------------------------------------------------------------------------------------------------
// ring-packed PCMM
// ------------------------------------------------------------------------------------------------
struct orc_pcmm {
    const orc_ctx* ctx; int N1, rank, np, nq;
    std::vector<u64> pq, mu_hi, mu_lo;
};
// PCMM_Context.cuh:7-36
orc_pcmm* orc_pcmm_create(const orc_ctx* c, int N1, int rank, const u64* p, int np, const u64* q, int nq) {
    orc_pcmm* h = new orc_pcmm(); h->ctx = c; h->N1 = N1; h->rank = rank; h->np = np; h->nq = nq;
    for (int i = 0; i < np; i++) h->pq.push_back(p[i]);
    for (int i = 0; i < nq; i++) h->pq.push_back(q[i]);
    h->mu_hi.resize(np + nq); h->mu_lo.resize(np + nq);
    for (int i = 0; i < np + nq; i++) orc_barrett_mu(h->pq[i], &h->mu_hi[i], &h->mu_lo[i]);
    return h;
}
void orc_pcmm_destroy(orc_pcmm* h) { delete h; }

static inline u64 negate_modq(u64 a, u64 q) { return a == 0 ? 0 : q - a; }    // uint128.cuh:309-313

// PCMM_Scheme.cuh:50-88 (the gather kernel only; coefficient-domain input)
int orc_rlwe_decompose(const orc_pcmm* h, const u64* rlwe, u64* const* mlwe, int mlwe_num, int l) {
    const orc_ctx* c = h->ctx; const long N = c->N; const int N1 = h->N1, k = h->rank, L = c->L, P = c->p_num;
    if (mlwe_num > k || mlwe_num <= 0 || (long)N1 * k != N) return -1;
    const int gap = k / mlwe_num;
    for (int m = 0; m < mlwe_num; m++)
        for (int im = 0; im <= l; im++) {
            u64 q = c->pqt[P + im];
            const u64* A = rlwe + N * im; const u64* B = rlwe + N * (L + 1 + im);
            u64* ax = mlwe[m] + (long)N1 * (k + 1) * im; u64* bx = ax + (long)N1 * k;
            for (int g = 0; g < N1; g++) {
                long addr = (long)m * gap + (long)g * k; bool over = addr >= N;
                ax[g] = over ? negate_modq(A[addr - N], q) : A[addr];
                bx[g] = over ? negate_modq(B[addr - N], q) : B[addr];
                for (int i = 1; i < k; i++) {
                    if (g == 0) {
                        addr = (long)(N1 - 1) * k + (k - i) + (long)m * gap; over = addr >= N;
                        ax[g + (long)i * N1] = over ? A[addr - N] : negate_modq(A[addr], q);
                    } else {
                        addr = (long)(g - 1) * k + (k - i) + (long)m * gap; over = addr >= N;
                        ax[g + (long)i * N1] = over ? negate_modq(A[addr - N], q) : A[addr];
                    }
                }
            }
        }
    return 0;
}

// PPMM_kernel.cuh:12-31, 93-252.  Generalised from the reference's two ring-pack primes to mod_num primes:
// the fused rescale divides by the LAST prime and uses (q_last)^-1 mod q_i, which for mod_num == 2 is exactly the
// table row the reference hard-wires (l = 1, PPMM_kernel.cuh:298,310).
int orc_ppmm(const orc_pcmm* h, const float* W, const u64* const* mlwe, u64* out, int M, int Kin, int mod_num,
             double scaler, long col_begin, long col_count) {
    const int N1 = h->N1, k = h->rank, np = h->np;
    if (mod_num < 1 || mod_num > h->nq) return -1;
    const long C = (long)(k + 1) * N1;
    if (col_begin < 0 || col_begin + col_count > C) return -1;
    std::vector<int64_t> A((size_t)M * Kin);
    for (long i = 0; i < (long)M * Kin; i++) A[i] = (int64_t)((double)W[i] * scaler);   // :148 float*double -> int64 (trunc)
    const u64 qlast = h->pq[np + mod_num - 1];
    for (int im = mod_num - 1; im >= 0; im--) {
        const u64 q = h->pq[np + im], mh = h->mu_hi[np + im], ml = h->mu_lo[np + im];
        u64 qinv = 0, qinv_s = 0;
        if (im != mod_num - 1) { qinv = orc_invmod(qlast, q); qinv_s = orc_xshoup(qinv, q); }   // Context_23.cuh:425-436
#pragma omp parallel for schedule(static)
        for (int m = 0; m < M; m++) {
            std::vector<u64> a(Kin);
            for (int n = 0; n < Kin; n++) { int64_t t = A[(size_t)m * Kin + n]; a[n] = t > 0 ? (u64)t : q + (u64)t; }   // :25
            for (long cc = col_begin; cc < col_begin + col_count; cc++) {
                u128 acc = 0;
                for (int n = 0; n < Kin; n++) acc += (u128)a[n] * mlwe[n][(long)im * C + cc];
                u64 r = orc_barrett128((u64)(acc >> 64), (u64)acc, q, mh, ml);
                u64* o = out + (long)m * C * mod_num;
                if (im == mod_num - 1) o[(long)im * C + cc] = r;                                 // :213-229
                else {
                    u64 temp = r + q - o[(long)(mod_num - 1) * C + cc];                          // :244
                    o[(long)im * C + cc] = orc_mulmod_shoup(temp, qinv, qinv_s, q);              // :247
                }
            }
        }
    }
    return 0;
}

// PCMM_Scheme::mlweCipherPacking (PCMM_Scheme.cuh:361-425) with its kernels: mlweCipherEmbedding_new_kernel (:309-358),
// mlweCipherMultRepackingKey_kernel (:262-289), ringpacking_ModDown_kernel (:291-306).
//   mlwe[m]   : [(nq-1) moduli][(rank+1)][N1]  (the PPMM output rows after the fused rescale), coefficient domain
//   keys      : rank switching keys, key i at keys + i*N*mod_num*2 = [a: mod_num limbs | b: mod_num limbs], NTT domain,
//               mod_num = np + nq - 1 limbs over the context primes K-np .. K-np+mod_num-1 (PCMM_Scheme.cuh:166-171)
//   rlwe_out  : [a: L+1 limbs | b: L+1 limbs]; limbs 0 .. nq-2 of both are written (NTT domain), level nq-2
// The reference's embedding writes the lifted value of modulus idx_mod to limb idx_mod and the value itself to limb
// np + idx_mod (:333-339), which only makes sense for one special prime and one remaining modulus; that is what is accepted.
int orc_mlwe_pack(const orc_pcmm* h, u64* rlwe_out, const u64* const* mlwe, int mlwe_num, const u64* keys) {
    const orc_ctx* c = h->ctx; const long N = c->N; const int N1 = h->N1, k = h->rank, np = h->np, nq = h->nq, K = c->p_num, L = c->L;
    if (np != 1 || nq != 2 || mlwe_num <= 0 || mlwe_num > k || k % mlwe_num || (long)N1 * k != N || K < np) return -1;
    const int mod_num = np + nq - 1, first_prime = K - np;
    for (int i = 0; i < mod_num; i++) if (c->pqt[first_prime + i] != h->pq[i]) return -1;
    const int gap = k / mlwe_num;
    const u64 p0 = h->pq[0];
    // embedding + centred lift q -> p (:309-340); the buffer starts zeroed (:386)
    std::vector<u64> embed((size_t)(k + 1) * mod_num * N, 0);
    for (int m = 0; m < mlwe_num; m++)
        for (int im = 0; im < nq - 1; im++) {
            const u64 qi = h->pq[np + im];
            for (int i = 0; i <= k; i++)
                for (int n = 0; n < N1; n++) {
                    const u64 v = mlwe[m][(long)im * N1 * (k + 1) + (long)i * N1 + n];
                    u64* big = embed.data() + (size_t)i * N * mod_num;
                    const long pos = (long)n * k + (long)m * gap;
                    big[(long)(np + im) * N + pos] = v;
                    big[(long)im * N + pos] = v > qi / 2 ? (p0 - (qi - v)) % p0 : v;
                }
        }
    // NTT of the k "a" polynomials over [p0, q0] (:389)
    orc_ntt_fwd(c, embed.data(), 0, first_prime, k, mod_num, mod_num);
    // sum_i a_i * key_i (:262-289): 128-bit accumulation, one Barrett reduction
    std::vector<u64> acc((size_t)2 * mod_num * N);
    for (int im = 0; im < mod_num; im++) {
        const u64 q = h->pq[im], mh = h->mu_hi[im], ml = h->mu_lo[im];
#pragma omp parallel for schedule(static)
        for (long x = 0; x < N; x++) {
            u128 sa = 0, sb = 0;
            for (int i = 0; i < k; i++) {
                const u64 ca = embed[(size_t)i * N * mod_num + (size_t)im * N + x];
                const u64* key = keys + (size_t)i * N * mod_num * 2;
                sa += (u128)ca * key[(size_t)im * N + x];
                sb += (u128)ca * key[(size_t)(im + mod_num) * N + x];
            }
            acc[(size_t)im * N + x] = orc_barrett128((u64)(sa >> 64), (u64)sa, q, mh, ml);
            acc[(size_t)(mod_num + im) * N + x] = orc_barrett128((u64)(sb >> 64), (u64)sb, q, mh, ml);
        }
    }
    orc_ntt_inv(c, acc.data(), 0, first_prime, 2, mod_num, mod_num);                         // :405
    // ModDown pq -> q (:291-306) and + (0, b) (:417)
    for (int y = 0; y < 2; y++)
        for (int im = 0; im < nq - 1; im++) {
            const u64 qi = h->pq[np + im];
            const u64 pinv = orc_invmod(p0 % qi, qi), pinv_s = orc_xshoup(pinv, qi);          // PCMM_Context.cuh:47-56
            const u64* in = acc.data() + (size_t)y * N * mod_num;
            u64* out = rlwe_out + (size_t)y * N * (L + 1) + (size_t)im * N;
            const u64* bpoly = embed.data() + (size_t)k * N * mod_num + (size_t)(np + im) * N;
            for (long x = 0; x < N; x++) {
                u64 ra = in[(size_t)im * N + x] % qi;
                ra = qi - ra + in[(size_t)(np + im) * N + x];
                u64 r = orc_mulmod_shoup(ra, pinv, pinv_s, qi);
                if (y == 1) { r += bpoly[x]; if (r >= qi) r -= qi; }
                out[x] = r;
            }
        }
    orc_ntt_fwd(c, rlwe_out, 0, K, 2, nq - 1, L + 1);                                        // :419
    return 0;
}

// PCMM_Context::ToNTTInplace / FromNTTInplace (PCMM_Context.cuh:243-273) with NTT256_kernel / INTT256_kernel
// (smallntt_60bit.cuh:7-152): the negacyclic transform of size N1 over the ring-pack primes, root findMthRootOfUnity(2*N1, q)
// (PCMM_Context.cuh:31), tables as fillTablePsi128_special (:73-77).  Layout [batch][mod][poly][N1]; prime of limb (z, j, y) is
// pq_ringpack[start_mod_idx + j]; the kernels ignore start_poly_idx (:27-29).  The reference runs N1 = 256 only (:256,271).
int orc_pcmm_ntt(const orc_pcmm* h, u64* data, int poly_num, int mod_num, int start_mod_idx, int mod_batch_size, int inverse) {
    const uint32_t n1 = (uint32_t)h->N1;
    if (poly_num < 0 || mod_num < 0 || start_mod_idx < 0 || start_mod_idx + mod_num > h->np + h->nq || (n1 & (n1 - 1)) || n1 < 2) return -1;
    for (int j = 0; j < mod_num; j++) {
        const u64 q = h->pq[start_mod_idx + j];
        if ((q - 1) % (2 * (u64)n1)) return -1;
        const u64 psi = orc_find_mth_root(2 * (u64)n1, q);
        std::vector<u64> tab(n1), itab(n1);
        orc_fill_psi_tables(psi, q, n1, tab.data(), itab.data(), nullptr, nullptr);
        const u64 ninv = orc_invmod(n1 % q, q);
        for (int z = 0; z < mod_batch_size; z++)
            for (int y = 0; y < poly_num; y++) {
                u64* limb = data + (((size_t)z * mod_num + j) * poly_num + y) * n1;
                if (inverse) orc_intt_limb(limb, n1, q, itab.data(), ninv);
                else orc_ntt_limb(limb, n1, q, tab.data());
            }
    }
    return 0;
}

// ------------------------------------------------------------------------------------------------
// randomness, samplers, pointwise arithmetic, keys, encryption, coefficient encoding
// ------------------------------------------------------------------------------------------------
static inline uint32_t rotl32(uint32_t u, int c) { return (u << c) | (u >> (32 - c)); }
static inline uint32_t le32(const uint8_t* x) { return (uint32_t)x[0] | ((uint32_t)x[1] << 8) | ((uint32_t)x[2] << 16) | ((uint32_t)x[3] << 24); }

// RNG::generateRandom_device (RNG.cuh:18-56) + VecCrypt (RNG_impl.cuh:72-176): the buffer is zeroed and the Salsa20/20 key stream
// of (key, 64-bit nonce) is XORed in, 64-byte block b at offset 64*b with block counter b.  The reference never initialises its
// `sigma` constant (RNG_impl.cuh:37), i.e. runs with zero diagonal words; here the diagonal is Salsa20's "expand 32-byte k",
// which makes the stream the published cipher's (pinned by the ECRYPT vectors).  A trailing partial block is truncated (the
// reference stops at floor(n/64) blocks).
void orc_salsa20_stream(uint8_t* out, size_t n, const uint8_t key[32], uint64_t nonce) {
    static const uint8_t sigma[17] = "expand 32-byte k";
    const size_t blocks = (n + 63) / 64;
    for (size_t b = 0; b < blocks; b++) {
        uint32_t j[16], x[16];
        j[0] = le32(sigma); j[5] = le32(sigma + 4); j[10] = le32(sigma + 8); j[15] = le32(sigma + 12);
        for (int i = 0; i < 4; i++) { j[1 + i] = le32(key + 4 * i); j[11 + i] = le32(key + 16 + 4 * i); }
        j[6] = (uint32_t)nonce; j[7] = (uint32_t)(nonce >> 32);
        j[8] = (uint32_t)b; j[9] = (uint32_t)((uint64_t)b >> 32);
        memcpy(x, j, sizeof(x));
        for (int r = 0; r < 20; r += 2) {
#define ORC_QR(a, b_, c, d) x[b_] ^= rotl32(x[a] + x[d], 7); x[c] ^= rotl32(x[b_] + x[a], 9); x[d] ^= rotl32(x[c] + x[b_], 13); x[a] ^= rotl32(x[d] + x[c], 18);
            ORC_QR(0, 4, 8, 12) ORC_QR(5, 9, 13, 1) ORC_QR(10, 14, 2, 6) ORC_QR(15, 3, 7, 11)     // columns
            ORC_QR(0, 1, 2, 3) ORC_QR(5, 6, 7, 4) ORC_QR(10, 11, 8, 9) ORC_QR(15, 12, 13, 14)      // rows
#undef ORC_QR
        }
        uint8_t blk[64];
        for (int i = 0; i < 16; i++) {
            uint32_t v = x[i] + j[i];
            blk[4 * i] = (uint8_t)v; blk[4 * i + 1] = (uint8_t)(v >> 8); blk[4 * i + 2] = (uint8_t)(v >> 16); blk[4 * i + 3] = (uint8_t)(v >> 24);
        }
        const size_t take = (n - 64 * b < 64) ? n - 64 * b : 64;
        memcpy(out + 64 * b, blk, take);
    }
}

// convert_gaussian_xq (Sampler_impl.cuh:27-70) maps a 32-bit word u to trunc(3.2 * Phi^-1(u / (2^32 - 1))) in float arithmetic,
// clamped to +-19.2.  That is a non-decreasing step function of u.  The oracle states it by its steps with the probability
// taken at the middle of the word's cell, p = (u + 0.5) / 2^32:  value >= k  <=>  p >= Phi(k / 3.2)  <=>  u >= thr[k-1],
// thr[k-1] = 2^32 - floor(2^32 * Q(k / 3.2) + 0.5), Q the upper tail 0.5 * erfc(x / sqrt 2), k = 1..19; negative side by the
// symmetry u -> 2^32 - 1 - u.  It differs from the float pipeline only for words within float rounding of a step
// (distribution-level agreement; the exact stream of the reference is not reproducible anyway: its key and nonce are rand()).
void orc_gauss_thresholds(uint32_t thr[19]) {
    for (int k = 1; k <= 19; k++) {
        const double tail = 0.5 * erfc(((double)k / 3.2) / sqrt(2.0));
        thr[k - 1] = (uint32_t)(4294967296.0 - floor(4294967296.0 * tail + 0.5));
    }
}
static int gauss_value(uint32_t u, const uint32_t thr[19]) {
    int v = 0;
    for (int k = 0; k < 19; k++) { v += (u >= thr[k]); v -= ((uint32_t)~u >= thr[k]); }
    return v;
}

// Sampler::uniformSampler_xq / convert_uniform_xq (Sampler.cuh:17-22, Sampler_impl.cuh:13-24): word i of mod_num*N 64-bit words
// -> (u64)((double)w / 2^64 * (double)(q - 1)), q = prime idx_mod + i / N, written at out[i + idx_out * N]
int orc_sample_uniform(const orc_ctx* c, const uint8_t* random, u64* out, int idx_out, int idx_mod, int mod_num) {
    if (idx_mod < 0 || mod_num < 0 || idx_mod + mod_num > (int)c->pqt.size()) return -1;
    const size_t N = (size_t)c->N;
    for (size_t i = 0; i < N * (size_t)mod_num; i++) {
        u64 w; memcpy(&w, random + 8 * i, 8);
        double d = (double)w;
        d /= 18446744073709551616.0;                        // (double)UINT64_MAX rounds to 2^64
        d *= (double)(c->pqt[idx_mod + i / N] - 1);
        out[i + (size_t)idx_out * N] = (u64)d;
    }
    return 0;
}
// Sampler::gaussianSampler_xq / convert_gaussian_xq (Sampler.cuh:24-29, Sampler_impl.cuh:27-70): N 32-bit words, one noise
// coefficient each, written to mod_num limbs as its residue
int orc_sample_gaussian(const orc_ctx* c, const uint8_t* random, u64* out, int idx_out, int idx_mod, int mod_num) {
    if (idx_mod < 0 || mod_num < 0 || idx_mod + mod_num > (int)c->pqt.size()) return -1;
    uint32_t thr[19];
    orc_gauss_thresholds(thr);
    const size_t N = (size_t)c->N;
    for (size_t i = 0; i < N; i++) {
        uint32_t u; memcpy(&u, random + 4 * i, 4);
        const int dd = gauss_value(u, thr);
        for (int t = 0; t < mod_num; t++)
            out[i + ((size_t)idx_out + t) * N] = dd < 0 ? c->pqt[idx_mod + t] + (long long)dd : (u64)dd;
    }
    return 0;
}
// Sampler::ZOSampler / convert_ZO (Sampler.cuh:36-41, Sampler_impl.cuh:96-113): byte d -> 0 if d < 256*prob, 1 if d < 256*(1+prob)/2,
// else q - 1
int orc_sample_zo(const orc_ctx* c, const uint8_t* random, u64* out, double probability, int idx_out, int idx_mod, int mod_num) {
    if (idx_mod < 0 || mod_num < 0 || idx_mod + mod_num > (int)c->pqt.size()) return -1;
    const size_t N = (size_t)c->N;
    for (size_t i = 0; i < N; i++) {
        const float d = (float)random[i];
        for (int t = 0; t < mod_num; t++) {
            const u64 q = c->pqt[idx_mod + t];
            u64 v;
            if (d < 256.0f * probability) v = 0;
            else if (d < 256.0f * (1 + probability) / 2) v = 1;
            else v = q - 1;
            out[i + ((size_t)idx_out + t) * N] = v;
        }
    }
    return 0;
}
// Sampler::HWTSampler / convert_HWT (Sampler.cuh:31-34, Sampler_impl.cuh:74-93): h 32-bit words give positions (low logN bits), h
// bytes after them give signs (byte >= 128 -> 1, else q - 1); output limb of prime t is idx_out + idx_mod + t (the reference adds
// idx_mod to the output offset).  The limbs are zeroed first (the reference writes into fresh cudaMalloc memory,
// SecretKey.cuh:27-29); when two words give the same position the later one wins (the reference leaves that to a race).
int orc_sample_hwt(const orc_ctx* c, const uint8_t* random, u64* out, int h, int idx_out, int idx_mod, int mod_num) {
    if (idx_mod < 0 || mod_num < 0 || idx_mod + mod_num > (int)c->pqt.size() || h < 0) return -1;
    const size_t N = (size_t)c->N;
    for (int t = 0; t < mod_num; t++) {
        u64* limb = out + ((size_t)idx_out + idx_mod + t) * N;
        const u64 q = c->pqt[idx_mod + t];
        memset(limb, 0, 8 * N);
        for (int k = 0; k < h; k++) {
            uint32_t w; memcpy(&w, random + 4 * k, 4);
            float d = (float)random[4 * (size_t)h + k];
            d /= (256.0f / 2);
            limb[w & (N - 1)] = d >= 1 ? 1 : q - 1;
        }
    }
    return 0;
}

// barrett_batch_3param_device, poly_add_3param_batch_device, poly_sub_3param_batch_device (poly_arithmetic.cuh:101-105, 423-427,
// 481-485): c[idx_c + t] = a[idx_a + t] (op) b[idx_b + t] mod prime idx_mod + t, t < mod_num; op 0 mul, 1 add, 2 sub
int orc_poly_op(const orc_ctx* c, int op, u64* out, const u64* a, const u64* b, int idx_c, int idx_a, int idx_b, int idx_mod, int mod_num) {
    if (idx_mod < 0 || mod_num < 0 || idx_mod + mod_num > (int)c->pqt.size() || op < 0 || op > 2) return -1;
    const size_t N = (size_t)c->N;
    for (int t = 0; t < mod_num; t++) {
        const u64 q = c->pqt[idx_mod + t];
        for (size_t i = 0; i < N; i++) {
            const u64 x = a[((size_t)idx_a + t) * N + i], y = b[((size_t)idx_b + t) * N + i];
            u64 r;
            if (op == 0) r = orc_barrett128((u64)(((u128)x * y) >> 64), x * y, q, c->mu_hi[idx_mod + t], c->mu_lo[idx_mod + t]);
            else if (op == 1) r = csub_q(x + y, q);
            else r = csub_q(q + x - y, q);
            out[((size_t)idx_c + t) * N + i] = r;
        }
    }
    return 0;
}

// SecretKey::SecretKey (SecretKey.cuh:18-31): sparse ternary secret over all of [P | Q] from h words + h bytes, then NTT
int orc_keygen_secret(const orc_ctx* c, u64* sx, const uint8_t* random, int h) {
    const int KL = c->K + c->L + 1;
    if (orc_sample_hwt(c, random, sx, h, 0, 0, KL)) return -1;
    return orc_ntt_fwd(c, sx, 0, 0, 1, KL, KL);
}
// Scheme_23::addEncKey (Scheme_23.cuh:54-80): pk = (a, e - a*s) over Q, NTT domain; a from 8*N*(L+1) random bytes, e from 4*N
int orc_keygen_public(const orc_ctx* c, u64* pk, const u64* sx, const uint8_t* random_a, const uint8_t* random_e) {
    const int K = c->K, L1 = c->L + 1;
    const size_t N = (size_t)c->N;
    u64* ax = pk; u64* bx = pk + N * L1;
    std::vector<u64> ex(N * L1);
    if (orc_sample_uniform(c, random_a, ax, 0, K, L1)) return -1;
    orc_sample_gaussian(c, random_e, ex.data(), 0, K, L1);
    orc_ntt_fwd(c, ex.data(), 0, K, 1, L1, L1);
    orc_poly_op(c, 0, bx, ax, sx, 0, 0, K, K, L1);
    orc_poly_op(c, 2, bx, ex.data(), bx, 0, 0, 0, K, L1);               // poly_sub2: b = e - b
    return 0;
}
// Scheme_23::encryptZero + encryptMsg (Scheme_23.cuh:82-112): random = N bytes (v) | N words (e0) | N words (e1);
// a = v*pk.a + e0, b = v*pk.b + e1 (+ m), limbs 0..l of a ciphertext [a: L+1 | b: L+1]; mx may be null
int orc_encrypt(const orc_ctx* c, u64* cipher, const u64* mx, const u64* pk, const uint8_t* random, int l) {
    const int K = c->K, L1 = c->L + 1;
    if (l < 0 || l > c->L) return -1;
    const size_t N = (size_t)c->N;
    u64* ax = cipher; u64* bx = cipher + N * L1;
    std::vector<u64> vx(N * L1), ex(N * L1);
    orc_sample_zo(c, random, vx.data(), 0.5, 0, K, l + 1);
    orc_ntt_fwd(c, vx.data(), 0, K, 1, l + 1, L1);
    orc_poly_op(c, 0, ax, vx.data(), pk, 0, 0, 0, K, l + 1);
    orc_sample_gaussian(c, random + N, ex.data(), 0, K, l + 1);
    orc_ntt_fwd(c, ex.data(), 0, K, 1, l + 1, L1);
    orc_poly_op(c, 1, ax, ax, ex.data(), 0, 0, 0, K, l + 1);
    orc_poly_op(c, 0, bx, vx.data(), pk + N * L1, 0, 0, 0, K, l + 1);
    orc_sample_gaussian(c, random + N + 4 * N, ex.data(), 0, K, l + 1);
    orc_ntt_fwd(c, ex.data(), 0, K, 1, l + 1, L1);
    orc_poly_op(c, 1, bx, bx, ex.data(), 0, 0, 0, K, l + 1);
    if (mx) orc_poly_op(c, 1, bx, bx, mx, 0, 0, 0, K, l + 1);
    return 0;
}
// Scheme_23::decryptMsg (Scheme_23.cuh:114-127): m = a*s + b on limbs 0..l, limbs above zeroed
int orc_decrypt(const orc_ctx* c, u64* mx, const u64* cipher, const u64* sx, int l) {
    const int K = c->K, L1 = c->L + 1;
    if (l < 0 || l > c->L) return -1;
    const size_t N = (size_t)c->N;
    memset(mx + (size_t)(l + 1) * N, 0, 8 * N * (size_t)(c->L - l));
    orc_poly_op(c, 0, mx, cipher, sx, 0, 0, K, K, l + 1);
    orc_poly_op(c, 1, mx, mx, cipher + N * L1, 0, 0, 0, K, l + 1);
    return 0;
}
// Context_23::encode_coeffs (Encoder.cuh:67-96): coefficient i = (long)(vals[i] * scale) reduced modulo each q_j, then NTT.
// The reference stores q + data for negative data, which is the residue whenever |data| < q; the true residue is taken here.
int orc_encode_coeffs(const orc_ctx* c, u64* mx, const double* vals, long scale, int l) {
    const int K = c->K, L1 = c->L + 1;
    if (l < 0 || l > c->L) return -1;
    const size_t N = (size_t)c->N;
    for (int j = 0; j <= l; j++) {
        const u64 q = c->pqt[K + j];
        for (size_t i = 0; i < N; i++) {
            const long data = (long)(vals[i] * scale);
            const long r = data % (long)q;
            mx[(size_t)j * N + i] = r < 0 ? (u64)(r + (long)q) : (u64)r;
        }
    }
    return orc_ntt_fwd(c, mx, 0, K, 1, l + 1, L1);
}

// ------------------------------------------------------------------------------------------------
// automorphisms in the NTT domain, switching keys in the T basis, homomorphic multiply / rotate / conjugate
// ------------------------------------------------------------------------------------------------
// Context_23.cuh:648-659: rotGroups[i] = 5^i mod 2N
u64 orc_rot_group(const orc_ctx* c, long idx) {
    const u64 M = 2 * (u64)c->N;
    u64 r = 1;
    for (long i = 0; i < idx; i++) r = r * 5 % M;
    return r;
}
// sk_and_poly_LeftRot_ntt_kernel / sk_and_poly_LeftRot_inv_kernel (poly_arithmetic.cuh:581-596, 639-653): NTT slot i holds the
// evaluation at psi^(2*bitrev(i)+1); out[j] = in[i] with 2*bitrev(j)+1 = pow * (2*bitrev(i)+1) mod 2N, on mod_num limbs
int orc_automorph_ntt(const orc_ctx* c, u64* out, const u64* in, u64 pow, int idx_out, int idx_in, int mod_num) {
    const long N = c->N;
    const u64 mask = 2 * (u64)N - 1;
    for (int t = 0; t < mod_num; t++)
        for (long i = 0; i < N; i++) {
            u64 e = 2 * (u64)orc_bitrev((uint32_t)i, c->logN) + 1;
            u64 j = (((pow * e) & mask) - 1) >> 1;
            out[((long)idx_out + t) * N + orc_bitrev((uint32_t)j, c->logN)] = in[((long)idx_in + t) * N + i];
        }
    return 0;
}
// sk_and_poly_conjugate_kernel (poly_arithmetic.cuh:666-674): out[i] = in[N-1-i]
int orc_conjugate_ntt(const orc_ctx* c, u64* out, const u64* in, int idx_out, int idx_in, int mod_num) {
    const long N = c->N;
    for (int t = 0; t < mod_num; t++)
        for (long i = 0; i < N; i++) out[((long)idx_out + t) * N + i] = in[((long)idx_in + t) * N + N - 1 - i];
    return 0;
}

// The body shared by Scheme_23::addMultKey_23 / addConjKey_23 / addLeftRotKey_23 (KeySwitch_23.cuh:36-64, 85-113, 136-165):
// digit i of the key is (a_i, P * s_from restricted to the digit's primes + e_i - a_i * s_to) over [P | Q], taken to the
// coefficient domain, lifted to the T basis block by block (modUpPQtoT_23) and transformed there.
// s_to: K+L+1 limbs (pqt order), s_from: L+1 limbs over Q, both NTT domain; random_a: dnum * 8*N*(K+L+1) bytes,
// random_e: dnum * 4*N bytes; swk: Key_decomp layout [2][dnum][Ri_blockNum * t_num] limbs.
int orc_keygen_switch_23(const orc_ctx* c, u64* swk, const u64* s_to, const u64* s_from, const uint8_t* random_a, const uint8_t* random_e) {
    const long N = c->N;
    const int K = c->K, L = c->L, T = c->t_num, RB = c->Ri_blockNum, dnum = c->dnum, KL = K + L + 1;
    if (K <= 0 || T <= 0 || RB * T < KL) return -1;
    const size_t digit = (size_t)N * T * RB;
    u64* ax = swk; u64* bx = swk + digit * dnum;
    std::vector<u64> temp((size_t)N * KL), ex((size_t)N * KL);
    for (int i = 0; i < dnum; i++) {
        std::fill(temp.begin(), temp.end(), 0);
        for (int t = 0; t < K && i * K + t <= L; t++) {                            // sxsx_mul_P_3param (poly_arithmetic.cuh:526-541)
            const int prime = K + i * K + t;
            const u64 q = c->pqt[prime], Pq = c->PModqt[prime - K];
            for (long x = 0; x < N; x++) {
                const u64 a = s_from[((long)i * K + t) * N + x];
                temp[(size_t)prime * N + x] = orc_barrett128((u64)(((u128)a * Pq) >> 64), a * Pq, q, c->mu_hi[prime], c->mu_lo[prime]);
            }
        }
        orc_sample_gaussian(c, random_e + (size_t)i * N * 4, ex.data(), 0, 0, KL);
        orc_ntt_fwd(c, ex.data(), 0, 0, 1, KL, KL);
        orc_poly_op(c, 1, temp.data(), temp.data(), ex.data(), 0, 0, 0, 0, KL);
        orc_sample_uniform(c, random_a + (size_t)i * N * KL * 8, ax + digit * i, 0, 0, KL);
        orc_poly_op(c, 0, bx + digit * i, ax + digit * i, s_to, 0, 0, 0, 0, KL);
        orc_poly_op(c, 2, bx + digit * i, temp.data(), bx + digit * i, 0, 0, 0, 0, KL);     // poly_sub2: b = temp - b
    }
    orc_ntt_inv(c, ax, 0, 0, dnum, KL, T * RB);
    orc_ntt_inv(c, bx, 0, 0, dnum, KL, T * RB);
    for (int i = 0; i < dnum; i++)
        for (u64* part : {ax + digit * i, bx + digit * i}) {
            std::copy(part, part + (size_t)N * KL, temp.begin());
            if (orc_modup_pq_to_t(c, part, temp.data(), L, 1)) return -1;
        }
    return orc_ntt_fwd(c, swk, 0, KL, dnum * RB * 2, T, T);
}

// compute_c0c1c2_kernel (poly_arithmetic.cuh:787-818): a1*a2, b1*b2 and a1*b2 + a2*b1 through (a1+b1)(a2+b2) in 128 bits
static void tensor_c0c1c2(const orc_ctx* c, u64* axbx, u64* axax, u64* bxbx, const u64* a1, const u64* a2, const u64* b1, const u64* b2, int limbs) {
    const long N = c->N; const int K = c->K;
    for (int t = 0; t < limbs; t++) {
        const u64 q = c->pqt[K + t], mh = c->mu_hi[K + t], ml = c->mu_lo[K + t];
        for (long x = 0; x < N; x++) {
            const long o = (long)t * N + x;
            const u128 t1 = (u128)a1[o] * a2[o], t2 = (u128)b1[o] * b2[o];
            const u128 t3 = (u128)(a1[o] + b1[o]) * (a2[o] + b2[o]) - t1 - t2;
            axax[o] = orc_barrett128((u64)(t1 >> 64), (u64)t1, q, mh, ml);
            bxbx[o] = orc_barrett128((u64)(t2 >> 64), (u64)t2, q, mh, ml);
            axbx[o] = orc_barrett128((u64)(t3 >> 64), (u64)t3, q, mh, ml);
        }
    }
}
// Scheme_23::mult_23 (KeySwitch_23.cuh:192-236): out = [a | b] with L+1 limbs each, limbs 0..l written
int orc_mult_23(const orc_ctx* c, u64* out, const u64* c1, const u64* c2, const u64* rlk, int l) {
    const long N = c->N; const int K = c->K, L1 = c->L + 1;
    if (l < 1 || l > c->L) return -4;
    std::vector<u64> axbx((size_t)N * L1, 0), axax((size_t)N * L1, 0), bxbx((size_t)N * L1, 0);
    tensor_c0c1c2(c, axbx.data(), axax.data(), bxbx.data(), c1, c2, c1 + N * L1, c2 + N * L1, l + 1);
    if (orc_keyswitch_23(c, out, axax.data(), rlk, l)) return -1;
    orc_poly_op(c, 1, out, out, axbx.data(), 0, 0, 0, K, l + 1);                   // cipher_add_axbx_batch_device (:159-172)
    orc_poly_op(c, 1, out + N * L1, out + N * L1, bxbx.data(), 0, 0, 0, K, l + 1);
    return 0;
}
// Scheme_23::leftRotate_23 (KeySwitch_23.cuh:556-586): key switch of a, + b, then the slot permutation with 5^(N/2 - rot)
int orc_rotate_23(const orc_ctx* c, u64* out, const u64* cipher, const u64* rotkey, long rot, int l) {
    const long N = c->N; const int K = c->K, L1 = c->L + 1;
    if (l < 0 || l > c->L || rot < 0 || rot > N / 2) return -1;
    std::vector<u64> tmp((size_t)2 * N * L1, 0);
    if (orc_keyswitch_23(c, tmp.data(), cipher, rotkey, l)) return -1;
    orc_poly_op(c, 1, tmp.data() + N * L1, tmp.data() + N * L1, cipher + N * L1, 0, 0, 0, K, l + 1);
    const u64 pow = orc_rot_group(c, N / 2 - rot);
    orc_automorph_ntt(c, out, tmp.data(), pow, 0, 0, l + 1);
    orc_automorph_ntt(c, out + N * L1, tmp.data() + N * L1, pow, 0, 0, l + 1);
    return 0;
}
// Scheme_23::conjugate_23 (KeySwitch_23.cuh:433-468): reverse both polynomials, key switch of the reversed a, + reversed b
int orc_conjugate_23(const orc_ctx* c, u64* out, const u64* cipher, const u64* conjkey, int l) {
    const long N = c->N; const int K = c->K, L1 = c->L + 1;
    if (l < 0 || l > c->L) return -1;
    std::vector<u64> ar((size_t)N * L1, 0), br((size_t)N * L1, 0);
    orc_conjugate_ntt(c, br.data(), cipher + N * L1, 0, 0, l + 1);
    orc_conjugate_ntt(c, ar.data(), cipher, 0, 0, l + 1);
    if (orc_keyswitch_23(c, out, ar.data(), conjkey, l)) return -1;
    orc_poly_op(c, 1, out + N * L1, out + N * L1, br.data(), 0, 0, 0, K, l + 1);
    return 0;
}

// ------------------------------------------------------------------------------------------------
// hoisted rotations of the slot <-> coefficient transforms (baby-step / giant-step over the T basis)
// ------------------------------------------------------------------------------------------------
// index the kernels read for output slot x under the rotation by `slots` (Bootstrapping_C2S_S2C_impl.cuh:37-41, 175-179):
// with e = 2 * bitrev(x) + 1, bitrev(((5^slots * e mod 2N) - 1) / 2)
static inline long hoist_perm(const orc_ctx* c, u64 pow, long x) {
    const u64 mask = 2 * (u64)c->N - 1;
    u64 e = 2 * (u64)orc_bitrev((uint32_t)x, c->logN) + 1;
    e = (((pow * e) & mask) - 1) >> 1;
    return (long)orc_bitrev((uint32_t)e, c->logN);
}
// cipher_mul_P_batch as the transforms call it (poly_arithmetic.cuh:863-887, Bootstrapping_C2S_S2C_impl.cuh:270): out is a pair over
// [P | Q] (K+L+1 limbs each); the special limbs are zero, limb K+i = cipher limb i times (P mod q_i), i <= l; the rest is untouched
int orc_cipher_mul_p(const orc_ctx* c, u64* out, const u64* cipher, int l) {
    const long N = c->N; const int K = c->K, L = c->L;
    if (l < 0 || l > L || K <= 0) return -1;
    for (int z = 0; z < 2; z++) {
        std::fill(out + (size_t)z * (K + L + 1) * N, out + ((size_t)z * (K + L + 1) + K) * N, 0);
        for (int i = 0; i <= l; i++) {
            const u64 q = c->pqt[K + i];
            for (long x = 0; x < N; x++)
                out[((size_t)z * (K + L + 1) + K + i) * N + x] = orc_mulmod(cipher[((size_t)z * (L + 1) + i) * N + x], c->PModqt[i], q);
        }
    }
    return 0;
}
// cipher_add_T_batch_device (poly_arithmetic.cuh:143-153, 409-413): a += b on `blocks` groups of t_num limbs modulo the T primes
int orc_cipher_add_t(const orc_ctx* c, u64* a, const u64* b, int blocks) {
    const long N = c->N; const int T = c->t_num, base = c->p_num + c->q_num;
    if (T <= 0 || blocks < 0) return -1;
    for (int z = 0; z < blocks; z++)
        for (int k = 0; k < T; k++) {
            const u64 t = c->pqt[base + k];
            for (long x = 0; x < N; x++) {
                const size_t i = ((size_t)z * T + k) * N + x;
                a[i] = csub_q(a[i] + b[i], t);
            }
        }
    return 0;
}
// Scheme_23::rescaleAndEqual_noNTT (Scheme_23.cuh:321-337, 427-440): coefficient-domain pair, limb i < l becomes
// (c_i + 2 q_i - c_l) * q_l^-1 mod q_i with the last limb used as an integer, not reduced modulo q_i first
int orc_rescale_coeff(const orc_ctx* c, u64* cipher, int l) {
    const long N = c->N; const int K = c->K, L = c->L;
    if (l < 1 || l > L) return -1;
    const u64* inv = &c->qiInvModql[(size_t)l * (l - 1) / 2]; const u64* inv_s = &c->qiInvModql_shoup[(size_t)l * (l - 1) / 2];
    for (int z = 0; z < 2; z++)
        for (int i = 0; i < l; i++) {
            const u64 q = c->pqt[K + i];
            for (long x = 0; x < N; x++) {
                const size_t idx = ((size_t)z * (L + 1) + i) * N + x;
                u64 ra = cipher[idx] + 2 * q - cipher[((size_t)z * (L + 1) + l) * N + x];
                ra = csub_q(ra, q);
                cipher[idx] = orc_mulmod_shoup(ra, inv[i], inv_s[i], q);
            }
        }
    return 0;
}
// EncodingMatrix::Giant_Rotate_And_Mult_PlaintT (Bootstrapping_C2S_S2C_impl.cuh:7-152).  For every rotation j < gs of the giant step
// the rotated pair in the T basis is formed on the fly - without a key (null pointer) the pair P*(a, b) itself, with a key the
// inner product of the digits of a with the key's two halves, plus P*b, all read at the rotation's index - and multiplied into the
// accumulators of the baby steps i < bs whose plaintext j exists (j < accNum[i]): 128-bit sums, one reduction at the end.
// PQ_to_T: [a | b][Ri_blockNum][t_num]; modUp_QjtoT: [digit][t_num]; key: [a | b][dnum][Ri_blockNum][t_num];
// plaintext (i, j): t_num limbs; bs_cipher_T: [bs][a | b][Ri_blockNum][t_num].  Blocks at and beyond ceil((K+l+1)/gamma) are untouched.
int orc_giant_rotate_mult_plain_t(const orc_ctx* c, u64* bs_cipher_T, const u64* PQ_to_T, const u64* modUp_QjtoT, const u64* const* rotKeys,
                                  const int* rotSlots, const u64* const* plaintextT, const int* accNum, int bs, int gs, int l) {
    const long N = c->N; const int g = c->gamma, P = c->p_num, Q = c->q_num, T = c->t_num, RB = c->Ri_blockNum, dnum = c->dnum;
    if (g <= 0 || T <= 0 || P <= 0 || l < 0 || l > c->L || bs < 1 || gs < 1 || bs > 16) return -1;
    const int cipher_blockNum = ceil_div(l + 1, P), blockNum = ceil_div(P + l + 1, g);
    if (cipher_blockNum > dnum) return -1;
    const size_t half = (size_t)RB * T * N;
    std::vector<u64> pows(gs, 1);
    for (int j = 0; j < gs; j++) if (rotKeys[j]) pows[j] = orc_rot_group(c, rotSlots[j]);
#pragma omp parallel for collapse(2) schedule(static)
    for (int blk = 0; blk < blockNum; blk++)
        for (int k = 0; k < T; k++)
            for (long x = 0; x < N; x++) {
                const size_t idx = (size_t)x + ((size_t)blk * T + k) * N;
                u128 acc_a[16], acc_b[16];
                for (int i = 0; i < bs; i++) acc_a[i] = acc_b[i] = 0;
                for (int j = 0; j < gs; j++) {
                    u64 ea, eb;
                    if (!rotKeys[j]) {
                        ea = PQ_to_T[idx]; eb = PQ_to_T[idx + half];
                    } else {
                        const long px = hoist_perm(c, pows[j], x);
                        u128 a1 = 0, a2 = 0;
                        for (int i = 0; i < cipher_blockNum; i++) {
                            const u64 d = modUp_QjtoT[((size_t)i * T + k) * N + px];
                            const size_t kidx = ((size_t)i * T * RB + (size_t)blk * T + k) * N + px;
                            a1 += (u128)d * rotKeys[j][kidx];
                            a2 += (u128)d * rotKeys[j][half * dnum + kidx];
                        }
                        a2 += PQ_to_T[(size_t)px + ((size_t)blk * T + k) * N + half];
                        ea = barrett_idx(c, a1, P + Q + k); eb = barrett_idx(c, a2, P + Q + k);
                    }
                    for (int i = 0; i < bs; i++)
                        if (j < accNum[i]) {
                            const u64 mx = plaintextT[(size_t)i * gs + j][(size_t)k * N + x];
                            acc_a[i] += (u128)ea * mx; acc_b[i] += (u128)eb * mx;
                        }
                }
                for (int i = 0; i < bs; i++) {
                    bs_cipher_T[idx + (size_t)(2 * i) * half] = barrett_idx(c, acc_a[i], P + Q + k);
                    bs_cipher_T[idx + (size_t)(2 * i + 1) * half] = barrett_idx(c, acc_b[i], P + Q + k);
                }
            }
    return 0;
}
// EncodingMatrix::Baby_Rotate (Bootstrapping_C2S_S2C_impl.cuh:154-228): output (a pair in the T basis) += the pair `input` rotated
// with each key given: a += <digits, key_a>, b += <digits, key_b> + input_b, digits / keys / input_b read at the rotation's index
int orc_baby_rotate(const orc_ctx* c, u64* output, const u64* modUp_QjtoT, const u64* input, int rotNum, const u64* const* rotKeys,
                    const int* rotSlots, int l) {
    const long N = c->N; const int g = c->gamma, P = c->p_num, Q = c->q_num, T = c->t_num, RB = c->Ri_blockNum, dnum = c->dnum;
    if (g <= 0 || T <= 0 || P <= 0 || l < 0 || l > c->L || rotNum < 0) return -1;
    const int cipher_blockNum = ceil_div(l + 1, P), blockNum = ceil_div(P + l + 1, g);
    const size_t half = (size_t)RB * T * N;
    for (int r = 0; r < rotNum; r++) {
        if (!rotKeys[r]) continue;
        const u64 pow = orc_rot_group(c, rotSlots[r]);
        std::vector<u64> next_a(half), next_b(half);
#pragma omp parallel for collapse(2) schedule(static)
        for (int blk = 0; blk < blockNum; blk++)
            for (int k = 0; k < T; k++)
                for (long x = 0; x < N; x++) {
                    const size_t idx = (size_t)x + ((size_t)blk * T + k) * N;
                    const long px = hoist_perm(c, pow, x);
                    u128 a1 = 0, a2 = 0;
                    for (int i = 0; i < cipher_blockNum; i++) {
                        const u64 d = modUp_QjtoT[((size_t)i * T + k) * N + px];
                        const size_t kidx = ((size_t)i * T * RB + (size_t)blk * T + k) * N + px;
                        a1 += (u128)d * rotKeys[r][kidx];
                        a2 += (u128)d * rotKeys[r][half * dnum + kidx];
                    }
                    a1 += output[idx];
                    a2 += input[(size_t)px + ((size_t)blk * T + k) * N + half];
                    a2 += output[idx + half];
                    next_a[idx] = barrett_idx(c, a1, P + Q + k); next_b[idx] = barrett_idx(c, a2, P + Q + k);
                }
        for (int blk = 0; blk < blockNum; blk++)
            for (int k = 0; k < T; k++) {
                const size_t o = ((size_t)blk * T + k) * N;
                std::copy(next_a.begin() + o, next_a.begin() + o + N, output + o);
                std::copy(next_b.begin() + o, next_b.begin() + o + N, output + half + o);
            }
    }
    return 0;
}
// One level of EncodingMatrix::EvalCoeffsToSlots / EvalSlotsToCoeffs (Bootstrapping_C2S_S2C_impl.cuh:254-382, 531-625) without
// its final rescale: cipher (coefficient domain, level l, in place) becomes sum_i rot_out[i]( sum_{j < accNum[i]} plain[i][j] *
// rot_in[j](cipher) ).  A rotation by 0 slots takes no key (null).
int orc_bsgs_level_23(const orc_ctx* c, u64* cipher, int l, const u64* const* plaintextT, const int* accNum, const int* rot_in,
                      const u64* const* rot_in_keys, const int* rot_out, const u64* const* rot_out_keys, int bs, int gs) {
    const long N = c->N; const int K = c->K, L = c->L, T = c->t_num, RB = c->Ri_blockNum, g = c->gamma;
    if (g <= 0 || T <= 0 || K <= 0 || l < 0 || l > L || bs < 1 || gs < 1) return -1;
    const int cipher_blockNum = ceil_div(l + 1, K), blockNum = ceil_div(K + l + 1, g);
    const size_t half = (size_t)RB * T * N;
    std::vector<u64> up((size_t)N * T * c->Qj_blockNum, 0), pq((size_t)2 * (K + L + 1) * N, 0), pqT(2 * half, 0), bsT((size_t)bs * 2 * half, 0),
        gsT(2 * half, 0), back(2 * half, 0);          // the T -> PQ buffer keeps the T-basis stride between a and b
    orc_modup_qj_to_t(c, up.data(), cipher, l, 1);                                                   // :262
    orc_ntt_fwd(c, up.data(), 0, K + L + 1, cipher_blockNum, T, T);                                  // :263
    orc_cipher_mul_p(c, pq.data(), cipher, l);                                                       // :267
    orc_modup_pq_to_t(c, pqT.data(), pq.data(), l, 2);                                               // :270
    orc_ntt_fwd_ext(c, pqT.data(), 0, K + L + 1, blockNum, T, T, RB * T, 2);                         // :272
    std::vector<const u64*> keys(gs);
    std::vector<int> slots(gs);
    for (int j = 0; j < gs; j++) { keys[j] = rot_in[j] != 0 ? rot_in_keys[j] : nullptr; slots[j] = rot_in[j] != 0 ? rot_in[j] : -1; }   // :275-288
    if (orc_giant_rotate_mult_plain_t(c, bsT.data(), pqT.data(), up.data(), keys.data(), slots.data(), plaintextT, accNum, bs, gs, l)) return -1;
    for (int i = 1; i < bs; i++) {                                                                   // :326-356
        u64* part = bsT.data() + (size_t)i * 2 * half;
        if (rot_out[i] == 0) { orc_cipher_add_t(c, bsT.data(), part, RB * 2); continue; }
        std::copy(part, part + 2 * half, gsT.begin());
        orc_ntt_inv_ext(c, part, 0, K + L + 1, blockNum, T, T, RB * T, 2);
        orc_modup_t_to_pql(c, back.data(), part, l, 1);
        orc_moddown_pql_to_ql(c, cipher, back.data(), l, 1);
        orc_modup_qj_to_t(c, up.data(), cipher, l, 1);
        orc_ntt_fwd(c, up.data(), 0, K + L + 1, cipher_blockNum, T, T);
        const u64* key1[1] = {rot_out_keys[i]};
        const int slot1[1] = {rot_out[i]};
        if (orc_baby_rotate(c, bsT.data(), up.data(), gsT.data(), 1, key1, slot1, l)) return -1;
    }
    orc_ntt_inv_ext(c, bsT.data(), 0, K + L + 1, blockNum, T, T, RB * T, 2);                         // :359
    orc_modup_t_to_pql(c, back.data(), bsT.data(), l, 2);                                            // :361
    orc_moddown_pql_to_ql(c, cipher, back.data(), l, 2);                                             // :363
    return 0;
}

// ------------------------------------------------------------------------------------------------
// MLWE secret key, repacking keys, MLWE decryption (the key side of the ring-packed PCMM)
// ------------------------------------------------------------------------------------------------
// PCMM_Scheme::convertMLWESKfromRLWESK (PCMM_Scheme.cuh:23-48) with ringDown_kernel (ringSwitch.cuh:7-19): the RLWE secret
// (K+L+1 limbs, NTT domain, left unchanged) goes to the coefficient domain; small polynomial i takes the big coefficients
// i + n*rank (n < N1).  The first launch copies RLWE limbs 0..nq-1 to key moduli 0..nq-1, the second RLWE limbs K..K+nq-1 to key
// moduli np..np+nq-1 (overwriting where they overlap), exactly as the reference's two launches do; then every modulus is
// transformed (size N1).  mlwe_sk: [np+nq moduli][rank][N1].
int orc_pcmm_convert_mlwe_sk(const orc_pcmm* h, u64* mlwe_sk, const u64* rlwe_sk) {
    const orc_ctx* c = h->ctx; const long N = c->N; const int N1 = h->N1, k = h->rank, np = h->np, nq = h->nq, K = c->K, KL = c->K + c->L + 1;
    if ((long)N1 * k != N || nq > KL || K + nq > KL) return -1;
    std::vector<u64> s(rlwe_sk, rlwe_sk + (size_t)KL * N);
    orc_ntt_inv(c, s.data(), 0, 0, 1, KL, KL);
    for (int pass = 0; pass < 2; pass++) {
        const u64* big = s.data() + (pass ? (size_t)K * N : 0);
        u64* small = mlwe_sk + (pass ? (size_t)np * N1 * k : 0);
        for (int im = 0; im < nq; im++)
            for (long g = 0; g < N; g++) small[(size_t)im * N + g] = big[(size_t)im * N + g / N1 + (g % N1) * k];
    }
    return orc_pcmm_ntt(h, mlwe_sk, k, np + nq, 0, 1, 0);
}

// PCMM_Scheme::addRepakcingKey (PCMM_Scheme.cuh:126-224) with EmbedMLWESKtoRLWESK (:126-149): key i over the context primes
// [last np special primes | q_0 .. q_{nq-2}] is (a, -a*s + p0 * iota(s_i) + e), iota placing coefficient n of the small secret at
// n*rank; layout key i at keys + i*2*mod_num*N = [a: mod_num limbs | b: mod_num limbs], mod_num = np+nq-1, NTT domain.
// random: per key 4*N bytes (e) then 8*N*mod_num bytes (a), keys one after the other.  mlwe_sk (NTT domain) is not modified: the
// reference transforms it back on np+nq-1 of its np+nq moduli only (:182), which leaves the last one in the coefficient domain.
// b starts from zero here (the reference writes the embedded secret into fresh cudaMalloc memory).
int orc_pcmm_add_repacking_key(const orc_pcmm* h, u64* keys, const u64* mlwe_sk, const u64* rlwe_sk, const uint8_t* random) {
    const orc_ctx* c = h->ctx; const long N = c->N; const int N1 = h->N1, k = h->rank, np = h->np, nq = h->nq, K = c->K;
    const int mod_num = np + nq - 1, first = K - np;
    if ((long)N1 * k != N || K < np || (nq - 1) / np != 1) return -1;                       // "dnum not supported!" (:178-180)
    for (int i = 0; i < mod_num; i++) if (c->pqt[first + i] != h->pq[i]) return -1;
    std::vector<u64> sk(mlwe_sk, mlwe_sk + (size_t)(np + nq) * N);
    orc_pcmm_ntt(h, sk.data(), k, np + nq, 0, 1, 1);
    const u64 p0 = h->pq[0];
    const size_t per_key = (size_t)4 * N + (size_t)8 * N * mod_num;
    std::vector<u64> ex((size_t)mod_num * N), tmp((size_t)mod_num * N);
    for (int i = 0; i < k; i++) {
        u64* ax = keys + (size_t)i * 2 * mod_num * N;
        u64* bx = ax + (size_t)mod_num * N;
        std::fill(bx, bx + (size_t)mod_num * N, 0);
        for (int im = 0; im < nq - 1; im++) {
            const u64 qi = h->pq[np + im];
            for (int n = 0; n < N1; n++) {
                const u64 v = sk[(size_t)(np + im) * N + (size_t)i * N1 + n];
                bx[(size_t)(np + im) * N + (size_t)n * k] = orc_barrett128((u64)(((u128)v * p0) >> 64), v * p0, qi, h->mu_hi[np + im], h->mu_lo[np + im]);
            }
        }
        const uint8_t* r = random + per_key * i;
        orc_sample_gaussian(c, r, ex.data(), 0, first, mod_num);
        orc_sample_uniform(c, r + 4 * N, ax, 0, first, mod_num);
        orc_poly_op(c, 1, bx, bx, ex.data(), 0, 0, 0, first, mod_num);
        orc_ntt_fwd(c, bx, 0, first, 1, mod_num, mod_num);
        orc_poly_op(c, 0, tmp.data(), rlwe_sk, ax, 0, first, 0, first, mod_num);
        orc_poly_op(c, 2, bx, bx, tmp.data(), 0, 0, 0, first, mod_num);
    }
    return 0;
}

// PCMM_Scheme::mlweDecrypt (PCMM_Scheme.cuh:531-576): plain[mod][n] = b + sum_i a_i * s_i in the size-N1 NTT domain (128-bit
// accumulation, one Barrett reduction), for moduli 0..l of the ciphertext = ring-pack primes np..np+l; the plaintext stays in
// the NTT domain, the ciphertext (coefficient domain) is left unchanged.  mlwe_sk as convertMLWESKfromRLWESK leaves it.
int orc_pcmm_mlwe_decrypt(const orc_pcmm* h, u64* plain, const u64* cipher, const u64* mlwe_sk, int l) {
    const int N1 = h->N1, k = h->rank, np = h->np, nq = h->nq;
    if (l < 0 || l + 1 > nq) return -1;
    std::vector<u64> ct(cipher, cipher + (size_t)(l + 1) * (k + 1) * N1);
    if (orc_pcmm_ntt(h, ct.data(), k + 1, l + 1, np, 1, 0)) return -1;
    for (int im = 0; im <= l; im++) {
        const u64 q = h->pq[np + im], mh = h->mu_hi[np + im], ml = h->mu_lo[np + im];
        const u64* a = ct.data() + (size_t)im * (k + 1) * N1;
        const u64* s = mlwe_sk + (size_t)(np + im) * k * N1;
        for (int n = 0; n < N1; n++) {
            u128 acc = a[(size_t)k * N1 + n];
            for (int i = 0; i < k; i++) acc += (u128)a[(size_t)i * N1 + n] * s[(size_t)i * N1 + n];
            plain[(size_t)im * N1 + n] = orc_barrett128((u64)(acc >> 64), (u64)acc, q, mh, ml);
        }
    }
    return 0;
}
// PCMM_Context::decodeCoeffs (PCMM_Context.cuh:149-178): inverse transform of moduli 0..l, then the centred residue modulo the first
// ring-pack modulus divided by the scale; N1 doubles
int orc_pcmm_decode_coeffs(const orc_pcmm* h, double* vals, const u64* plain, long long scaler, int l) {
    const int N1 = h->N1, np = h->np;
    if (l < 0 || l + 1 > h->nq) return -1;
    std::vector<u64> buf(plain, plain + (size_t)(l + 1) * N1);
    if (orc_pcmm_ntt(h, buf.data(), 1, l + 1, np, 1, 1)) return -1;
    const u64 mod = h->pq[np], mod2 = mod >> 1;
    for (int n = 0; n < N1; n++) {
        const long mi = (long)buf[n];
        vals[n] = (u64)mi <= mod2 ? (double)mi / scaler : ((double)mi - (double)mod) / scaler;
    }
    return 0;
}

int orc_max_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}
