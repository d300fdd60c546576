// C ABI of the MI355X quantized ConvBias / RelayoutFormat path (declared in
// include/mi355_convbias.h): descriptor validation, the shape-keyed algorithm chooser and the
// kernel dispatch.  No allocation, no exceptions; every entry point returns an mi355_status.
#include <math.h>
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include <mutex>
#include <shared_mutex>
#include <unordered_map>
#include <vector>

#include "common.h"

using namespace mi355;

namespace {

thread_local char g_err[256] = "";

int fail(int status, const char* fmt, ...) __attribute__((format(printf, 2, 3)));
int fail(int status, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return status;
}

int in_pack(uint32_t fmt) {
    switch (fmt) {
        case MI355_FMT_NCHW: return 1;
        case MI355_FMT_NCHW4: case MI355_FMT_NCHW44: case MI355_FMT_NCHW4_NCHW32: case MI355_FMT_NCHW4_NCHW: return 4;
        case MI355_FMT_NCHW32: case MI355_FMT_NCHW32_NCHW4: return 32;
        default: return 0;
    }
}
int out_pack(uint32_t fmt) {
    switch (fmt) {
        case MI355_FMT_NCHW: case MI355_FMT_NCHW4_NCHW: return 1;
        case MI355_FMT_NCHW4: case MI355_FMT_NCHW44: case MI355_FMT_NCHW32_NCHW4: return 4;
        case MI355_FMT_NCHW32: case MI355_FMT_NCHW4_NCHW32: return 32;
        default: return 0;
    }
}

// The fast epilogue form needs: positive normal dst scale (RELU folds into the clamp, the
// reciprocal pair is exact enough), and magnitudes that keep every intermediate finite:
// |r| <= 2^31*s_b + 128*s_z, H_SWISH multiplies by at most 6, then r * y_hi.
bool epi_fast_ok(float s_b, float s_z, float s_d, bool has_z) {
    auto sane = [](float s) { return s >= 0x1p-60f && s <= 0x1p40f; };
    if (!(s_d >= 0x1p-40f && s_d <= 0x1p40f)) return false;
    if (!sane(s_b)) return false;
    if (has_z && !sane(s_z)) return false;
    return true;
}

// ---- divide-free quotient of the fast epilogue form (epilogue.h): host-side proof per dst scale --------------------
// From the float r on, the contract is  clamp(roundf(RN(r / s_d)))  and the fast form replaces RN(r / s_d) by
//     t = RN(r y_lo);  q = fma(r, y_hi, t)          y_hi = RN(1 / s_d),  y_lo = RN(1 / s_d - y_hi)
// y_hi + y_lo is 1 / s_d to 2^-48 relative, t carries a rounding error 2^-24 below its own size, which is 2^-24 below q:
// q is r / s_d with a relative error of about 2^-47 before its single rounding, i.e. the correctly rounded quotient
// except where r / s_d lies that close to the midpoint of two floats, and never more than one ulp from it, for every
// s_d and r that epi_fast_ok admits (no intermediate leaves the normal range).  Such a quotient can change the result
// only where RN(r / s_d) lies within one ulp of a rounding boundary k + 0.5 of roundf, i.e. for a handful of consecutive
// floats r around each of the 128 boundary magnitudes.  The proof therefore finds every boundary of the literal chain
// by bisection over the floats and evaluates BOTH forms, with the device's own operations (IEEE multiply and fma, clamp,
// the two integer conversions), on the 33 floats around it, on both signs.  Equal there = equal on every float r.  A
// scale that fails (none is known: 20 000 log-uniform draws and the special scales of the tests all pass) runs the
// literal chain with the IEEE divide.  (One instruction shorter than the reciprocal-times-residual correction it
// replaces: q0 = r y; e = fma(-q0, s_d, r); q = fma(e, y, q0).)
float epi_recip_lo(float s_d) { return (float)(1.0 / (double)s_d - (double)(1.0f / s_d)); }
int epi_tail_contract(float r, float s_d) {
    float v = roundf(r / s_d);
    v = fminf(fmaxf(-128.f, v), 127.f);
    return (int)v;
}
int epi_tail_fast(float r, float y_hi, float y_lo, bool relu) {
    const float t = r * y_lo;
    float q = fmaf(r, y_hi, t);
    if (relu) {
        q = fminf(fmaxf(q, 0.f), 127.f);
        return (int)floor((double)q + 0.5);  // v_cvt_rpi_i32_f32: floor(q + 0.5) without an intermediate rounding
    }
    q = fminf(fmaxf(q, -128.f), 127.f);
    return (int)(q + copysignf(0.49999997f, q));
}
float f_from_bits(uint32_t b) {
    float f;
    memcpy(&f, &b, 4);
    return f;
}
bool epi_prove_quotient(float s_d) {
    const float y_hi = 1.0f / s_d, y_lo = epi_recip_lo(s_d);
    const float top = 130.f * s_d;  // beyond the last boundary: finite by epi_fast_ok
    uint32_t top_bits;
    memcpy(&top_bits, &top, 4);
    if (epi_tail_contract(top, s_d) != 127 || epi_tail_contract(-top, s_d) != -128) return false;
    for (int k = 1; k <= 128; ++k) {
        // smallest magnitude (as a bit pattern) whose negative reaches -k; magnitudes below give > -k
        uint32_t lo = 0, hi = top_bits;  // contract(-lo) = 0 > -k >= contract(-hi)
        while (hi - lo > 1) {
            const uint32_t m = lo + (hi - lo) / 2;
            if (epi_tail_contract(-f_from_bits(m), s_d) <= -k) hi = m; else lo = m;
        }
        for (int d = -16; d <= 16; ++d) {
            const int64_t b = (int64_t)hi + d;
            if (b <= 0 || b >= 0x7f800000) continue;
            const float m = f_from_bits((uint32_t)b);
            if (epi_tail_fast(-m, y_hi, y_lo, false) != epi_tail_contract(-m, s_d)) return false;
            // the positive side has the same boundaries (round half away from zero) up to the clamp at 127
            if (epi_tail_fast(m, y_hi, y_lo, false) != epi_tail_contract(m, s_d)) return false;
            if (epi_tail_fast(m, y_hi, y_lo, true) != epi_tail_contract(m, s_d)) return false;
            if (epi_tail_fast(-m, y_hi, y_lo, true) != 0) return false;  // RELU folded into the clamp
        }
    }
    return true;
}

// Verdicts are kept for the life of the process, one per dst scale: a proof costs ~0.15 ms of host time and an operator
// asks for it on every call, so an entry, once made, is never evicted (a growing hash map; readers share the lock).
// Beyond kProofCacheCap entries -- a caller cycling through millions of distinct scales -- new verdicts are computed
// but no longer stored.
constexpr size_t kProofCacheCap = 1u << 20;

template <class V>
class ProofCache {
public:
    bool find(uint64_t key, V* out) {
        std::shared_lock<std::shared_mutex> lk(mu_);
        auto it = map_.find(key);
        if (it == map_.end()) return false;
        *out = it->second;
        return true;
    }
    void insert(uint64_t key, const V& v) {
        std::unique_lock<std::shared_mutex> lk(mu_);
        if (map_.size() < kProofCacheCap) map_.emplace(key, v);
    }
    size_t size() {
        std::shared_lock<std::shared_mutex> lk(mu_);
        return map_.size();
    }

private:
    std::shared_mutex mu_;
    std::unordered_map<uint64_t, V> map_;
};

ProofCache<bool> g_quot;

bool epi_quotient_proved(float s_d) {
    uint32_t kd;
    memcpy(&kd, &s_d, 4);
    bool ok;
    if (g_quot.find(kd, &ok)) return ok;
    ok = epi_prove_quotient(s_d);
    g_quot.insert(kd, ok);
    return ok;
}

// ---- linear epilogue form (epilogue.h): host-side search and proof ---------------------------------
// The contract without z, as a function of the integer sfb (every operation a separately rounded
// binary32 operation; this host code is compiled without contraction and without fast-math):
int epi_contract(int t, float s_b, float s_d, bool relu) {
    float r = (float)t * s_b;
    if (relu) r = r <= 0.f ? 0.f : r;
    float v = roundf(r / s_d);
    v = fminf(fmaxf(-128.f, v), 127.f);
    return (int)v;
}
// The device's linear form on the same integer: one fused multiply-add, clamp, floor.
int epi_linear(int t, float c, float d, float lo) {
    float x = fmaf((float)t, c, d);
    x = fminf(fmaxf(x, lo), 127.5f);
    return (int)floorf(x);
}

// Finds (c, d) such that epi_linear == epi_contract on EVERY int32, or reports that it found none.
// Both are non-decreasing step functions of t (s_b, s_d, c > 0).  T[k] = the smallest t with contract(t) >= k is
// found by bisection inside [-2^24, 2^24], where float(t) is exact; a candidate is accepted only if
// linear(T[k]) >= k and linear(T[k] - 1) <= k - 1 for every k, which by monotonicity gives equality on all
// of [T[kmin] - 1, T[127]], and on both sides of that range the two functions sit at the same clamp.
bool epi_solve_linear(float s_b, float s_d, bool relu, float* c_out, float* d_out) {
    const int LIM = 1 << 24;
    const int kmin = relu ? 1 : -127, kmax = 127;
    int T[255];
    if (epi_contract(LIM, s_b, s_d, relu) < kmax) return false;
    if (epi_contract(-LIM, s_b, s_d, relu) >= kmin) return false;
    for (int k = kmin; k <= kmax; ++k) {
        int lo = -LIM, hi = LIM;  // contract(lo) < k <= contract(hi)
        while (hi - lo > 1) {
            const int m = lo + (hi - lo) / 2;
            if (epi_contract(m, s_b, s_d, relu) >= k) hi = m; else lo = m;
        }
        T[k - kmin] = hi;
    }
    const float lo_clamp = relu ? 0.f : -128.f;
    const float c0 = (float)((double)s_b / (double)s_d);
    if (!(c0 > 0.f) || !(c0 < 0x1p20f)) return false;
    for (int u = 0; u <= 16; ++u) {
        for (int sgn = -1; sgn <= 1; sgn += 2) {
            if (u == 0 && sgn == 1) continue;
            float c = c0;
            for (int i = 0; i < u; ++i) c = nextafterf(c, sgn > 0 ? INFINITY : 0.f);
            if (!(c > 0.f)) continue;
            // in real arithmetic step k sits at T[k] iff  k - T[k] c <= d < k - (T[k] - 1) c
            double dlo = -1e300, dhi = 1e300;
            for (int k = kmin; k <= kmax; ++k) {
                const double a = (double)k - (double)T[k - kmin] * (double)c;
                if (a > dlo) dlo = a;
                if (a + (double)c < dhi) dhi = a + (double)c;
            }
            if (!(dlo < dhi)) continue;
            for (int j = 1; j <= 3; ++j) {
                const float d = (float)(dlo + (dhi - dlo) * j / 4.0);
                bool ok = true;
                for (int k = kmin; k <= kmax && ok; ++k) {
                    const int t = T[k - kmin];
                    ok = epi_linear(t, c, d, lo_clamp) >= k && epi_linear(t - 1, c, d, lo_clamp) <= k - 1;
                }
                if (ok) {
                    *c_out = c;
                    *d_out = d;
                    return true;
                }
            }
        }
    }
    return false;
}

// Results are kept per (s_b, s_d, activation) for the life of the process (never evicted, see ProofCache): a search is
// ~0.1 ms of host time, a hit a hash lookup.
struct LinEntry {
    bool solved;
    float c, d;
};
ProofCache<LinEntry> g_lin[2];  // [relu]

bool epi_linear_cached(float s_b, float s_d, bool relu, float* c, float* d) {
    uint32_t kb, kd;
    memcpy(&kb, &s_b, 4);
    memcpy(&kd, &s_d, 4);
    const uint64_t key = ((uint64_t)kb << 32) | kd;
    LinEntry e;
    if (!g_lin[relu].find(key, &e)) {
        e.c = e.d = 0.f;
        e.solved = epi_solve_linear(s_b, s_d, relu, &e.c, &e.d);
        g_lin[relu].insert(key, e);
    }
    *c = e.c;
    *d = e.d;
    return e.solved;
}

// ---- residual table form (epilogue.h): the linear form with a residual ------------------------------------------
// The contract WITH z, as a function of the integer sfb and the residual byte (separately rounded binary32 operations):
int epi_contract_z(int t, int z, float s_b, float s_z, float s_d, bool relu) {
    float r = (float)t * s_b;
    const float zf = (float)z * s_z;
    r = r + zf;
    if (relu) r = r <= 0.f ? 0.f : r;
    float v = roundf(r / s_d);
    v = fminf(fmaxf(-128.f, v), 127.f);
    return (int)v;
}

// For every one of the 256 residual values the contract is a non-decreasing step function of sfb, like the contract
// without z, and its steps are those of the others shifted by about z s_z / s_b: one slope c serves all of them and each
// gets an offset of its own, tab[z].  Finds c and the 256 offsets such that epi_linear(t, c, tab[z], lo) ==
// epi_contract_z(t, z) on EVERY int32 t for every z, or reports that it found none.  Per z this is epi_solve_linear's
// argument: the step positions T[k] of the contract by bisection (started from the real-arithmetic position, a handful
// of evaluations each), a candidate accepted only if it has step k at T[k] for every k, evaluated with the device's
// arithmetic.  It fails where s_b / s_d is small (below about 3e-3: an offset then has less room than the literal
// chain's own roundings move the steps).  ~1 ms of host time.
bool epi_solve_table(float s_b, float s_z, float s_d, bool relu, float* c_out, float* tab) {
    const int LIM = 1 << 24;
    const int kmin = relu ? 1 : -127, kmax = 127, NK = kmax - kmin + 1;
    const float c0 = (float)((double)s_b / (double)s_d);
    if (!(c0 > 0.f) || !(c0 < 0x1p20f)) return false;
    std::vector<int> T((size_t)256 * NK);
    for (int zi = 0; zi < 256; ++zi) {
        const int z = zi - 128;
        if (epi_contract_z(LIM, z, s_b, s_z, s_d, relu) < kmax) return false;
        if (epi_contract_z(-LIM, z, s_b, s_z, s_d, relu) >= kmin) return false;
        for (int k = kmin; k <= kmax; ++k) {
            const double g = (((double)k - 0.5) * (double)s_d - (double)z * (double)s_z) / (double)s_b;
            int64_t gi = (int64_t)ceil(g);
            if (gi > LIM - 1) gi = LIM - 1;
            if (gi < -LIM + 1) gi = -LIM + 1;
            int64_t lo, hi, step = 1;  // contract(lo) < k <= contract(hi)
            if (epi_contract_z((int)gi, z, s_b, s_z, s_d, relu) >= k) {
                hi = gi;
                lo = gi - 1;
                while (lo > -LIM && epi_contract_z((int)lo, z, s_b, s_z, s_d, relu) >= k) {
                    hi = lo;
                    lo -= step;
                    step *= 2;
                }
                if (lo < -LIM) lo = -LIM;
            } else {
                lo = gi;
                hi = gi + 1;
                while (hi < LIM && epi_contract_z((int)hi, z, s_b, s_z, s_d, relu) < k) {
                    lo = hi;
                    hi += step;
                    step *= 2;
                }
                if (hi > LIM) hi = LIM;
            }
            while (hi - lo > 1) {
                const int64_t m = lo + (hi - lo) / 2;
                if (epi_contract_z((int)m, z, s_b, s_z, s_d, relu) >= k) hi = m; else lo = m;
            }
            if (hi >= LIM || hi <= -LIM + 1) return false;  // float(t) must be exact around every step
            T[(size_t)zi * NK + (k - kmin)] = (int)hi;
        }
    }
    const float lo_clamp = relu ? 0.f : -128.f;
    for (int u = 0; u <= 8; ++u) {
        for (int sgn = -1; sgn <= 1; sgn += 2) {
            if (u == 0 && sgn == 1) continue;
            float c = c0;
            for (int i = 0; i < u; ++i) c = nextafterf(c, sgn > 0 ? INFINITY : 0.f);
            if (!(c > 0.f)) continue;
            bool all = true;
            for (int zi = 0; zi < 256 && all; ++zi) {
                const int* Tz = &T[(size_t)zi * NK];
                double dlo = -1e300, dhi = 1e300;
                for (int k = kmin; k <= kmax; ++k) {
                    const double a = (double)k - (double)Tz[k - kmin] * (double)c;
                    if (a > dlo) dlo = a;
                    if (a + (double)c < dhi) dhi = a + (double)c;
                }
                bool found = false;
                for (int j = 1; j <= 3 && dlo < dhi && !found; ++j) {
                    const float d = (float)(dlo + (dhi - dlo) * j / 4.0);
                    bool ok = true;
                    for (int k = kmin; k <= kmax && ok; ++k) {
                        const int t = Tz[k - kmin];
                        ok = epi_linear(t, c, d, lo_clamp) >= k && epi_linear(t - 1, c, d, lo_clamp) <= k - 1;
                    }
                    if (ok) {
                        tab[zi] = d;
                        found = true;
                    }
                }
                all = found;
            }
            if (all) {
                *c_out = c;
                return true;
            }
        }
    }
    return false;
}

// One entry per (s_b, s_z, s_d, activation), kept for the life of the process like the other proofs (node-based map:
// the address of an entry never changes, launches copy the table from it).  At most kTableCacheCap entries are stored
// (1 KiB each); beyond that a new triple is reported unsolved and runs the multi-step form.
struct TableKey {
    uint32_t b, z, d, relu;
    bool operator==(const TableKey& o) const { return b == o.b && z == o.z && d == o.d && relu == o.relu; }
};
struct TableKeyHash {
    size_t operator()(const TableKey& k) const {
        uint64_t h = ((uint64_t)k.b << 32 | k.d) * 0x9e3779b97f4a7c15ull;
        h ^= ((uint64_t)k.z << 1 | k.relu) * 0xc2b2ae3d27d4eb4full;
        return (size_t)(h ^ (h >> 29));
    }
};
struct TableEntry {
    bool solved;
    float c;
    float tab[256];  // indexed by the residual byte as an unsigned value
};
constexpr size_t kTableCacheCap = 4096;
std::shared_mutex g_table_mu;
std::unordered_map<TableKey, TableEntry, TableKeyHash> g_table;

const TableEntry* epi_table_cached(float s_b, float s_z, float s_d, bool relu) {
    TableKey key;
    memcpy(&key.b, &s_b, 4);
    memcpy(&key.z, &s_z, 4);
    memcpy(&key.d, &s_d, 4);
    key.relu = relu ? 1u : 0u;
    {
        std::shared_lock<std::shared_mutex> lk(g_table_mu);
        auto it = g_table.find(key);
        if (it != g_table.end()) return &it->second;
        if (g_table.size() >= kTableCacheCap) return nullptr;
    }
    TableEntry e;
    float by_z[256];
    e.c = 0.f;
    e.solved = epi_solve_table(s_b, s_z, s_d, relu, &e.c, by_z);
    for (int u = 0; u < 256; ++u) e.tab[u] = e.solved ? by_z[(int)(int8_t)u + 128] : 0.f;
    std::unique_lock<std::shared_mutex> lk(g_table_mu);
    if (g_table.size() >= kTableCacheCap) return nullptr;
    return &g_table.emplace(key, e).first->second;
}

// All epilogue parameters of one launch.  qs8: the destination is QuantizedS8 (the only dtype with the fast forms).
void epi_fill(EpiParams* e, float s_b, float s_z, float s_d, uint32_t nonline, bool has_z, bool qs8) {
    e->s_b = s_b;
    e->s_z = s_z;
    e->s_d = s_d;
    e->nonline = (int)nonline;
    e->has_z = has_z ? 1 : 0;
    e->fast = qs8 && epi_fast_ok(s_b, s_z, s_d, has_z) && epi_quotient_proved(s_d);
    e->y_hi = 1.0f / s_d;
    e->y_lo = epi_recip_lo(s_d);
    e->lin = 0;
    e->lin_c = e->lin_d = 0.f;
    e->lin_lo = nonline == MI355_NL_RELU ? 0.f : -128.f;
    e->zlin = 0;
    if (e->fast && !has_z && (nonline == MI355_NL_IDENTITY || nonline == MI355_NL_RELU))
        e->lin = epi_linear_cached(s_b, s_d, nonline == MI355_NL_RELU, &e->lin_c, &e->lin_d) ? 1 : 0;
}

// Validation of a descriptor: the checks of ConvolutionBase::deduce_layout_fwd
// (dnn/src/common/convolution.cpp:633-1049) and do_check_exec_common
// (dnn/src/common/conv_bias.cpp:8-133) that survive the translation to a flat descriptor.
int canonize_checked(const mi355_conv_desc* d, ConvProblem* p) {
    const int pi = in_pack(d->format), po = out_pack(d->format);
    if (!pi) return fail(MI355_ERR_UNSUPPORTED, "format %u not supported by this backend", d->format);
    if (d->sparse > MI355_SPARSE_GROUP) return fail(MI355_ERR_BAD_ARG, "invalid convolution sparse type");
    if (d->mode > MI355_MODE_CONVOLUTION) return fail(MI355_ERR_BAD_ARG, "invalid conv mode");
    if (!d->group || !d->fh || !d->fw || !d->stride_h || !d->stride_w || !d->dilate_h || !d->dilate_w)
        return fail(MI355_ERR_BAD_ARG, "zero group/filter/stride/dilation");
    if (d->sparse == MI355_SPARSE_DENSE && d->group != 1)
        return fail(MI355_ERR_SHAPE, "dense convolution with group=%u", d->group);
    if (d->ic % d->group || d->oc % d->group)
        return fail(MI355_ERR_SHAPE, "group conv channel mismatch: ic=%u oc=%u group=%u", d->ic, d->oc, d->group);
    p->d = *d;
    p->icpg = d->ic / d->group;
    p->ocpg = d->oc / d->group;
    p->pin = pi;
    p->pout = po;
    p->dw4 = (d->format == MI355_FMT_NCHW44 || d->format == MI355_FMT_NCHW4) && d->group > 1 && p->icpg == 1 &&
             p->ocpg == 1;
    if (d->format != MI355_FMT_NCHW && (d->dilate_h != 1 || d->dilate_w != 1))
        return fail(MI355_ERR_SHAPE, "NCHWx has invalid dilation %ux%u, require to be 1", d->dilate_h, d->dilate_w);
    if (p->dw4) {
        if (d->group % 4) return fail(MI355_ERR_SHAPE, "channel-wise packed conv needs channels %% 4 == 0");
    } else {
        if (p->icpg % pi)
            return fail(MI355_ERR_SHAPE, "input channels per group (%u) not a multiple of the pack (%d)", p->icpg, pi);
        if (d->format == MI355_FMT_NCHW44 && (p->ocpg % 4))
            return fail(MI355_ERR_SHAPE, "NCHW44 needs output channels per group %% 4 == 0");
    }
    if (d->oc % po) return fail(MI355_ERR_SHAPE, "output channels (%u) not a multiple of the pack (%d)", d->oc, po);
    if (d->nonline == MI355_NL_SIGMOID)
        return fail(MI355_ERR_UNSUPPORTED, "SIGMOID is not defined for quantized ConvBias");
    if (d->nonline > MI355_NL_H_SWISH) return fail(MI355_ERR_BAD_ARG, "invalid nonlineMode %u", d->nonline);
    if (d->bias_mode > MI355_BIAS_FULL) return fail(MI355_ERR_BAD_ARG, "invalid bias mode");
    if (d->dst_dtype > MI355_DT_F32) return fail(MI355_ERR_BAD_ARG, "invalid dst dtype");
    if (d->dst_dtype == MI355_DT_F32 && d->format != MI355_FMT_NCHW4_NCHW)
        return fail(MI355_ERR_UNSUPPORTED, "a Float32 dst needs format NCHW4_NCHW");
    if (d->has_z && (d->format == MI355_FMT_NCHW4_NCHW32 || d->format == MI355_FMT_NCHW32_NCHW4))
        return fail(MI355_ERR_SHAPE, "z is not allowed for NCHW4_NCHW32 / NCHW32_NCHW4");
    // 64-bit: huge paddings or dilations must not wrap past the test
    const uint64_t dfh = (uint64_t)(d->fh - 1) * d->dilate_h + 1, dfw = (uint64_t)(d->fw - 1) * d->dilate_w + 1;
    const uint64_t pih = (uint64_t)d->ih + 2ull * d->pad_h, piw = (uint64_t)d->iw + 2ull * d->pad_w;
    if (pih < dfh || piw < dfw)
        return fail(MI355_ERR_SHAPE, "filter %llux%llu larger than padded input %llux%llu", (unsigned long long)dfh,
                    (unsigned long long)dfw, (unsigned long long)pih, (unsigned long long)piw);
    if (dfh > 0x7fffffffull || dfw > 0x7fffffffull || pih > 0x7fffffffull || piw > 0x7fffffffull)
        return fail(MI355_ERR_SHAPE, "convolution geometry out of range");
    p->oh = conv_out_size(d->ih, d->fh, d->dilate_h, d->stride_h, d->pad_h);
    p->ow = conv_out_size(d->iw, d->fw, d->dilate_w, d->stride_w, d->pad_w);
    const int64_t src_img = (int64_t)d->ic * d->ih * d->iw, dst_img = (int64_t)d->oc * p->oh * p->ow;
    p->src_sn = d->src_stride_n ? d->src_stride_n : src_img;
    p->dst_sn = d->dst_stride_n ? d->dst_stride_n : dst_img;
    p->z_sn = d->z_stride_n ? d->z_stride_n : dst_img;
    if (p->src_sn < src_img || p->dst_sn < dst_img || p->z_sn < dst_img)
        return fail(MI355_ERR_SHAPE, "batch stride smaller than one image");
    // Float32 dst: scale_bias / scale_z carry the scales of src and filter; one factor dequantises the exact sum
    epi_fill(&p->epi, d->scale_bias, d->scale_z, d->scale_dst, d->nonline, d->has_z != 0, d->dst_dtype == MI355_DT_QS8);
    if (d->dst_dtype == MI355_DT_F32) p->epi.s_b = d->scale_bias * d->scale_z;
    return MI355_OK;
}

// An operator call canonizes the same descriptor several times in a row (get_workspace_in_bytes, the algorithm
// choice, exec): each thread remembers the last descriptor that passed and its canonical form.  Equal bytes mean an
// equal descriptor; different padding bytes only cost the full path.
int canonize(const mi355_conv_desc* d, ConvProblem* p) {
    if (!d) return fail(MI355_ERR_BAD_ARG, "null descriptor");
    thread_local bool have = false;
    thread_local ConvProblem last;
    if (have && memcmp(d, &last.d, sizeof(*d)) == 0) {
        *p = last;
        return MI355_OK;
    }
    const int st = canonize_checked(d, p);
    if (st == MI355_OK) {
        last = *p;
        memcpy(&last.d, d, sizeof(*d));  // padding bytes included, so that the comparison above can hit
        have = true;
    }
    return st;
}

struct DevInfo {
    bool ok = false;
    int cu = 0;
};
DevInfo g_dev[64];
std::mutex g_dev_mu;

int cu_count() {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 0;
    std::lock_guard<std::mutex> lk(g_dev_mu);
    if (!g_dev[dev].ok) {
        hipDeviceProp_t pr;
        if (hipGetDeviceProperties(&pr, dev) != hipSuccess) return 0;
        g_dev[dev].cu = pr.multiProcessorCount;
        g_dev[dev].ok = true;
    }
    return g_dev[dev].cu;
}

const char* kAlgoNames[ALGO_COUNT] = {"MI355_DIRECT_DOT4", "MI355_IGEMM_MFMA_I8", "MI355_DEPTHWISE_DOT4",
                                      "MI355_C4_MFMA_I8", "MI355_NCHW_RELAYOUT_MFMA_I8"};

bool algo_usable(const ConvProblem& p, int id) {
    switch (id) {
        case ALGO_DIRECT: return true;
        case ALGO_IGEMM_MFMA: return igemm_usable(p);
        case ALGO_DEPTHWISE: return depthwise_usable(p);
        case ALGO_C4_MFMA: return c4_usable(p);
        case ALGO_NCHW_MFMA: return nchw_mfma_usable(p);
        default: return false;
    }
}

// Heuristic order (cf. the reference's per-backend get_algorithm_heuristic, e.g.
// dnn/src/cuda/conv_bias/opr_impl.cpp:44-238): channel-wise kernel, the 4-channel first-layer kernel,
// then the MFMA implicit GEMM, then the generic direct kernel.  Plain NCHW takes the relayout + MFMA algorithm once
// the problem is large enough to pay for its five extra launches (the generic kernel runs ~4 M multiply-adds in the time
// those take); workspace_limit is get_algorithm_heuristic's (dnn/include/megdnn/oprs/base.h:595-614).
int pick_algo(const ConvProblem& p, size_t workspace_limit = SIZE_MAX) {
    if (depthwise_usable(p)) return ALGO_DEPTHWISE;
    if (c4_usable(p)) return ALGO_C4_MFMA;
    if (igemm_usable(p)) return ALGO_IGEMM_MFMA;
    if (p.d.format == MI355_FMT_NCHW) {
        const uint64_t macs = (uint64_t)p.d.n * p.d.oc * p.oh * p.ow * p.icpg * p.d.fh * p.d.fw;
        if (macs >= (1ull << 22) && nchw_mfma_usable(p) && nchw_mfma_workspace(p) <= workspace_limit) return ALGO_NCHW_MFMA;
    }
    return ALGO_DIRECT;
}

size_t algo_workspace(const ConvProblem& p, int id) { return id == ALGO_NCHW_MFMA ? nchw_mfma_workspace(p) : 0; }

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

}  // namespace

namespace mi355 {
bool epi_residual_table(const EpiParams& e, float* c, const float** tab) {
    if (!e.fast || !e.has_z || (e.nonline != MI355_NL_IDENTITY && e.nonline != MI355_NL_RELU)) return false;
    const TableEntry* t = epi_table_cached(e.s_b, e.s_z, e.s_d, e.nonline == MI355_NL_RELU);
    if (!t || !t->solved) return false;
    *c = t->c;
    *tab = t->tab;
    return true;
}
}  // namespace mi355

extern "C" {

int mi355_abi_version(void) { return MI355_CONVBIAS_ABI_VERSION; }

const char* mi355_status_string(int status) {
    switch (status) {
        case MI355_OK: return "ok";
        case MI355_ERR_BAD_ARG: return "bad argument";
        case MI355_ERR_UNSUPPORTED: return "unsupported by the MI355 backend";
        case MI355_ERR_SHAPE: return "inconsistent shapes";
        case MI355_ERR_WORKSPACE: return "workspace too small";
        case MI355_ERR_LAUNCH: return "HIP launch/runtime error";
        case MI355_ERR_NO_DEVICE: return "no usable device";
        case MI355_ERR_ALGO: return "algorithm not usable for this problem";
        default: return "unknown status";
    }
}

const char* mi355_last_error(void) { return g_err; }

int mi355_get_device_info(int device, mi355_device_info* out) {
    if (!out) return fail(MI355_ERR_BAD_ARG, "null out");
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess || device < 0 || device >= n) {
        (void)hipGetLastError();
        return fail(MI355_ERR_NO_DEVICE, "device %d not available", device);
    }
    hipDeviceProp_t pr;
    hipError_t e = hipGetDeviceProperties(&pr, device);
    if (e != hipSuccess) return fail(MI355_ERR_NO_DEVICE, "%s", hipGetErrorString(e));
    memset(out, 0, sizeof(*out));
    out->device = device;
    out->compute_units = pr.multiProcessorCount;
    out->clock_khz = pr.clockRate;
    out->lds_bytes_per_cu = (int32_t)pr.maxSharedMemoryPerMultiProcessor;
    out->hbm_bytes = (int64_t)pr.totalGlobalMem;
    snprintf(out->arch, sizeof(out->arch), "%s", pr.gcnArchName);
    snprintf(out->name, sizeof(out->name), "%s", pr.name);
    return MI355_OK;
}

int mi355_convbias_deduce_out(const mi355_conv_desc* d, uint32_t* oh, uint32_t* ow) {
    ConvProblem p;
    int st = canonize(d, &p);
    if (st) return st;
    if (oh) *oh = p.oh;
    if (ow) *ow = p.ow;
    return MI355_OK;
}

int mi355_convbias_algo_count(void) { return ALGO_COUNT; }

const char* mi355_convbias_algo_name(int id) { return id >= 0 && id < ALGO_COUNT ? kAlgoNames[id] : NULL; }

int mi355_convbias_algo_usable(const mi355_conv_desc* d, int id) {
    ConvProblem p;
    int st = canonize(d, &p);
    if (st) return st;
    if (id < 0 || id >= ALGO_COUNT) return fail(MI355_ERR_ALGO, "unknown algorithm id %d", id);
    return algo_usable(p, id) ? MI355_OK : fail(MI355_ERR_ALGO, "%s cannot run this problem", kAlgoNames[id]);
}

int mi355_convbias_s8_query(const mi355_conv_desc* d, int algo_request, mi355_algo* algo_out,
                            size_t* workspace_bytes) {
    ConvProblem p;
    int st = canonize(d, &p);
    if (st) return st;
    int id = algo_request;
    const bool pre = algo_request == MI355_ALGO_HEURISTIC_PREPROCESS;
    if (id == MI355_ALGO_HEURISTIC || pre) {
        id = pick_algo(p);
    } else if (id < 0 || id >= ALGO_COUNT) {
        return fail(MI355_ERR_ALGO, "unknown algorithm id %d", id);
    } else if (!algo_usable(p, id)) {
        return fail(MI355_ERR_ALGO, "%s cannot run this problem", kAlgoNames[id]);
    }
    if (algo_out) {
        algo_out->id = id;
        algo_out->tile_cfg = id == ALGO_IGEMM_MFMA ? igemm_pick_cfg(p, cu_count(), pre) : 0;
        // an algorithm the heuristic chose may be replaced by the generic kernel at exec time (misaligned tensors);
        // one the caller asked for by id may not
        algo_out->reserved = algo_request == MI355_ALGO_HEURISTIC || pre ? MI355_ALGO_FLAG_HEURISTIC : 0;
    }
    // the packed-format kernels read the reference layouts in place (no filter repack, no float staging): 0 bytes;
    // the plain-NCHW algorithm keeps its packed intermediates in the workspace
    if (workspace_bytes) *workspace_bytes = algo_workspace(p, id);
    return MI355_OK;
}

// filter: the reference layout, or (preprocessed) the artefact of mi355_convbias_s8_preprocess for this algorithm
static int exec_impl(void* stream, const mi355_conv_desc* d, const mi355_algo* algo, const int8_t* src, const int8_t* filter,
                     bool preprocessed, const int32_t* bias, const int8_t* z, void* dst, void* workspace, size_t workspace_bytes) {
    ConvProblem p;
    int st = canonize(d, &p);
    if (st) return st;
    if (!src || !filter || !dst) return fail(MI355_ERR_BAD_ARG, "null tensor pointer");
    if (d->bias_mode != MI355_BIAS_NONE && !bias) return fail(MI355_ERR_BAD_ARG, "bias_mode set but bias is null");
    if (d->has_z && !z) return fail(MI355_ERR_BAD_ARG, "has_z set but z is null");
    int id = algo ? algo->id : MI355_ALGO_HEURISTIC;
    int cfg = algo ? algo->tile_cfg : -1;
    if (id == MI355_ALGO_HEURISTIC) {
        id = pick_algo(p, workspace ? workspace_bytes : 0);  // whatever fits the workspace the caller brought
        cfg = -1;
    }
    if (id < 0 || id >= ALGO_COUNT) return fail(MI355_ERR_ALGO, "unknown algorithm id %d", id);
    if (!algo_usable(p, id)) return fail(MI355_ERR_ALGO, "%s cannot run this problem", kAlgoNames[id]);
    // check_exec's workspace rule (dnn/src/common/conv_bias.cpp:32-37)
    const size_t ws_need = algo_workspace(p, id);
    if (ws_need) {
        if (!workspace || workspace_bytes < ws_need)
            return fail(MI355_ERR_WORKSPACE, "workspace of %zu bytes, %s needs %zu", workspace ? workspace_bytes : (size_t)0,
                        kAlgoNames[id], ws_need);
        if (!aligned16(workspace)) return fail(MI355_ERR_BAD_ARG, "the workspace needs 16-byte alignment");
    }
    const bool by_heuristic = !algo || algo->id == MI355_ALGO_HEURISTIC || (algo->reserved & MI355_ALGO_FLAG_HEURISTIC);
    if (id == ALGO_IGEMM_MFMA) {
        if (cfg < 0 || cfg >= igemm_num_cfgs()) {
            cfg = igemm_pick_cfg(p, cu_count());
        } else {
            // the tile that runs is the tile that was named: a tile the caller forced and that cannot run this problem is an
            // error (a fast-run chooser must not time one kernel under two names); a choice of the heuristic is replaced
            const int runs = igemm_resolve_cfg(p, cfg);
            if (runs != cfg && !by_heuristic)
                return fail(MI355_ERR_ALGO, "tile %s cannot run this problem (%s would)", igemm_cfg_name(cfg),
                            runs >= 0 ? igemm_cfg_name(runs) : "none");
            cfg = runs;
        }
    }
    if (preprocessed && (id != ALGO_IGEMM_MFMA || igemm_preprocessed_bytes(p, cfg) == 0))
        return fail(MI355_ERR_ALGO, "this algorithm has no pre-processed filter form");
    // the tiled kernels use 16-byte vector accesses; misaligned tensors take the generic kernel
    if (id != ALGO_DIRECT && id != ALGO_NCHW_MFMA) {  // (the relayouts of plain NCHW tensors take any pointer)
        // (pack-32 tensors move as 16-byte vectors, pack-4 tensors as dwords)
        // (a planar destination is written element by element: dst, z and a Float32 bias need their natural alignment only)
        const int sa = p.pin == 32 ? 16 : 4, da = p.pout == 32 ? 16 : p.pout == 1 ? 1 : 4;
        const bool planar = p.pout == 1 && id == ALGO_IGEMM_MFMA;
        const uintptr_t el = d->dst_dtype == MI355_DT_F32 ? 3 : 0;
        auto natural = [el](const void* q) { return (reinterpret_cast<uintptr_t>(q) & el) == 0; };
        bool al = aligned16(src) && aligned16(filter) && (planar ? natural(dst) : aligned16(dst)) &&
                  (!bias || (planar ? (reinterpret_cast<uintptr_t>(bias) & 3) == 0 : aligned16(bias))) &&
                  (!z || (planar ? natural(z) : aligned16(z))) && p.src_sn % sa == 0 && p.dst_sn % da == 0 && p.z_sn % da == 0;
        if (!al) {
            // the generic kernel reads the reference filter layout only
            if (preprocessed || !by_heuristic)
                return fail(MI355_ERR_ALGO, "%s needs 16-byte aligned tensors", kAlgoNames[id]);
            id = ALGO_DIRECT;
        }
    }
    hipStream_t hs = reinterpret_cast<hipStream_t>(stream);
    int rc = 0;
    switch (id) {
        case ALGO_DIRECT:
            rc = launch_conv_direct(hs, p, src, filter, bias, z, dst);
            break;
        case ALGO_IGEMM_MFMA:
            rc = launch_conv_igemm(hs, p, cfg, cu_count(), src, filter, bias, z, reinterpret_cast<int8_t*>(dst), preprocessed);
            break;
        case ALGO_DEPTHWISE:
            rc = launch_conv_depthwise(hs, p, src, filter, bias, z, reinterpret_cast<int8_t*>(dst));
            break;
        case ALGO_C4_MFMA:
            rc = launch_conv_c4(hs, p, cu_count(), src, filter, bias, z, reinterpret_cast<int8_t*>(dst));
            break;
        case ALGO_NCHW_MFMA:
            rc = launch_conv_nchw_mfma(hs, p, cu_count(), src, filter, bias, z, reinterpret_cast<int8_t*>(dst), workspace);
            break;
    }
    if (rc) return fail(MI355_ERR_LAUNCH, "%s: %s", kAlgoNames[id], hipGetErrorString((hipError_t)rc));
    return MI355_OK;
}

int mi355_convbias_s8_exec(void* stream, const mi355_conv_desc* d, const mi355_algo* algo, const int8_t* src,
                           const int8_t* filter, const int32_t* bias, const int8_t* z, void* dst, void* workspace,
                           size_t workspace_bytes) {
    return exec_impl(stream, d, algo, src, filter, false, bias, z, dst, workspace, workspace_bytes);
}

// ---- exec for callers that cannot allocate: the workspace is an array of the library's own --------------------------
// One array per GPU, alive from the moment the code object is loaded on that GPU until the process ends.  In host code
// the array's name is a stand-in, not a device address: its address on the CURRENT device comes from
// hipGetSymbolAddress, once per device, and only that pointer is ever handed to a kernel.
constexpr size_t kStaticWorkspaceBytes = (size_t)MI355_STATIC_WORKSPACE_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticWorkspaceBytes];

namespace {
void* g_scratch_ptr[64];  // per device, under g_dev_mu
int static_workspace(void** out) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) {
        (void)hipGetLastError();
        return fail(MI355_ERR_NO_DEVICE, "no current device");
    }
    std::lock_guard<std::mutex> lk(g_dev_mu);
    if (!g_scratch_ptr[dev]) {
        void* p = nullptr;
        const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) {
            (void)hipGetLastError();
            return fail(MI355_ERR_LAUNCH, "address of the static workspace on device %d: %s", dev, hipGetErrorString(e));
        }
        g_scratch_ptr[dev] = p;
    }
    *out = g_scratch_ptr[dev];
    return MI355_OK;
}
}  // namespace

size_t mi355_static_workspace_bytes(void) { return kStaticWorkspaceBytes; }

int mi355_convbias_s8_exec_static_workspace(void* stream, const mi355_conv_desc* d, const mi355_algo* algo, const int8_t* src,
                                            const int8_t* filter, const int32_t* bias, const int8_t* z, void* dst) {
    // sizes first: a problem beyond the array is refused before anything touches the device
    ConvProblem p;
    int st = canonize(d, &p);
    if (st) return st;
    if (algo && algo->id != MI355_ALGO_HEURISTIC) {
        if (algo->id < 0 || algo->id >= ALGO_COUNT) return fail(MI355_ERR_ALGO, "unknown algorithm id %d", algo->id);
        const size_t need = algo_usable(p, algo->id) ? algo_workspace(p, algo->id) : 0;
        if (need > kStaticWorkspaceBytes)
            return fail(MI355_ERR_WORKSPACE, "%s needs a workspace of %zu bytes, the static workspace holds %zu", kAlgoNames[algo->id],
                        need, kStaticWorkspaceBytes);
    }
    void* ws = nullptr;
    st = static_workspace(&ws);
    if (st) return st;
    // no algorithm given: the heuristic stays within the array (exec_impl passes the size on as its workspace limit)
    return exec_impl(stream, d, algo, src, filter, false, bias, z, dst, ws, kStaticWorkspaceBytes);
}

// ---- weight pre-processing ----
static int preprocess_problem(const mi355_conv_desc* d, const mi355_algo* algo, ConvProblem* p, size_t* bytes) {
    int st = canonize(d, p);
    if (st) return st;
    if (!algo) return fail(MI355_ERR_BAD_ARG, "pre-processing belongs to one algorithm: pass the result of query()");
    *bytes = 0;
    if (algo->id == ALGO_IGEMM_MFMA && igemm_usable(*p)) {
        int cfg = algo->tile_cfg;
        if (cfg < 0 || cfg >= igemm_num_cfgs()) cfg = igemm_pick_cfg(*p, cu_count());
        *bytes = igemm_preprocessed_bytes(*p, cfg);
    }
    return MI355_OK;
}

int mi355_convbias_s8_preprocess_size(const mi355_conv_desc* d, const mi355_algo* algo, size_t* bytes) {
    if (!bytes) return fail(MI355_ERR_BAD_ARG, "null argument");
    ConvProblem p;
    return preprocess_problem(d, algo, &p, bytes);
}

int mi355_convbias_s8_preprocess(void* stream, const mi355_conv_desc* d, const mi355_algo* algo, const int8_t* filter,
                                 void* preprocessed, size_t preprocessed_bytes) {
    ConvProblem p;
    size_t need = 0;
    int st = preprocess_problem(d, algo, &p, &need);
    if (st) return st;
    if (need == 0) return MI355_OK;  // nothing to hoist for this algorithm (the reference's naive form)
    if (!filter || !preprocessed) return fail(MI355_ERR_BAD_ARG, "null tensor pointer");
    if (preprocessed_bytes < need)
        return fail(MI355_ERR_WORKSPACE, "pre-processed filter of %zu bytes, %zu needed", preprocessed_bytes, need);
    if (!aligned16(filter) || !aligned16(preprocessed)) return fail(MI355_ERR_BAD_ARG, "filter tensors need 16-byte alignment");
    int rc = launch_igemm_preprocess(reinterpret_cast<hipStream_t>(stream), p, filter, reinterpret_cast<int8_t*>(preprocessed));
    if (rc) return fail(MI355_ERR_LAUNCH, "preprocess: %s", hipGetErrorString((hipError_t)rc));
    return MI355_OK;
}

int mi355_convbias_s8_exec_preprocessed(void* stream, const mi355_conv_desc* d, const mi355_algo* algo, const int8_t* src,
                                        const void* preprocessed, size_t preprocessed_bytes, const int32_t* bias,
                                        const int8_t* z, void* dst, void* workspace, size_t workspace_bytes) {
    ConvProblem p;
    size_t need = 0;
    int st = preprocess_problem(d, algo, &p, &need);
    if (st) return st;
    if (need == 0) return fail(MI355_ERR_ALGO, "this algorithm has no pre-processed filter form");
    if (preprocessed_bytes < need)
        return fail(MI355_ERR_WORKSPACE, "pre-processed filter of %zu bytes, %zu needed", preprocessed_bytes, need);
    return exec_impl(stream, d, algo, src, reinterpret_cast<const int8_t*>(preprocessed), true, bias, z, dst, workspace,
                     workspace_bytes);
}

int mi355_convbias_s8_profile(void* stream, const mi355_conv_desc* d, const mi355_algo* algo, const int8_t* src,
                              const int8_t* filter, const int32_t* bias, const int8_t* z, void* dst, void* workspace,
                              size_t workspace_bytes, int warmup, int iters, float* avg_usec) {
    if (!avg_usec || iters <= 0 || warmup < 0) return fail(MI355_ERR_BAD_ARG, "profile: bad iteration counts or null result");
    hipStream_t hs = reinterpret_cast<hipStream_t>(stream);
    for (int i = 0; i < warmup; ++i) {
        int st = mi355_convbias_s8_exec(stream, d, algo, src, filter, bias, z, dst, workspace, workspace_bytes);
        if (st) return st;
    }
    hipEvent_t e0, e1;
    if (hipEventCreate(&e0) != hipSuccess) return fail(MI355_ERR_LAUNCH, "profile: cannot create an event");
    if (hipEventCreate(&e1) != hipSuccess) {
        (void)hipEventDestroy(e0);
        return fail(MI355_ERR_LAUNCH, "profile: cannot create an event");
    }
    int st = MI355_OK;
    hipError_t he = hipEventRecord(e0, hs);
    for (int i = 0; i < iters && st == MI355_OK && he == hipSuccess; ++i)
        st = mi355_convbias_s8_exec(stream, d, algo, src, filter, bias, z, dst, workspace, workspace_bytes);
    if (he == hipSuccess) he = hipEventRecord(e1, hs);
    if (he == hipSuccess) he = hipEventSynchronize(e1);
    float ms = 0.f;
    if (he == hipSuccess) he = hipEventElapsedTime(&ms, e0, e1);
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    if (st) return st;
    if (he != hipSuccess) return fail(MI355_ERR_LAUNCH, "profile: %s", hipGetErrorString(he));
    *avg_usec = ms * 1000.f / (float)iters;
    return MI355_OK;
}

int mi355_stream_probe(void* stream, const void* src, uint64_t read_bytes, void* dst, uint64_t write_bytes) {
    if ((read_bytes && !src) || (write_bytes && !dst)) return fail(MI355_ERR_BAD_ARG, "null buffer");
    if ((read_bytes | write_bytes) & 15) return fail(MI355_ERR_BAD_ARG, "byte counts must be multiples of 16");
    // loads whose values reach no store may be dropped by the compiler: a read-only probe would move nothing
    if (read_bytes && !write_bytes) return fail(MI355_ERR_BAD_ARG, "a probe that reads must write at least 16 bytes");
    if (!aligned16(src) || !aligned16(dst)) return fail(MI355_ERR_BAD_ARG, "buffers need 16-byte alignment");
    hipError_t e = (hipError_t)launch_stream_probe(reinterpret_cast<hipStream_t>(stream), src, read_bytes, dst, write_bytes, cu_count());
    if (e != hipSuccess) return fail(MI355_ERR_LAUNCH, "stream probe: %s", hipGetErrorString(e));
    return MI355_OK;
}

int mi355_requant_s32_s8_exec(void* stream, const mi355_requant_desc* d, const int32_t* src, const int8_t* z, int8_t* dst) {
    if (!d) return fail(MI355_ERR_BAD_ARG, "null descriptor");
    if (d->nonline == MI355_NL_SIGMOID || d->nonline > MI355_NL_H_SWISH)
        return fail(MI355_ERR_UNSUPPORTED, "nonlinearity %u has no quantized definition", d->nonline);
    if (d->count == 0) return MI355_OK;
    if (!src || !dst) return fail(MI355_ERR_BAD_ARG, "null tensor pointer");
    if (d->has_z && !z) return fail(MI355_ERR_BAD_ARG, "has_z set but z is null");
    if (!aligned16(src) || (reinterpret_cast<uintptr_t>(dst) & 3) || (d->has_z && (reinterpret_cast<uintptr_t>(z) & 3)))
        return fail(MI355_ERR_BAD_ARG, "src needs 16-byte, z and dst 4-byte alignment");
    EpiParams e;
    epi_fill(&e, d->scale_src, d->scale_z, d->scale_dst, d->nonline, d->has_z != 0, true);
    int rc = launch_requant(reinterpret_cast<hipStream_t>(stream), e, src, z, dst, d->count, cu_count());
    if (rc) return fail(MI355_ERR_LAUNCH, "requant: %s", hipGetErrorString((hipError_t)rc));
    return MI355_OK;
}

int mi355_requant_s8_s8_exec(void* stream, const mi355_requant_desc* d, const int8_t* src, const int8_t* z, int8_t* dst) {
    if (!d) return fail(MI355_ERR_BAD_ARG, "null descriptor");
    if (d->nonline == MI355_NL_SIGMOID || d->nonline > MI355_NL_H_SWISH)
        return fail(MI355_ERR_UNSUPPORTED, "nonlinearity %u has no quantized definition", d->nonline);
    if (d->count == 0) return MI355_OK;
    if (!src || !dst) return fail(MI355_ERR_BAD_ARG, "null tensor pointer");
    if (d->has_z && !z) return fail(MI355_ERR_BAD_ARG, "has_z set but z is null");
    if (!aligned16(src) || !aligned16(dst) || (d->has_z && !aligned16(z)))
        return fail(MI355_ERR_BAD_ARG, "src, z and dst need 16-byte alignment");
    EpiParams e;
    epi_fill(&e, d->scale_src, d->scale_z, d->scale_dst, d->nonline, d->has_z != 0, true);
    int rc = launch_requant8(reinterpret_cast<hipStream_t>(stream), e, src, z, dst, d->count, cu_count());
    if (rc) return fail(MI355_ERR_LAUNCH, "requant: %s", hipGetErrorString((hipError_t)rc));
    return MI355_OK;
}

int mi355_elemwise_q_exec(void* stream, const mi355_elemwise_desc* d, const void* src0, const void* src1, const void* src2,
                          void* dst) {
    if (!d) return fail(MI355_ERR_BAD_ARG, "null descriptor");
    const int arity = elemwise_q_arity(d->mode);
    if (arity == 0)
        return fail(MI355_ERR_UNSUPPORTED, "elemwise mode %u is not served (no such mode, or its float kernel calls the C math library)",
                    d->mode);
    if ((int)d->arity != arity) return fail(MI355_ERR_BAD_ARG, "elemwise mode %u takes %d inputs, descriptor says %u", d->mode, arity, d->arity);
    if ((d->src_dtype != MI355_DT_QS8 && d->src_dtype != MI355_DT_QS32) || (d->dst_dtype != MI355_DT_QS8 && d->dst_dtype != MI355_DT_QS32))
        return fail(MI355_ERR_UNSUPPORTED, "quantized elemwise takes QuantizedS8 or QuantizedS32 tensors");
    if (d->count == 0) return MI355_OK;
    const void* srcs[3] = {src0, src1, src2};
    const uintptr_t src_mask = d->src_dtype == MI355_DT_QS32 ? 15 : 3, dst_mask = d->dst_dtype == MI355_DT_QS32 ? 15 : 3;
    for (int i = 0; i < arity; ++i) {
        if (!srcs[i]) return fail(MI355_ERR_BAD_ARG, "input %d is null", i);
        if (reinterpret_cast<uintptr_t>(srcs[i]) & src_mask) return fail(MI355_ERR_BAD_ARG, "input %d is misaligned", i);
    }
    if (!dst) return fail(MI355_ERR_BAD_ARG, "null tensor pointer");
    if (reinterpret_cast<uintptr_t>(dst) & dst_mask) return fail(MI355_ERR_BAD_ARG, "dst is misaligned");
    int rc = launch_elemwise_q(reinterpret_cast<hipStream_t>(stream), *d, src0, src1, src2, dst, cu_count());
    if (rc) return fail(MI355_ERR_LAUNCH, "elemwise: %s", hipGetErrorString((hipError_t)rc));
    return MI355_OK;
}

int mi355_typecvt_f32_s8_exec(void* stream, uint64_t count, float scale_dst, const float* src, int8_t* dst) {
    if (count == 0) return MI355_OK;
    if (!src || !dst) return fail(MI355_ERR_BAD_ARG, "null tensor pointer");
    if (!aligned16(src) || ((uintptr_t)dst & 3)) return fail(MI355_ERR_BAD_ARG, "src needs 16-byte, dst 4-byte alignment");
    int rc = launch_cvt_f32_s8(reinterpret_cast<hipStream_t>(stream), scale_dst, src, dst, count, cu_count());
    if (rc) return fail(MI355_ERR_LAUNCH, "typecvt: %s", hipGetErrorString((hipError_t)rc));
    return MI355_OK;
}

int mi355_typecvt_s8_f32_exec(void* stream, uint64_t count, float scale_src, const int8_t* src, float* dst) {
    if (count == 0) return MI355_OK;
    if (!src || !dst) return fail(MI355_ERR_BAD_ARG, "null tensor pointer");
    if (((uintptr_t)src & 3) || !aligned16(dst)) return fail(MI355_ERR_BAD_ARG, "src needs 4-byte, dst 16-byte alignment");
    int rc = launch_cvt_s8_f32(reinterpret_cast<hipStream_t>(stream), scale_src, src, dst, count, cu_count());
    if (rc) return fail(MI355_ERR_LAUNCH, "typecvt: %s", hipGetErrorString((hipError_t)rc));
    return MI355_OK;
}

// ---- Pooling ----
static int pooling_check(const mi355_pooling_desc* d, int* pack, uint32_t* oh, uint32_t* ow) {
    if (!d) return fail(MI355_ERR_BAD_ARG, "null descriptor");
    if (d->mode > MI355_POOL_AVERAGE_COUNT_EXCLUDE_PADDING) return fail(MI355_ERR_UNSUPPORTED, "pooling mode %u", d->mode);
    switch (d->format) {
        case MI355_FMT_NCHW: *pack = 1; break;
        case MI355_FMT_NCHW4:
        case MI355_FMT_NCHW44: *pack = 4; break;
        case MI355_FMT_NCHW32: *pack = 32; break;
        default: return fail(MI355_ERR_UNSUPPORTED, "invalid pooling format %u", d->format);
    }
    if (d->c % (uint32_t)*pack) return fail(MI355_ERR_SHAPE, "channels %u not a multiple of %d", d->c, *pack);
    if (!d->window_h || !d->window_w || !d->stride_h || !d->stride_w) return fail(MI355_ERR_SHAPE, "zero window or stride");
    if ((uint64_t)d->ih + 2ull * d->pad_h < d->window_h || (uint64_t)d->iw + 2ull * d->pad_w < d->window_w)
        return fail(MI355_ERR_SHAPE, "window %ux%u larger than the padded input %ux%u", d->window_h, d->window_w,
                    d->ih + 2 * d->pad_h, d->iw + 2 * d->pad_w);
    if (d->ih > (1u << 24) || d->iw > (1u << 24) || d->pad_h > (1u << 24) || d->pad_w > (1u << 24) ||
        (uint64_t)d->window_h * d->window_w > 65535)
        return fail(MI355_ERR_SHAPE, "pooling geometry out of range");
    *oh = (d->ih + 2 * d->pad_h - d->window_h) / d->stride_h + 1;
    *ow = (d->iw + 2 * d->pad_w - d->window_w) / d->stride_w + 1;
    return MI355_OK;
}

int mi355_pooling_deduce_out(const mi355_pooling_desc* d, uint32_t* oh, uint32_t* ow) {
    if (!oh || !ow) return fail(MI355_ERR_BAD_ARG, "null argument");
    int pack;
    return pooling_check(d, &pack, oh, ow);
}

int mi355_pooling_s8_exec(void* stream, const mi355_pooling_desc* d, const int8_t* src, int8_t* dst) {
    int pack;
    uint32_t oh, ow;
    int rc = pooling_check(d, &pack, &oh, &ow);
    if (rc) return rc;
    const uint64_t out_elems = (uint64_t)d->n * d->c * oh * ow;
    if (out_elems == 0) return MI355_OK;
    if ((uint64_t)d->n * d->c * d->ih * d->iw == 0) return fail(MI355_ERR_SHAPE, "empty input with a non-empty output");
    if (out_elems / (pack == 32 ? 16 : pack) >= (1ull << 31)) return fail(MI355_ERR_SHAPE, "pooling output too large");
    if (!src || !dst) return fail(MI355_ERR_BAD_ARG, "null tensor pointer");
    const uintptr_t al = pack == 32 ? 15 : pack == 4 ? 3 : 0;
    if (((uintptr_t)src & al) || ((uintptr_t)dst & al)) return fail(MI355_ERR_BAD_ARG, "src and dst need %d-byte alignment", (int)al + 1);
    if (d->mode != MI355_POOL_AVERAGE) {
        // the last window along an axis starts at (o - 1) * stride - pad; the first ends at window - pad
        const bool out_h = d->pad_h >= d->window_h || (uint64_t)(oh - 1) * d->stride_h >= (uint64_t)d->ih + d->pad_h;
        const bool out_w = d->pad_w >= d->window_w || (uint64_t)(ow - 1) * d->stride_w >= (uint64_t)d->iw + d->pad_w;
        if (out_h || out_w) return fail(MI355_ERR_SHAPE, "The pooling window lies outside completely");
    }
    rc = launch_pooling(reinterpret_cast<hipStream_t>(stream), *d, pack, oh, ow, src, dst, cu_count());
    if (rc) return fail(MI355_ERR_LAUNCH, "pooling: %s", hipGetErrorString((hipError_t)rc));
    return MI355_OK;
}

int mi355_igemm_tile_count(void) { return igemm_num_cfgs(); }
const char* mi355_igemm_tile_name(int cfg) { return igemm_cfg_name(cfg); }

int mi355_igemm_tile_usable(const mi355_conv_desc* d, int tile_cfg) {
    ConvProblem p;
    int st = canonize(d, &p);
    if (st) return st;
    if (!igemm_usable(p)) return fail(MI355_ERR_ALGO, "%s cannot run this problem", kAlgoNames[ALGO_IGEMM_MFMA]);
    if (tile_cfg < 0 || tile_cfg >= igemm_num_cfgs()) return fail(MI355_ERR_ALGO, "unknown tile configuration %d", tile_cfg);
    const int runs = igemm_resolve_cfg(p, tile_cfg);
    if (runs != tile_cfg)
        return fail(MI355_ERR_ALGO, "tile %s cannot run this problem (%s would)", igemm_cfg_name(tile_cfg),
                    runs >= 0 ? igemm_cfg_name(runs) : "none");
    return MI355_OK;
}

int mi355_epilogue_quotient_form(float scale_dst, float* y_hi, float* y_lo) {
    if (!y_hi || !y_lo) return -fail(MI355_ERR_BAD_ARG, "null argument");
    *y_hi = 1.0f / scale_dst;
    *y_lo = epi_recip_lo(scale_dst);
    if (!epi_fast_ok(1.f, 1.f, scale_dst, false)) return 0;
    return epi_quotient_proved(scale_dst) ? 1 : 0;
}

int mi355_epilogue_linear_form(float scale_bias, float scale_dst, uint32_t nonline, float* c, float* d) {
    if (!c || !d) return -fail(MI355_ERR_BAD_ARG, "null argument");
    if (nonline != MI355_NL_IDENTITY && nonline != MI355_NL_RELU)
        return -fail(MI355_ERR_BAD_ARG, "the linear form exists for IDENTITY and RELU only");
    EpiParams e;
    epi_fill(&e, scale_bias, 1.f, scale_dst, nonline, false, true);
    *c = e.lin_c;
    *d = e.lin_d;
    return e.lin;
}

int mi355_epilogue_residual_table(float scale_bias, float scale_z, float scale_dst, uint32_t nonline, float* c, float* table) {
    if (!c || !table) return -fail(MI355_ERR_BAD_ARG, "null output");
    if (nonline != MI355_NL_IDENTITY && nonline != MI355_NL_RELU)
        return -fail(MI355_ERR_BAD_ARG, "the residual table form exists for IDENTITY and RELU only");
    EpiParams e;
    epi_fill(&e, scale_bias, scale_z, scale_dst, nonline, true, true);
    const float* t;
    if (!epi_residual_table(e, c, &t)) return 0;
    memcpy(table, t, 256 * sizeof(float));
    return 1;
}

// ---- RelayoutFormat ----
static uint32_t cdiv(uint32_t a, uint32_t b) { return (a + b - 1) / b; }

int mi355_relayout_deduce(const mi355_relayout_desc* d, uint32_t* ndim, uint32_t shape[7]) {
    if (!d || !ndim || !shape) return fail(MI355_ERR_BAD_ARG, "null argument");
    if (d->elem_bytes != 1 && d->elem_bytes != 4) return fail(MI355_ERR_UNSUPPORTED, "element size %u", d->elem_bytes);
    const uint32_t* s = d->shape;
    const uint32_t g = d->group ? d->group : 1;
    for (int i = 0; i < 7; ++i) shape[i] = 0;
    switch (d->mode) {
        case MI355_RL_NCHW_NCHW4_IC_SMALL:
            if (d->ndim != 4) return fail(MI355_ERR_SHAPE, "src must be 4-dim");
            if (s[1] > 4) return fail(MI355_ERR_SHAPE, "ic should be less equal 4");
            *ndim = 5; shape[0] = s[0]; shape[1] = cdiv(s[1], 4); shape[2] = s[2]; shape[3] = s[3]; shape[4] = 4;
            return MI355_OK;
        case MI355_RL_NCHW_NCHW4:
        case MI355_RL_NCHW_NCHW32: {
            const uint32_t p = d->mode == MI355_RL_NCHW_NCHW4 ? 4 : 32;
            if (d->ndim != 4) return fail(MI355_ERR_SHAPE, "src must be 4-dim");
            if (s[1] % g) return fail(MI355_ERR_SHAPE, "channels %u not divisible by group %u", s[1], g);
            *ndim = 5; shape[0] = s[0]; shape[1] = g * cdiv(s[1] / g, p); shape[2] = s[2]; shape[3] = s[3];
            shape[4] = p;
            return MI355_OK;
        }
        case MI355_RL_NCHW4_NCHW:
        case MI355_RL_NCHW32_NCHW: {
            const uint32_t p = d->mode == MI355_RL_NCHW4_NCHW ? 4 : 32;
            if (d->ndim != 5 || s[4] != p) return fail(MI355_ERR_SHAPE, "src must be (n, c/%u, h, w, %u)", p, p);
            const uint32_t c = d->oc ? d->oc : s[1] * p;
            if (c % g) return fail(MI355_ERR_SHAPE, "oc %u not divisible by group %u", c, g);
            if (c > s[1] * p || g * cdiv(c / g, p) != s[1])
                return fail(MI355_ERR_SHAPE, "oc %u / group %u do not match %u packed blocks", c, g, s[1]);
            *ndim = 4; shape[0] = s[0]; shape[1] = c; shape[2] = s[2]; shape[3] = s[3];
            return MI355_OK;
        }
        case MI355_RL_NCHW_NCHW4_WEIGHT:
            if (d->ndim == 4) {
                *ndim = 5; shape[0] = cdiv(s[0], 4) * 4; shape[1] = cdiv(s[1], 4); shape[2] = s[2]; shape[3] = s[3];
                shape[4] = 4;
                return MI355_OK;
            }
            if (d->ndim == 5) {
                *ndim = 6; shape[0] = s[0]; shape[1] = cdiv(s[1], 4) * 4; shape[2] = cdiv(s[2], 4); shape[3] = s[3];
                shape[4] = s[4]; shape[5] = 4;
                return MI355_OK;
            }
            return fail(MI355_ERR_SHAPE, "weight must be 4-dim (dense) or 5-dim (group)");
        case MI355_RL_NCHW4_NCHW32:
            if (d->ndim != 5 || s[4] != 4 || s[1] % 8) return fail(MI355_ERR_SHAPE, "src must be (n, c/4, h, w, 4), c %% 32 == 0");
            *ndim = 5; shape[0] = s[0]; shape[1] = s[1] / 8; shape[2] = s[2]; shape[3] = s[3]; shape[4] = 32;
            return MI355_OK;
        case MI355_RL_NCHW32_NCHW4:
            if (d->ndim != 5 || s[4] != 32) return fail(MI355_ERR_SHAPE, "src must be (n, c/32, h, w, 32)");
            *ndim = 5; shape[0] = s[0]; shape[1] = s[1] * 8; shape[2] = s[2]; shape[3] = s[3]; shape[4] = 4;
            return MI355_OK;
        default:
            return fail(MI355_ERR_UNSUPPORTED, "Invalid RelayoutFormat Mode %u", d->mode);
    }
}

int mi355_relayout_exec(void* stream, const mi355_relayout_desc* d, const void* src, void* dst) {
    uint32_t ondim = 0, oshape[7];
    int st = mi355_relayout_deduce(d, &ondim, oshape);
    if (st) return st;
    if (!src || !dst) return fail(MI355_ERR_BAD_ARG, "null tensor pointer");
    // the byte-transposing kernels use 16-byte vectors; misaligned tensors take the generic kernel
    const bool fast = aligned16(src) && aligned16(dst);
    int rc = launch_relayout(reinterpret_cast<hipStream_t>(stream), *d, oshape, ondim, src, dst, fast);
    if (rc) return fail(MI355_ERR_LAUNCH, "relayout: %s", hipGetErrorString((hipError_t)rc));
    return MI355_OK;
}

}  // extern "C"
