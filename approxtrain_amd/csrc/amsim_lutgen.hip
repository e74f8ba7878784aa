// Mantissa-product table generation (host code): the counterpart of the
// reference's lut/lut_gen.cc + lut/lut_gen.sh flow.  A table is made either by
// evaluating a caller-supplied multiplier `float f(float, float)` on every pair
// of m-bit mantissas at biased exponent 127 (the plug-in route of
// developer.md:38-86), or from the closed integer rules of the built-in
// designs (no floating point involved).
#include "amsim_internal.h"

#include <cstring>
#include <string>

namespace amsim {

namespace {

struct Entry {
    uint32_t carry;  // 0 / 1: the product's exponent went up by one
    uint32_t mant;   // m-bit result mantissa, right-aligned
};

inline uint32_t bits_of(float f)
{
    uint32_t u;
    std::memcpy(&u, &f, 4);
    return u;
}
inline float float_of(uint32_t u)
{
    float f;
    std::memcpy(&f, &u, 4);
    return f;
}

// lut/lut_gen.cc:106-122: a = 1.i, b = 1.j at exponent 127; the entry keeps the
// top m mantissa bits of f(a, b) and whether its exponent field exceeds 127.
Entry entry_from_function(amsim_multiplier_fn fn, void *user, int m, uint32_t i, uint32_t j)
{
    const uint32_t at = 0x3f800000u | (i << (23 - m)), bt = 0x3f800000u | (j << (23 - m));
    const uint32_t ct = bits_of(fn(float_of(at), float_of(bt), user));
    const uint32_t mask = ((1u << m) - 1u) << (23 - m);
    Entry e;
    e.mant = (ct & mask) >> (23 - m);
    e.carry = (ct & 0x7f800000u) > 0x3f800000u ? 1u : 0u;
    return e;
}

// Mitchell's logarithmic multiplier (lut/Mitchell_16.inl:21-38): the mantissa
// fractions add; an overflow of the sum is the carry.
Entry entry_mitchell(int m, uint32_t i, uint32_t j)
{
    const uint32_t s = i + j;
    return Entry{s >> m, s & ((1u << m) - 1u)};
}

// Minimally biased multiplier (lut/FPmultMBM_fast16.inl:18-40 and the narrower
// variants): Mitchell's sum on fractions whose bit below the kept width is
// forced to one, plus a constant correction that is halved after a carry and
// dropped where it would overflow the sum.
Entry entry_mbm(int m, uint32_t i, uint32_t j)
{
    const uint32_t tm = ((1u << m) - 1u) << (23 - m);  // kept fraction bits
    const uint32_t sb = 1u << (23 - m);                // the kept width's LSB, forced to one
    const uint32_t a = i << (23 - m), b = j << (23 - m);
    const uint32_t s = ((a & tm) | sb) + ((b & tm) | sb);
    const uint32_t carry = s >= (1u << 23) ? 1u : 0u;
    const uint32_t corr = (0xA0000u >> carry) & tm;
    uint32_t sc = (s & 0x7fffffu) + corr;
    if (carry && sc >= (1u << 23)) sc = s;
    uint32_t wh = ((1u << 23) + sc) << carry;
    uint32_t n = wh >= (1u << 24) ? 1u : 0u;
    if (n) wh >>= 1;
    return Entry{n, (wh & 0x7fffffu & tm) >> (23 - m)};
}

// Exact product of the truncated significands, truncated again (lut/bfloat.inl).
Entry entry_exact_truncated(int m, uint32_t i, uint32_t j)
{
    const uint64_t p = (uint64_t)((1u << m) + i) * ((1u << m) + j);
    const uint32_t n = p >= ((uint64_t)1 << (2 * m + 1)) ? 1u : 0u;
    return Entry{n, (uint32_t)(p >> (m + n)) & ((1u << m) - 1u)};
}

enum Builtin { B_NONE, B_MBM, B_MIT, B_ACC, B_ZEROS };

Builtin builtin_of(const char *name)
{
    if (!name) return B_NONE;
    const std::string s(name);
    if (s == "MBM") return B_MBM;
    if (s == "MIT") return B_MIT;
    if (s == "ACC") return B_ACC;
    if (s == "ZEROS") return B_ZEROS;
    return B_NONE;
}

template <typename F>
int fill(int m, int entry_bytes, void *out, size_t n_bytes, F entry)
{
    if (!out) return fail(AMSIM_ERR_INVALID, "no output buffer for the table");
    if (entry_bytes == 1 ? (m < 1 || m > 7) : entry_bytes == 4 ? (m < 1 || m > 11) : true)
        return fail(AMSIM_ERR_LUT_FORMAT, "mantissa width must be 1..7 for 1-byte entries, 1..11 for 4-byte entries");
    const size_t n = (size_t)1 << (2 * m);
    if (n_bytes < n * (size_t)entry_bytes)
        return fail(AMSIM_ERR_INVALID, "table buffer smaller than 2^(2m) entries");
    for (uint32_t i = 0; i < (1u << m); ++i)
        for (uint32_t j = 0; j < (1u << m); ++j) {
            const Entry e = entry(i, j);
            const size_t idx = ((size_t)i << m) | j;
            if (entry_bytes == 1) static_cast<uint8_t *>(out)[idx] = (uint8_t)((e.carry << 7) | e.mant);
            else static_cast<uint32_t *>(out)[idx] = (e.carry << 31) | (e.mant << (23 - m));
        }
    return AMSIM_OK;
}

}  // namespace

}  // namespace amsim

using namespace amsim;

extern "C" {

int amsim_lut_generate(amsim_multiplier_fn fn, void *user, int mant_width, int entry_bytes, void *entries,
                       size_t n_bytes)
{
    if (!fn) return fail(AMSIM_ERR_INVALID, "no multiplier function");
    return fill(mant_width, entry_bytes, entries, n_bytes,
                [&](uint32_t i, uint32_t j) { return entry_from_function(fn, user, mant_width, i, j); });
}

int amsim_lut_generate_builtin(const char *name, int mant_width, int entry_bytes, void *entries, size_t n_bytes)
{
    const int m = mant_width;
    switch (builtin_of(name)) {
    case B_MBM: return fill(m, entry_bytes, entries, n_bytes, [&](uint32_t i, uint32_t j) { return entry_mbm(m, i, j); });
    case B_MIT: return fill(m, entry_bytes, entries, n_bytes, [&](uint32_t i, uint32_t j) { return entry_mitchell(m, i, j); });
    case B_ACC: return fill(m, entry_bytes, entries, n_bytes, [&](uint32_t i, uint32_t j) { return entry_exact_truncated(m, i, j); });
    case B_ZEROS: return fill(m, entry_bytes, entries, n_bytes, [&](uint32_t, uint32_t) { return Entry{0u, 0u}; });
    default: return fail(AMSIM_ERR_INVALID, std::string("unknown built-in multiplier '") + (name ? name : "") +
                                                "' (MBM, MIT, ACC, ZEROS)");
    }
}

}  // extern "C"
