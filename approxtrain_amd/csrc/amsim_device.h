// Device-side building blocks of the approximate product (gfx950).
#ifndef AMSIM_DEVICE_H_
#define AMSIM_DEVICE_H_

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <type_traits>

namespace amsim {

__device__ __forceinline__ uint32_t f2u(float f) { return __float_as_uint(f); }
__device__ __forceinline__ float u2f(uint32_t u) { return __uint_as_float(u); }

// An operand is "safe" when it is a zero or a normal number with biased
// exponent in [64, 190].  For two safe operands the product of the functional
// models (lut/FPmultMBM_fast16.inl:45-134) reduces to
//     sign(a)^sign(b) | (ea + eb - 127 + carry) << 23 | mantissa
// with no underflow, overflow or special case: ea + eb lies in [128, 380], and
// a zero operand gives a zero product.  Everything else takes am_exact().
__device__ __forceinline__ bool operand_unsafe(uint32_t bits)
{
    uint32_t mag = bits & 0x7fffffffu;
    uint32_t e = mag >> 23;
    return mag != 0u && (e - 64u) > 126u;
}

// Range bookkeeping for many operands at once (two min/max updates per operand
// instead of a compare chain): t = bits << 1 drops the sign; zeros wrap to the
// top of the range in (t - 1) and so never lower the minimum.
struct SafeRange {
    uint32_t tmax = 0u, tmin = 0xffffffffu;
    __device__ __forceinline__ void add(uint32_t bits)
    {
        const uint32_t t = bits << 1;
        tmax = max(tmax, t);
        tmin = min(tmin, t - 1u);
    }
    // same predicate as operand_unsafe() over everything added
    __device__ __forceinline__ bool unsafe() const { return tmax >= (191u << 24) || tmin < (64u << 24) - 1u; }
};

// The quick test above is per operand.  Whether a PRODUCT can take the fast form depends on both
// operands: sign | (ea + eb - 127 + carry) << 23 | mantissa is right whenever both are normal (or
// zero) and ea + eb lies in [128, 380] -- e.g. gradients far below 2^-63 multiplied with weights
// near 1.  A set of operands is therefore summarised as a "span" word:
//   bit 31      some operand fails the quick test (zero, or exponent in [64, 190])
//   bit 30      a subnormal, an infinity or a NaN is among them (also set, conservatively, for the
//               smallest normal binade and for the largest: the carry of the LUT entry is added to
//               an operand's exponent field, which must not run into 255): only the full-domain
//               product will do
//   bits 15..8  smallest biased exponent among the non-zero operands (may read one less for an
//               exact power of two), 255 if all are zero
//   bits 7..0   largest biased exponent, 0 if all are zero
// and two spans are compatible if every product of their operands can take the fast form.
constexpr uint32_t SPAN_QUICK_FAIL = 0x80000000u, SPAN_HARD = 0x40000000u;
__device__ __forceinline__ uint32_t span_word(const SafeRange &r)
{
    const uint32_t emax = r.tmax >> 24;
    const bool all_zero = r.tmin == 0xffffffffu && r.tmax == 0u;
    const uint32_t emin = all_zero ? 255u : (r.tmin == 0xffffffffu ? emax : r.tmin >> 24);
    const bool hard = !all_zero && (emin == 0u || emax >= 254u);
    return (r.unsafe() ? SPAN_QUICK_FAIL : 0u) | (hard ? SPAN_HARD : 0u) | (emin << 8) | emax;
}
__device__ __forceinline__ bool spans_compatible(uint32_t a, uint32_t b)
{
    if ((a | b) & SPAN_HARD) return false;
    const uint32_t lo = ((a >> 8) & 255u) + ((b >> 8) & 255u), hi = (a & 255u) + (b & 255u);
    return lo >= 128u && hi <= 380u;
}
// union of the lanes' ranges, the same in every lane: max / min over the wavefront by data-parallel
// primitives (shifts inside rows of 16 lanes, then broadcasts of a row's last lane to the rows after
// it; lanes without a source keep the identity), the totals read back from lane 63
__device__ __forceinline__ uint32_t wave_max_u32(uint32_t v)
{
#if defined(__HIP_DEVICE_COMPILE__)
    v = max(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x111, 0xf, 0xf, false));  // row_shr:1
    v = max(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x112, 0xf, 0xf, false));  // row_shr:2
    v = max(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x114, 0xf, 0xe, false));  // row_shr:4
    v = max(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x118, 0xf, 0xc, false));  // row_shr:8
    v = max(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x142, 0xa, 0xf, false));  // row_bcast:15
    v = max(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x143, 0xc, 0xf, false));  // row_bcast:31
    return (uint32_t)__builtin_amdgcn_readlane((int)v, 63);
#else
    return v;
#endif
}
__device__ __forceinline__ SafeRange wave_union(SafeRange r)
{
    r.tmax = wave_max_u32(r.tmax);
    r.tmin = ~wave_max_u32(~r.tmin);  // min(x) == ~max(~x)
    return r;
}

// 64-bit add of a vector register pair and a scalar register pair in one instruction (the
// compiler's own choice for this sum is a multiply-add form that issues several times slower).
__device__ __forceinline__ uint64_t add_u64_vs(uint64_t v, uint64_t s_uniform)
{
    uint64_t d;
    asm("v_lshl_add_u64 %0, %1, 0, %2" : "=v"(d) : "v"(v), "s"(s_uniform));
    return d;
}

// LDS byte address of a pointer into a __shared__ object
__device__ __forceinline__ uint32_t lds_address(const void *p)
{
    return (uint32_t)(uintptr_t)(const __attribute__((address_space(3))) void *)p;
}

// Byte gather from LDS into the upper half of a register: the byte arrives already shifted left by
// 16, where the product factor wants it.  The lower half of d must be zero before (a device either
// keeps or clears the half that such a load does not write; either way it is zero afterwards).  The
// compiler does not know that this is a load: whoever reads the result first waits for it
// (wait_add_u64_vs).  Issued in program order (volatile).
__device__ __forceinline__ void lds_gather_u8_hi(uint32_t &d, uint32_t lds_byte_address)
{
    asm volatile("ds_read_u8_d16_hi %0, %1" : "+v"(d) : "v"(lds_byte_address));
}

// add_u64_vs after waiting until at most OUTSTANDING of the LDS / scalar-memory operations issued so
// far are still in flight (LDS operations complete in order, so this names the gathers that have
// landed; operations the compiler adds on its own only make the wait stricter).  Kept in program
// order relative to the gathers (volatile): the count is only meaningful after all of them.
template <int OUTSTANDING>
__device__ __forceinline__ uint64_t wait_add_u64_vs(uint64_t v, uint64_t s_uniform)
{
    uint64_t d;
    asm volatile("s_waitcnt lgkmcnt(%3)\n\tv_lshl_add_u64 %0, %1, 0, %2" : "=v"(d) : "v"(v), "s"(s_uniform), "n"(OUTSTANDING));
    return d;
}

// The same sum and a fused multiply-add, kept where they are written relative to the gathers and
// waits above (volatile): the inner loop's instruction order is chosen by hand.
__device__ __forceinline__ uint64_t add_u64_vs_ordered(uint64_t v, uint64_t s_uniform)
{
    uint64_t d;
    asm volatile("v_lshl_add_u64 %0, %1, 0, %2" : "=v"(d) : "v"(v), "s"(s_uniform));
    return d;
}
__device__ __forceinline__ void fmac_ordered(float &acc, float a, float b)
{
    asm volatile("v_fmac_f32 %0, %1, %2" : "+v"(acc) : "v"(a), "v"(b));
}

template <int I, int N, class F>
__device__ __forceinline__ void static_for(F &&f)
{
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for<I + 1, N>(f);
    }
}

// Full-domain product.  `entry16` is the LUT byte (carry << 7 | mantissa
// left-aligned in 7 bits) shifted left by 16, i.e. carry << 23 | mantissa.
// Restates the exponent / special-case logic of the C functional models:
//   p = a * b (IEEE, subnormals kept) supplies sign, exponent and class;
//   exp(p) == 255 -> p itself (inf / NaN pass through, :99-101);
//   exp(p) == 0   -> +0 (:102-104);
//   else exponent = exp(p) - accurate_normalised + carry (:106-112), where
//   accurate_normalised is whether the exact significand product, rounded to
//   nearest even, reached 2.0 (:58-96).
__device__ __forceinline__ float am_exact(uint32_t at, uint32_t bt, uint32_t entry16)
{
    float p = u2f(at) * u2f(bt);
    uint32_t pt = f2u(p);
    uint32_t pe = (pt >> 23) & 255u;
    if (pe == 255u) return p;
    if (pe == 0u) return 0.0f;
    float sa = u2f(0x3f800000u | (at & 0x7fffffu));
    float sb = u2f(0x3f800000u | (bt & 0x7fffffu));
    uint32_t acc = (sa * sb >= 2.0f) ? 1u : 0u;
    return u2f((pt & 0x80000000u) + ((pe - acc) << 23) + entry16);
}

}  // namespace amsim
#endif
