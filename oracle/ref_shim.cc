// Build shim for oracle/_ref: wraps ONE of the reference's C functional-model
// files (passed on the command line as -DREF_INL='"<path>.inl"', read in place
// from the reference tree) in an extern "C" block, and adds an array driver
// around the reference's scalar function REF_FN so that it can be swept through
// ctypes at C speed.  Holds no reference code itself.  Test infrastructure only.
#include <stdint.h>
#include <math.h>
extern "C" {
#include REF_INL
}
#define CAT_(a, b) a##b
#define CAT(a, b) CAT_(a, b)
extern "C" void CAT(ref_array_, REF_FN)(const float *a, const float *b, float *out, long n)
{
    for (long i = 0; i < n; ++i) out[i] = REF_FN(a[i], b[i]);
}
