// Division by a run-time constant as multiply and shift, for the index arithmetic of the implicit-GEMM
// convolution gathers: q = (n * mul) >> shift is floor(n / d) for every 0 <= n < 2^31 when
// shift = 31 + ceil(log2 d) and mul = floor(2^shift / d) + 1 (the error term n * (d - 2^shift mod d) / 2^shift
// stays below 1).  A general 32-bit integer division costs forty-odd instructions on the GPU; this one costs
// a 64-bit multiply and a shift.
#pragma once

#include <hip/hip_runtime.h>

namespace helix_fastdiv {

struct FastDiv {
    unsigned mul;
    int shift;
    int d;
    __host__ __device__ __forceinline__ int div(int n) const {
        return (int)(((unsigned long long)(unsigned)n * mul) >> shift);
    }
};

inline FastDiv make(int d) {
    int l = 0;
    while ((1LL << l) < d) l++;
    FastDiv f;
    f.shift = 31 + l;
    f.mul = (unsigned)(((1ULL << f.shift) / (unsigned long long)d) + 1ULL);
    f.d = d;
    return f;
}

}  // namespace helix_fastdiv
