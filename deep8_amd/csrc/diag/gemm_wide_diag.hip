// Diagnostic builds of the large-output fp16 GEMM (../gemm_wide_kernel.h).  Not part of the library: `python bench.py
// --phases --wide-diagnostic NAME` compiles this file with the switches of NAME and links it in place of
// gemm_wide.hip's object into a scratch copy of the library, then prints the kernel's phase record.  Each build
// leaves one part of the kernel out and so answers what that part costs -- in cycles on all-zero operands
// (`--operands zeros`), in clock, i.e. energy, on the configuration's data.  Every one of them computes wrong
// results; none reads or writes outside the operands.
//   -DD8_DIAG_NO_LOADS           the K loop without its global -> LDS loads
//   -DD8_DIAG_NO_FRAGMENT_READS  ... without its LDS reads (the MFMAs keep the first fragments)
//   -DD8_DIAG_NO_BARRIER         ... without its barrier
//   -DD8_DIAG_NO_STORES          the epilogue does everything but the stores to C
//   -DD8_DIAG_SAME_K             every K step fetches the tile's first step again: all loads hit in cache
#include "../gemm_wide_kernel.h"

namespace d8 {
namespace wide {

struct Diagnostic {
#ifdef D8_DIAG_NO_LOADS
    static constexpr bool LOADS = false;
#else
    static constexpr bool LOADS = true;
#endif
#ifdef D8_DIAG_NO_FRAGMENT_READS
    static constexpr bool FRAGMENT_READS = false;
#else
    static constexpr bool FRAGMENT_READS = true;
#endif
#ifdef D8_DIAG_NO_BARRIER
    static constexpr bool BARRIER = false;
#else
    static constexpr bool BARRIER = true;
#endif
#ifdef D8_DIAG_NO_STORES
    static constexpr bool STORES = false;
#else
    static constexpr bool STORES = true;
#endif
#ifdef D8_DIAG_SAME_K
    static constexpr bool ADVANCE_K = false;
#else
    static constexpr bool ADVANCE_K = true;
#endif
};

}  // namespace wide
}  // namespace d8

#define D8_WIDE_POLICY wide::Diagnostic
#include "../gemm_wide.hip"
