// The 15 elementwise binary operators of BIDMat (BinOp codes GMat.scala:2245-2261, device
// table Operators.cu:86-101), as a compile-time template and as a run-time switch for epilogues.
#pragma once
#include <hip/hip_runtime.h>
#include <math.h>

namespace bm {

template <int OP>
__device__ __forceinline__ float binop(float a, float b) {
    if constexpr (OP == 0) return a + b;
    else if constexpr (OP == 1) return a - b;
    else if constexpr (OP == 2) return a * b;
    else if constexpr (OP == 3) return a / b;
    else if constexpr (OP == 4) return (a > b) ? 1.0f : 0.0f;
    else if constexpr (OP == 5) return (a < b) ? 1.0f : 0.0f;
    else if constexpr (OP == 6) return (a == b) ? 1.0f : 0.0f;
    else if constexpr (OP == 7) return (a >= b) ? 1.0f : 0.0f;
    else if constexpr (OP == 8) return (a <= b) ? 1.0f : 0.0f;
    else if constexpr (OP == 9) return (a != b) ? 1.0f : 0.0f;
    else if constexpr (OP == 10) return fmaxf(a, b);
    else if constexpr (OP == 11) return fminf(a, b);
    else if constexpr (OP == 12) return atan2f(a, b);
    else if constexpr (OP == 13) return powf(a, b);
    else return (a > 0) ? b : 0.0f;
}

// Run-time form: one switch per call site, for places where the op is applied once per many loads.
__device__ __forceinline__ float binop_rt(int opn, float a, float b) {
    switch (opn) {
    case 0: return binop<0>(a, b);
    case 1: return binop<1>(a, b);
    case 2: return binop<2>(a, b);
    case 3: return binop<3>(a, b);
    case 4: return binop<4>(a, b);
    case 5: return binop<5>(a, b);
    case 6: return binop<6>(a, b);
    case 7: return binop<7>(a, b);
    case 8: return binop<8>(a, b);
    case 9: return binop<9>(a, b);
    case 10: return binop<10>(a, b);
    case 11: return binop<11>(a, b);
    case 12: return binop<12>(a, b);
    case 13: return binop<13>(a, b);
    default: return binop<14>(a, b);
    }
}

}  // namespace bm
