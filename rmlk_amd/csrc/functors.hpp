// Element functors of the broadcast binary ops, the contiguous maps and Cast: one definition for the
// kernels that run an operator over a whole tensor (binary.hip, unary.hip) and for the kernel that
// runs a batch of tiny ones (batch.hip), so that an element gets the same bits either way.
#pragma once

#include <limits>
#include <type_traits>

#include "common.hpp"

namespace rmlk {

template <typename T>
struct AddF {
    static __device__ __forceinline__ T apply(T x, T y) {
        if constexpr (std::is_integral<T>::value) {
            using U = typename std::make_unsigned<T>::type;
            return static_cast<T>(static_cast<U>(x) + static_cast<U>(y));
        } else {
            return x + y;
        }
    }
};
template <typename T>
struct SubF {
    static __device__ __forceinline__ T apply(T x, T y) {
        if constexpr (std::is_integral<T>::value) {
            using U = typename std::make_unsigned<T>::type;
            return static_cast<T>(static_cast<U>(x) - static_cast<U>(y));
        } else {
            return x - y;
        }
    }
};
template <typename T>
struct MulF {
    static __device__ __forceinline__ T apply(T x, T y) {
        if constexpr (std::is_integral<T>::value) {
            using U = typename std::make_unsigned<T>::type;
            return static_cast<T>(static_cast<U>(x) * static_cast<U>(y));
        } else {
            return x * y;
        }
    }
};
// Integer division truncates toward zero (cuda/src/ptx/div.cu:9-12). The reference leaves x/0 and
// MIN/-1 undefined; here x/0 = 0 and MIN/-1 wraps to MIN so that no input can trap.
template <typename T>
struct DivF {
    static __device__ __forceinline__ T apply(T x, T y) {
        if constexpr (std::is_integral<T>::value) {
            using U = typename std::make_unsigned<T>::type;
            if (y == 0) return 0;
            if (y == static_cast<T>(-1)) return static_cast<T>(U(0) - static_cast<U>(x));
            return x / y;
        } else {
            return x / y;
        }
    }
};
template <typename T>
struct EqualF {
    static __device__ __forceinline__ uint8_t apply(T x, T y) { return x == y ? 1 : 0; }
};
template <typename T>
struct GreaterF {
    static __device__ __forceinline__ uint8_t apply(T x, T y) { return x > y ? 1 : 0; }
};

// Pow (cuda/src/ptx/pow.cu:18-65): float base -> powf(x, (float)y); double base -> pow; integer
// base -> llround(pow((double)x, (double)y)). Exponents 2, 3 and 0.5 take the product / sqrt
// forms, which are the correctly rounded results the CPU oracle produces for them.
template <typename TX, typename TY>
struct PowF {
    static __device__ __forceinline__ TX apply(TX x, TY y) {
        if constexpr (std::is_same<TX, float>::value) {
            float e = static_cast<float>(y);
            if (e == 2.0f) return x * x;
            if (e == 3.0f) return x * x * x;
            if (e == 0.5f) return sqrtf(x);
            return powf(x, e);
        } else if constexpr (std::is_same<TX, double>::value) {
            double e = static_cast<double>(y);
            if (e == 2.0) return x * x;
            if (e == 3.0) return x * x * x;
            if (e == 0.5) return sqrt(x);
            return pow(x, e);
        } else {
            double r = pow(static_cast<double>(x), static_cast<double>(y));
            return static_cast<TX>(llround(r));
        }
    }
};

template <typename T>
struct SqrtF {
    static __device__ __forceinline__ T apply(T x) {
        if constexpr (std::is_same<T, float>::value) return sqrtf(x);
        else return sqrt(x);
    }
};
// The reference multiplies by -1 (cuda/src/ptx/neg.cu:6); a sign flip gives the same bits.
template <typename T>
struct NegF {
    static __device__ __forceinline__ T apply(T x) {
        if constexpr (std::is_integral<T>::value) {
            using U = typename std::make_unsigned<T>::type;
            return static_cast<T>(U(0) - static_cast<U>(x));
        } else {
            return -x;
        }
    }
};
template <typename T>
struct SinF {
    static __device__ __forceinline__ T apply(T x) {
        if constexpr (std::is_same<T, float>::value) return sinf(x);
        else return sin(x);
    }
};
template <typename T>
struct CosF {
    static __device__ __forceinline__ T apply(T x) {
        if constexpr (std::is_same<T, float>::value) return cosf(x);
        else return cos(x);
    }
};
template <typename T>
struct SigmoidF {
    static __device__ __forceinline__ T apply(T x) {
        if constexpr (std::is_same<T, float>::value) return 1.0f / (1.0f + expf(-x));
        else return 1.0 / (1.0 + exp(-x));
    }
};

struct BoolTag {
    uint8_t b;
};

template <typename TI, typename TO>
struct CastF {
    static __device__ __forceinline__ TO apply(TI x) {
        constexpr bool in_bool = std::is_same<TI, BoolTag>::value;
        constexpr bool out_bool = std::is_same<TO, BoolTag>::value;
        if constexpr (in_bool && out_bool) {
            return BoolTag{static_cast<uint8_t>(x.b ? 1 : 0)};
        } else if constexpr (in_bool) {
            return static_cast<TO>(x.b ? 1 : 0);
        } else if constexpr (out_bool) {
            return BoolTag{static_cast<uint8_t>(x != static_cast<TI>(0) ? 1 : 0)};
        } else if constexpr (std::is_integral<TO>::value && !std::is_integral<TI>::value) {
            // float -> int: truncate toward zero; NaN -> 0; out of range saturates at the limits of
            // the 32-bit type of the same signedness (64-bit for 64-bit targets), and an 8- or
            // 16-bit target keeps the low bits of that: what the reference's `static_cast` compiles
            // to (a 32-bit conversion, then a narrowing move), pinned by its own vector
            // half 32768.0 -> int16 -32768 (cuda/src/kernels/cast.rs:524-539).
            using Wide = std::conditional_t<(sizeof(TO) > 4),
                                            TO,
                                            std::conditional_t<std::is_signed<TO>::value, int32_t, uint32_t>>;
            double v = static_cast<double>(x);
            if (v != v) return 0;
            constexpr double lo = static_cast<double>(std::numeric_limits<Wide>::min());
            // max() of 64-bit types is not a double; 2^63 / 2^64 is the first value out of range.
            constexpr double hi = static_cast<double>(std::numeric_limits<Wide>::max());
            if (v <= lo) return static_cast<TO>(std::numeric_limits<Wide>::min());
            if (v >= hi) return static_cast<TO>(std::numeric_limits<Wide>::max());
            return static_cast<TO>(static_cast<Wide>(v));
        } else {
            return static_cast<TO>(x);
        }
    }
};

}  // namespace rmlk
