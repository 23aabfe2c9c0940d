// Concepts that group the element types; operator overloads are constrained with them
// (same names as the reference's srcs/core/core_concepts.hpp:17-42).
#ifndef __CORE_CONCEPTS__
#define __CORE_CONCEPTS__

#include "core.hpp"
#include <concepts>
#include <type_traits>

template<typename T>
concept SmallFloatType = std::is_same_v<T, float16> || std::is_same_v<T, bfloat16> ||
                         std::is_same_v<T, fp8e4m3> || std::is_same_v<T, fp8e5m2>;

template<typename T>
concept FloatingPointType = std::floating_point<T> || SmallFloatType<T>;

template<typename T>
concept IntegerType = std::integral<T>;

template<typename T>
concept ArithmeticType = FloatingPointType<T> || IntegerType<T>;

template<typename T>
concept HalfFloatType = FloatingPointType<T> && sizeof(T) == 2;

template<typename T>
concept FP8Type = FloatingPointType<T> && sizeof(T) == 1;

template<typename T>
concept PreciseFloatType = FloatingPointType<T> && (sizeof(T) > 2);

template<typename T>
concept NotHalfFloatType = IntegerType<T> || PreciseFloatType<T>;

#endif  // __CORE_CONCEPTS__
