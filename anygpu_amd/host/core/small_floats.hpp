// Storage-only 16- and 8-bit floating point element types for host code: bfloat16 and the two
// OCP fp8 formats (E4M3 with no infinities and a single NaN pattern per sign, E5M2 IEEE-like).
// gfx950 uses the OCP encodings.  Conversion goes through float32 with round-to-nearest-even.
#pragma once

#include <cmath>
#include <cstdint>
#include <cstring>
#include <limits>

namespace anygpu_host {

inline uint32_t float_bits(float f) { uint32_t u; std::memcpy(&u, &f, 4); return u; }
inline float bits_float(uint32_t u) { float f; std::memcpy(&f, &u, 4); return f; }

struct BFloat16
{
	uint16_t bits = 0;
	BFloat16() = default;
	BFloat16(float f)
	{
		uint32_t u = float_bits(f);
		if ((u & 0x7FFFFFFFu) > 0x7F800000u) { bits = static_cast<uint16_t>((u >> 16) | 0x40u); return; }  // NaN
		u += 0x7FFFu + ((u >> 16) & 1u);
		bits = static_cast<uint16_t>(u >> 16);
	}
	operator float() const { return bits_float(static_cast<uint32_t>(bits) << 16); }
};

// Generic small float with EXP exponent bits and MAN mantissa bits in one byte.
// IEEE_SPECIALS = true: top exponent encodes inf / NaN (E5M2).  false: only the all-ones
// pattern is NaN and the top exponent carries normal values (E4M3, max 448).
template <int EXP, int MAN, bool IEEE_SPECIALS>
struct Fp8
{
	uint8_t bits = 0;
	static constexpr int kBias = (1 << (EXP - 1)) - 1;

	Fp8() = default;
	Fp8(float f) { bits = encode(f); }
	Fp8(int v) { bits = encode(static_cast<float>(v)); }
	operator float() const { return decode(bits); }

	static float max_finite()
	{
		const int top = (1 << EXP) - 1;
		if (IEEE_SPECIALS) return std::ldexp(2.0f - std::ldexp(1.0f, -MAN), top - 1 - kBias);
		return std::ldexp(2.0f - 2.0f * std::ldexp(1.0f, -MAN), top - kBias);
	}

	// Largest code that holds a finite value.
	static constexpr int kMaxCode = IEEE_SPECIALS ? ((((1 << EXP) - 1) << MAN) - 1) : 0x7E;

	// Nearest representable magnitude, ties to the even code.  Codes are monotone in value, so
	// a binary search over the positive codes finds the bracketing pair.
	static uint8_t encode(float f)
	{
		const uint8_t sign = std::signbit(f) ? 0x80 : 0x00;
		if (std::isnan(f)) return static_cast<uint8_t>(sign | 0x7F);
		const float a = std::fabs(f);
		if (a >= max_finite())
		{
			if (IEEE_SPECIALS && (std::isinf(a) || a >= max_finite() + std::ldexp(1.0f, (1 << EXP) - 2 - kBias - MAN - 1)))
				return static_cast<uint8_t>(sign | (((1 << EXP) - 1) << MAN));   // rounds to infinity
			if (!IEEE_SPECIALS && std::isinf(a)) return static_cast<uint8_t>(sign | 0x7F);
			return static_cast<uint8_t>(sign | kMaxCode);                        // saturate
		}
		int lo = 0, hi = kMaxCode;               // decode(lo) <= a < decode(hi)
		while (hi - lo > 1)
		{
			const int mid = (lo + hi) / 2;
			if (decode(static_cast<uint8_t>(mid)) <= a) lo = mid; else hi = mid;
		}
		const float dl = a - decode(static_cast<uint8_t>(lo));
		const float dh = decode(static_cast<uint8_t>(hi)) - a;
		int code = lo;
		if (dh < dl || (dh == dl && (hi & 1) == 0)) code = hi;
		return static_cast<uint8_t>(sign | code);
	}

	static float decode(uint8_t b)
	{
		const float sign = (b & 0x80) ? -1.0f : 1.0f;
		const int exp = (b >> MAN) & ((1 << EXP) - 1);
		const int man = b & ((1 << MAN) - 1);
		if (IEEE_SPECIALS && exp == (1 << EXP) - 1)
			return man == 0 ? sign * std::numeric_limits<float>::infinity() : std::numeric_limits<float>::quiet_NaN();
		if (!IEEE_SPECIALS && (b & 0x7F) == 0x7F) return std::numeric_limits<float>::quiet_NaN();
		if (exp == 0) return sign * std::ldexp(static_cast<float>(man), 1 - kBias - MAN);
		return sign * std::ldexp(1.0f + std::ldexp(static_cast<float>(man), -MAN), exp - kBias);
	}
};

using Fp8E4M3 = Fp8<4, 3, false>;
using Fp8E5M2 = Fp8<5, 2, true>;

}  // namespace anygpu_host
