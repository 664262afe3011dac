// Number formats of the bfAintBGemm harness.
// Same names and meaning as /root/reference/bfAintBGemm/datatype.hpp: bf16 travels as a raw
// 16-bit pattern (`bfloat16 = unsigned short`, :4-7); `type_convert<bhalf_t,float>` truncates
// (:44-55); `type_convert<float,bhalf_t>` widens (:31-42); `bf16_convert_rtn` rounds to nearest
// even and keeps signalling NaNs NaN (:80-121).  Host-only here (no HIP header needed).
#pragma once
#include <cstdint>
#include <cstring>
#include <type_traits>

using bfloat16 = unsigned short;
using bhalf_t = bfloat16;

namespace bfaintb_host {
inline std::uint32_t f32_bits(float x) { std::uint32_t u; std::memcpy(&u, &x, 4); return u; }
inline float bits_f32(std::uint32_t u) { float x; std::memcpy(&x, &u, 4); return x; }
}  // namespace bfaintb_host

// Generic case: a plain static_cast (datatype.hpp:9-16).
template <typename Y, typename X>
inline Y type_convert(X x)
{
    static_assert(!std::is_reference<Y>::value && !std::is_reference<X>::value, "value types only");
    return static_cast<Y>(x);
}

// bf16 -> fp32: the 16 bits become the high half.
template <>
inline float type_convert<float, bhalf_t>(bhalf_t x) { return bfaintb_host::bits_f32(std::uint32_t(x) << 16); }

// fp32 -> bf16 by truncation (what the reference's mem_transfer uses for A).
template <>
inline bhalf_t type_convert<bhalf_t, float>(float x) { return bhalf_t(bfaintb_host::f32_bits(x) >> 16); }

// bf16 -> int8 and int8 -> bf16, both by way of fp32 (datatype.hpp:57-73).
template <>
inline std::int8_t type_convert<std::int8_t, bhalf_t>(bhalf_t x) { return static_cast<std::int8_t>(type_convert<float, bhalf_t>(x)); }
template <>
inline bhalf_t type_convert<bhalf_t, std::int8_t>(std::int8_t x) { return type_convert<bhalf_t, float>(static_cast<float>(x)); }

template <typename Y, typename X>
inline Y bf16_convert_rtn(X x);

// fp32 -> bf16, round to nearest even.  Finite values: add 0x7fff plus the parity of the bit that
// becomes the bf16 LSB, then drop the low half (carries ripple into the exponent, up to Inf).
// Inf passes through; a NaN whose payload would be dropped entirely gets a payload bit set.
template <>
inline bhalf_t bf16_convert_rtn<bhalf_t, float>(float x)
{
    std::uint32_t u = bfaintb_host::f32_bits(x);
    const bool finite = (~u & 0x7f800000u) != 0u;
    if (finite) u += 0x7fffu + ((u >> 16) & 1u);
    else if (u & 0xffffu) u |= 0x10000u;
    return bhalf_t(u >> 16);
}
