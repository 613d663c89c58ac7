// Wrapper translation unit that compiles the reference's own E4M3 byte
// contract (include/ida_native/fp8_e4m3.hpp, found through -I at its place in
// the reference tree) into oracle/_ref/libcf_ref_e4m3.so.  The header calls
// signbit/isfinite unqualified (fp8_e4m3.hpp:32,34), which a host C++ compiler
// only resolves after these using-declarations.  TEST INFRASTRUCTURE ONLY.
#include <cmath>
#include <cstddef>
#include <cstdint>
using std::isfinite;
using std::signbit;
#include "ida_native/fp8_e4m3.hpp"

extern "C" {
void ref_e4m3_pack_n(const float* in, std::uint8_t* out, std::uint8_t* finite, std::size_t n) {
    for (std::size_t i = 0; i < n; ++i) {
        const auto p = ida_native::fp8_e4m3::pack(in[i]);
        out[i] = p.bits;
        if (finite) finite[i] = p.finite ? 1 : 0;
    }
}
void ref_e4m3_unpack_n(const std::uint8_t* in, float* out, std::size_t n) {
    for (std::size_t i = 0; i < n; ++i) out[i] = ida_native::fp8_e4m3::unpack(in[i]);
}
// Sweeps fp32 bit patterns first, first+stride, ... (count of them) and returns
// how many differ from `mine`, a pack function with the oracle's signature.
std::uint64_t ref_e4m3_sweep(std::uint8_t (*mine)(float, int*), std::uint32_t first,
                             std::uint32_t stride, std::uint64_t count, std::uint32_t* first_bad) {
    std::uint64_t bad = 0;
    std::uint32_t bits = first;
    for (std::uint64_t i = 0; i < count; ++i, bits += stride) {
        float v;
        __builtin_memcpy(&v, &bits, 4);
        int fin = 1;
        const std::uint8_t got = mine(v, &fin);
        const auto want = ida_native::fp8_e4m3::pack(v);
        if (got != want.bits || (fin != 0) != want.finite) {
            if (bad == 0 && first_bad) *first_bad = bits;
            ++bad;
        }
    }
    return bad;
}
}
