// neura.hpp -- C++ host layer over the C ABI of libneura_hip.so.
//
// The reference's host side is Rust (neura-gguf, neura-source, neura-decoder, neura-generate,
// neura-runtime); no Rust toolchain exists in this build, so the same interfaces are written
// in C++ with the same names, argument meaning and error behaviour.  Where the reference
// panics with a prose message this layer throws neura::Panic carrying the same sentence.
// Everything below the classes goes through include/neura_hip.h only.
#pragma once

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <deque>
#include <fstream>
#include <functional>
#include <map>
#include <memory>
#include <optional>
#include <stdexcept>
#include <string>
#include <unordered_map>
#include <vector>

#include "../../include/neura_hip.h"

namespace neura {

struct Panic : std::runtime_error {
    using std::runtime_error::runtime_error;
};

template <typename... Args>
[[noreturn]] inline void panic(const char *format, Args... args) {
    char text[1024];
    if constexpr (sizeof...(Args) == 0)
        snprintf(text, sizeof(text), "%s", format);
    else
        snprintf(text, sizeof(text), format, args...);
    throw Panic(text);
}

#define NEURA_ASSERT(condition, ...) \
    do {                             \
        if (!(condition)) ::neura::panic(__VA_ARGS__); \
    } while (0)

// ---- neura-abi: storage formats (crates/neura-abi/src/element.rs:3-17, :145-178, :231-240) ----

enum class Element : int32_t { Single = 0, Half = 1, Q8_0 = 8, Q3K = 11, Q4K = 12, Q5K = 13, Q6K = 14, Bfloat16 = 30 };

struct Block {
    uint32_t elements, bytes;
};

inline const char *name(Element element) {
    switch (element) {
    case Element::Single: return "single";
    case Element::Half: return "half";
    case Element::Q8_0: return "q8_0";
    case Element::Q3K: return "q3_k";
    case Element::Q4K: return "q4_k";
    case Element::Q5K: return "q5_k";
    case Element::Q6K: return "q6_k";
    case Element::Bfloat16: return "bfloat16";
    }
    return "unknown";
}

inline std::optional<Block> block(Element element) {
    switch (element) {
    case Element::Q8_0: return Block{32, 34};
    case Element::Q4K: return Block{256, 144};
    case Element::Q5K: return Block{256, 176};
    case Element::Q6K: return Block{256, 210};
    case Element::Q3K: return Block{256, 110};
    default: return std::nullopt;
    }
}

inline uint32_t bits_per_element(Element element) { return element == Element::Single ? 32 : 16; }

inline uint64_t payload_bytes(Element element, uint64_t elements) {
    if (auto held = block(element)) return (elements + held->elements - 1) / held->elements * held->bytes;
    return (elements * bits_per_element(element) + 7) / 8;
}

// ---- neura-precision: host encoders and decoders of the storage formats ------------------------
//
// pack() lays numbers out in a format's bytes and unpack() reads them back, as
// crates/neura-precision/src/lib.rs:5-68 does for the formats a GGUF decoder meets: single, half,
// bfloat16 and the five block formats of crates/neura-precision/src/ggml.rs.  Every product,
// quotient and rounding below is the reference's, in its order, in IEEE single precision, so the
// bytes are the reference's bytes.

namespace precision {

// IEEE half from single, round to nearest even (what half::f16::from_f32 does)
inline uint16_t half_bits(float value) {
    uint32_t bits;
    std::memcpy(&bits, &value, 4);
    const uint32_t sign = (bits >> 16) & 0x8000u;
    bits &= 0x7fffffffu;
    if (bits >= 0x7f800000u) return (uint16_t)(sign | 0x7c00u | (bits > 0x7f800000u ? 0x0200u | ((bits >> 13) & 0x3ffu) : 0u));
    if (bits >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u);  // rounds past the largest half
    if (bits < 0x33000001u) return (uint16_t)sign;               // at most half of the least subnormal
    const int32_t exponent = (int32_t)(bits >> 23) - 127;
    uint32_t mantissa = (bits & 0x7fffffu) | 0x800000u;
    const int32_t drop = exponent < -14 ? 13 + (-14 - exponent) : 13;
    const uint32_t kept = mantissa >> drop, rest = mantissa & ((1u << drop) - 1u), middle = 1u << (drop - 1);
    uint32_t out = exponent < -14 ? kept : (((uint32_t)(exponent + 15) << 10) + (kept & 0x3ffu));
    if (rest > middle || (rest == middle && (out & 1u))) out++;
    return (uint16_t)(sign | out);
}

inline float half_value(uint16_t half) {
    const uint32_t sign = (uint32_t)(half & 0x8000u) << 16, exponent = (half >> 10) & 31u, mantissa = half & 0x3ffu;
    uint32_t bits;
    if (exponent == 31)
        bits = sign | 0x7f800000u | (mantissa << 13);
    else if (exponent != 0)
        bits = sign | ((exponent + 112u) << 23) | (mantissa << 13);
    else if (mantissa == 0)
        bits = sign;
    else {
        int shift = 0;
        uint32_t m = mantissa;
        while (!(m & 0x400u)) m <<= 1, shift++;
        bits = sign | ((uint32_t)(113 - shift) << 23) | ((m & 0x3ffu) << 13);
    }
    float value;
    std::memcpy(&value, &bits, 4);
    return value;
}

// crates/neura-precision/src/lib.rs:325-329
inline uint16_t bfloat16_bits(float value) {
    uint32_t bits;
    std::memcpy(&bits, &value, 4);
    return (uint16_t)((bits + 0x7fffu + ((bits >> 16) & 1u)) >> 16);
}

namespace detail {

inline float least(float value, float other) { return value < other ? value : other; }     // ggml.rs:90-92
inline float greatest(float value, float other) { return value > other ? value : other; }  // ggml.rs:94-96
inline float rounded(float value) { return std::round(value); }                            // f32::round: halves away from zero
inline float clamped(float value, float low, float high) { return value < low ? low : value > high ? high : value; }

inline void put_half(uint8_t *field, size_t at, float value) {
    const uint16_t bits = half_bits(value);
    field[at] = (uint8_t)bits, field[at + 1] = (uint8_t)(bits >> 8);
}
inline float half_at(const uint8_t *field, size_t at) { return half_value((uint16_t)(field[at] | field[at + 1] << 8)); }
inline void put_nibble(uint8_t *field, size_t at, bool high, uint32_t value) { field[at] |= (uint8_t)((value & 0x0fu) << (high ? 4 : 0)); }
inline uint32_t nibble_at(uint8_t byte, bool high) { return high ? byte >> 4 : byte & 0x0fu; }

// ggml.rs:120-125: the quotient rounds, clamps and converts to an unsigned integer, a conversion
// that saturates: whatever lies below zero after the clamp becomes 0
inline uint32_t quantized(float value, float quantum, float low, float high) {
    if (quantum == 0.0f) return 0;
    const float held = clamped(rounded(value / quantum), low, high);
    return held < 0.0f ? 0u : (uint32_t)held;
}

// ggml.rs:127-149: eight six-bit scales and eight six-bit minima in twelve bytes
inline void scale_min_k4(const uint8_t *scales, size_t at, uint32_t &scale, uint32_t &min) {
    if (at < 4) {
        scale = scales[at] & 63u, min = scales[at + 4] & 63u;
    } else {
        scale = (scales[at + 4] & 0x0fu) | (uint32_t)(scales[at - 4] >> 6) << 4;
        min = (uint32_t)(scales[at + 4] >> 4) | (uint32_t)(scales[at] >> 6) << 4;
    }
}
inline void put_scale_min_k4(uint8_t *scales, size_t at, uint32_t scale, uint32_t min) {
    if (at < 4) {
        scales[at] = (uint8_t)scale, scales[at + 4] = (uint8_t)min;
    } else {
        scales[at + 4] = (uint8_t)((scale & 0x0fu) | (min & 0x0fu) << 4);
        scales[at - 4] |= (uint8_t)((scale >> 4) << 6);
        scales[at] |= (uint8_t)((min >> 4) << 6);
    }
}

// ggml.rs:209-216: quantum = the largest magnitude / 127, codes round(value * (1 / quantum))
inline void q8_0(const float *values, uint8_t *field) {
    float size = 0.0f;
    for (int at = 0; at < 32; at++)
        if (size < std::fabs(values[at])) size = std::fabs(values[at]);
    const float quantum = size / 127.0f;
    const float inverse = quantum == 0.0f ? 0.0f : 1.0f / quantum;
    put_half(field, 0, quantum);
    for (int at = 0; at < 32; at++) field[2 + at] = (uint8_t)(int8_t)clamped(rounded(values[at] * inverse), -127.0f, 127.0f);
}

// ggml.rs:151-207: Q4_K (steps 15) and Q5_K (steps 31).  Each 32-element sub-block spans from
// min(0, its least) to its greatest in `steps` steps; the super-block stores the widest step and
// the deepest low over 63 as halves and each sub-block a six-bit multiple of either.
inline void affine_block(Element element, const float *values, uint8_t *field, uint32_t steps) {
    const size_t bytes = element == Element::Q5K ? 176 : 144, quants = element == Element::Q5K ? 48 : 16;
    float lows[8], quantums[8];
    for (int at = 0; at < 8; at++) {
        float low = 0.0f, high = 0.0f;
        for (int i = 0; i < 32; i++) low = least(low, values[at * 32 + i]), high = greatest(high, values[at * 32 + i]);
        lows[at] = least(0.0f, low);
        quantums[at] = (high - lows[at]) / (float)steps;
    }
    float scale = 0.0f, min = 0.0f;
    for (int at = 0; at < 8; at++) scale = greatest(scale, quantums[at]), min = greatest(min, -lows[at]);
    scale = scale / 63.0f, min = min / 63.0f;
    uint8_t codes[8], mins[8];
    for (int at = 0; at < 8; at++) {
        codes[at] = (uint8_t)clamped(rounded(scale == 0.0f ? 0.0f : quantums[at] / scale), 0.0f, 63.0f);
        mins[at] = (uint8_t)clamped(rounded(min == 0.0f ? 0.0f : -lows[at] / min), 0.0f, 63.0f);
    }
    std::memset(field, 0, bytes);
    put_half(field, 0, scale);
    put_half(field, 2, min);
    for (int at = 0; at < 8; at++) put_scale_min_k4(field + 4, at, codes[at], mins[at]);
    for (int at = 0; at < 8; at++) {
        const float quantum = scale * (float)codes[at], low = min * (float)mins[at];
        const int group = at / 2;
        const bool seat = at % 2 == 1;
        for (int within = 0; within < 32; within++) {
            const uint32_t code = quantized(values[at * 32 + within] + low, quantum, 0.0f, (float)steps);
            put_nibble(field, quants + group * 32 + within, seat, code);
            if (element == Element::Q5K && (code & 0x10u)) field[16 + within] |= (uint8_t)(1u << (2 * group + (seat ? 1 : 0)));
        }
    }
}

// ggml.rs:242-289: sixteen sub-blocks of 16; d = the widest magnitude / 4 / 31, six-bit scale
// codes 32..63, three-bit codes -4..3 whose top bit (set when not negative) lies in bytes 0..31
inline void q3_k(const float *values, uint8_t *field) {
    float peaks[16], widest = 0.0f;
    for (int at = 0; at < 16; at++) {
        float peak = 0.0f;
        for (int i = 0; i < 16; i++) peak = greatest(peak, std::fabs(values[at * 16 + i]));
        peaks[at] = peak;
        widest = greatest(widest, peak);
    }
    if (!(widest >= 1.17549435e-38f)) widest = 1.17549435e-38f;  // f32::max(MIN_POSITIVE)
    const float d = widest / 4.0f / 31.0f;
    uint32_t codes[16];
    for (int at = 0; at < 16; at++) codes[at] = (uint32_t)clamped(rounded(peaks[at] / 4.0f / d), 0.0f, 31.0f) + 32u;
    std::memset(field, 0, 110);
    for (uint32_t at = 0; at < 16; at++) {  // put_q3_k_scale, ggml.rs:231-240
        const uint8_t low = (uint8_t)(codes[at] & 0x0fu), high = (uint8_t)((codes[at] >> 4) & 3u);
        field[96 + at % 8] |= (uint8_t)(at < 8 ? low : low << 4);
        field[96 + 8 + at % 4] |= (uint8_t)(high << (2 * (at / 4)));
    }
    for (uint32_t at = 0; at < 256; at++) {
        const uint32_t sub = at / 16, lane = at % 16;
        const float quantum = d * (float)(codes[sub] - 32u);
        const int quant = quantum == 0.0f ? 0 : (int)clamped(rounded(values[at] / quantum), -4.0f, 3.0f);
        const uint32_t half = sub / 8, j = sub % 8 / 2, second = sub % 2;
        field[32 + half * 32 + second * 16 + lane] |= (uint8_t)(((uint32_t)quant & 3u) << (2 * j));
        if (quant >= 0) field[second * 16 + lane] |= (uint8_t)(1u << (half * 4 + j));
    }
    put_half(field, 108, d);
}

// ggml.rs:352-392: sixteen sub-blocks of 16; factor = the largest magnitude / 32, the super scale
// = the largest factor / 127 (stored as a half while the single quantizes), signed byte multiples
// per sub-block, six-bit codes offset by 32.  `quantized` saturates below zero, so a negative
// number packs as code 32; this keeps the reference's bytes.
inline void q6_k(const float *values, uint8_t *field) {
    float factors[16], scale = 0.0f;
    for (int at = 0; at < 16; at++) {
        float size = 0.0f;
        for (int i = 0; i < 16; i++)
            if (size < std::fabs(values[at * 16 + i])) size = std::fabs(values[at * 16 + i]);
        factors[at] = size / 32.0f;
        scale = greatest(scale, std::fabs(factors[at]));
    }
    scale = scale / 127.0f;
    std::memset(field, 0, 210);
    put_half(field, 208, scale);
    for (int at = 0; at < 16; at++) {
        const int8_t code = scale == 0.0f ? (int8_t)0 : (int8_t)clamped(rounded(factors[at] / scale), -127.0f, 127.0f);
        field[192 + at] = (uint8_t)code;
        const float factor = scale * (float)code;
        for (int within = 0; within < 16; within++) {
            const int element = at * 16 + within, half = element / 128, group = element % 128 / 32, seat = element % 32;
            const uint32_t quant = quantized(values[element], factor, -32.0f, 31.0f) + 32u;
            put_nibble(field, half * 64 + (group % 2) * 32 + seat, group >= 2, quant);
            field[128 + half * 32 + seat] |= (uint8_t)(((quant >> 4) & 3u) << (2 * group));
        }
    }
}

inline void encode(Element element, const float *values, uint8_t *field) {
    switch (element) {
    case Element::Q8_0: return q8_0(values, field);
    case Element::Q3K: return q3_k(values, field);
    case Element::Q4K: return affine_block(element, values, field, 15);  // ggml.rs:295-297
    case Element::Q5K: return affine_block(element, values, field, 31);  // ggml.rs:291-293
    case Element::Q6K: return q6_k(values, field);
    default: panic("%s storage packs numbers a host quantizes by its element", neura::name(element));
    }
}

// the decoders: ggml.rs:218-223 (Q8_0), :291-309 (Q3_K), :311-350 (Q5_K, Q4_K), :394-408 (Q6_K)
inline void decode(Element element, const uint8_t *field, float *out) {
    switch (element) {
    case Element::Q8_0: {
        const float quantum = half_at(field, 0);
        for (int at = 0; at < 32; at++) out[at] = (float)(int8_t)field[2 + at] * quantum;
        return;
    }
    case Element::Q4K:
    case Element::Q5K: {
        const float scale = half_at(field, 0), min = half_at(field, 2);
        const bool five = element == Element::Q5K;
        for (int group = 0; group < 4; group++)
            for (int seat = 0; seat < 2; seat++) {
                uint32_t code, offset;
                scale_min_k4(field + 4, group * 2 + seat, code, offset);
                const float quantum = scale * (float)code, low = min * (float)offset;
                for (int within = 0; within < 32; within++) {
                    uint32_t quant = nibble_at(field[(five ? 48 : 16) + group * 32 + within], seat == 1);
                    if (five) quant |= (uint32_t)((field[16 + within] >> (2 * group + seat)) & 1u) << 4;
                    *out++ = quantum * (float)quant - low;
                }
            }
        return;
    }
    case Element::Q3K: {
        const float d = half_at(field, 108);
        for (uint32_t at = 0; at < 256; at++) {
            const uint32_t sub = at / 16, lane = at % 16, half = sub / 8, j = sub % 8 / 2, second = sub % 2;
            const uint8_t low_byte = field[96 + sub % 8], high_byte = field[96 + 8 + sub % 4];
            const uint32_t code = (sub < 8 ? low_byte & 0x0fu : low_byte >> 4) | (uint32_t)((high_byte >> (2 * (sub / 4))) & 3u) << 4;
            const int low = (field[32 + half * 32 + second * 16 + lane] >> (2 * j)) & 3;
            const bool high = (field[second * 16 + lane] & (1u << (half * 4 + j))) != 0;
            out[at] = d * ((float)(uint8_t)code - 32.0f) * (float)(low - (high ? 0 : 4));
        }
        return;
    }
    case Element::Q6K: {
        const float scale = half_at(field, 208);
        for (int seat = 0; seat < 2; seat++)
            for (int group = 0; group < 4; group++)
                for (int within = 0; within < 32; within++) {
                    const int8_t sub = (int8_t)field[192 + seat * 8 + group * 2 + within / 16];
                    const uint32_t quant = nibble_at(field[seat * 64 + (group % 2) * 32 + within], group >= 2) |
                                           (uint32_t)((field[128 + seat * 32 + within] >> (2 * group)) & 3u) << 4;
                    *out++ = scale * (float)sub * ((float)quant - 32.0f);
                }
        return;
    }
    default: panic("%s storage walks numbers a host reads by its element", neura::name(element));
    }
}

}  // namespace detail

// crates/neura-precision/src/lib.rs:5-24 and ggml.rs:8-20.  `quantum` only matters to the
// per-tensor integer formats, which no GGUF holds; it is kept so calls read like the reference's.
// A ragged last block is packed with zeros behind it, and the bytes end on a four-byte word.
inline std::vector<uint8_t> pack(Element element, float quantum, const float *values, size_t count) {
    (void)quantum;
    std::vector<uint8_t> bytes;
    if (element == Element::Single) {
        bytes.resize(count * 4);
        if (count) std::memcpy(bytes.data(), values, count * 4);
        return bytes;
    }
    if (element == Element::Half || element == Element::Bfloat16) {
        bytes.assign((count + 1) / 2 * 4, 0);
        for (size_t at = 0; at < count; at++) {
            const uint16_t bits = element == Element::Half ? half_bits(values[at]) : bfloat16_bits(values[at]);
            bytes[2 * at] = (uint8_t)bits, bytes[2 * at + 1] = (uint8_t)(bits >> 8);
        }
        return bytes;
    }
    const auto layout = block(element);
    NEURA_ASSERT(layout.has_value(), "%s storage packs numbers a host quantizes by its element", neura::name(element));
    const size_t blocks = (count + layout->elements - 1) / layout->elements;
    bytes.assign((blocks * layout->bytes + 3) / 4 * 4, 0);
    float held[256];
    for (size_t at = 0; at < blocks; at++) {
        const size_t first = at * layout->elements, lane = std::min<size_t>(layout->elements, count - first);
        std::fill(held, held + 256, 0.0f);
        std::copy(values + first, values + first + lane, held);
        detail::encode(element, held, bytes.data() + at * layout->bytes);
    }
    return bytes;
}
inline std::vector<uint8_t> pack(Element element, float quantum, const std::vector<float> &values) {
    return pack(element, quantum, values.data(), values.size());
}

// crates/neura-precision/src/lib.rs:26-68 and ggml.rs:22-38
inline std::vector<float> unpack(Element element, size_t elements, const uint8_t *bytes, size_t size) {
    const uint64_t held = (payload_bytes(element, elements) + 3) / 4 * 4;
    NEURA_ASSERT(size >= held, "unpacking %zu %s numbers out of %zu bytes where they pack %llu", elements, neura::name(element), size,
                 (unsigned long long)held);
    std::vector<float> values;
    if (element == Element::Single) {
        values.resize(elements);
        if (elements) std::memcpy(values.data(), bytes, elements * 4);
        return values;
    }
    if (element == Element::Half || element == Element::Bfloat16) {
        values.resize(elements);
        for (size_t at = 0; at < elements; at++) {
            const uint16_t bits = (uint16_t)(bytes[2 * at] | bytes[2 * at + 1] << 8);
            if (element == Element::Half) {
                values[at] = half_value(bits);
            } else {
                const uint32_t word = (uint32_t)bits << 16;
                std::memcpy(&values[at], &word, 4);
            }
        }
        return values;
    }
    const auto layout = block(element);
    NEURA_ASSERT(layout.has_value(), "%s storage walks numbers a host reads by its element", neura::name(element));
    const size_t blocks = (elements + layout->elements - 1) / layout->elements;
    values.resize(blocks * layout->elements);
    for (size_t at = 0; at < blocks; at++) detail::decode(element, bytes + at * layout->bytes, values.data() + at * layout->elements);
    values.resize(elements);
    return values;
}
inline std::vector<float> unpack(Element element, size_t elements, const std::vector<uint8_t> &bytes) {
    return unpack(element, elements, bytes.data(), bytes.size());
}

}  // namespace precision

// ---- neura-gguf (crates/neura-gguf/src/{value,metadata,header,lib}.rs) ------------------------

namespace gguf {

struct Value {
    enum Kind { Unsigned8, Signed8, Unsigned16, Signed16, Unsigned32, Signed32, Single, Flag, Text, Array, Unsigned64, Signed64, Double };
    Kind kind = Unsigned8;
    uint64_t bits = 0;  // integers (two's complement for signed), flag
    double real = 0.0;  // Single, Double
    std::string string;
    std::vector<Value> items;

    const char *name() const {
        static const char *names[] = {"u8", "i8", "u16", "i16", "u32", "i32", "f32", "bool", "string", "array", "u64", "i64", "f64"};
        return names[kind];
    }
    std::optional<std::string> text() const { return kind == Text ? std::optional<std::string>(string) : std::nullopt; }
    // whole numbers; signed ones travel as their two's complement (crates/neura-gguf/tests/gguf.rs:83-86)
    std::optional<uint64_t> integer() const {
        switch (kind) {
        case Unsigned8: case Signed8: case Unsigned16: case Signed16: case Unsigned32: case Signed32: case Unsigned64: case Signed64:
            return bits;
        default: return std::nullopt;
        }
    }
    std::optional<double> number() const {
        if (kind == Single || kind == Double) return real;
        if (auto held = integer()) {
            bool is_signed = kind == Signed8 || kind == Signed16 || kind == Signed32 || kind == Signed64;
            return is_signed ? (double)(int64_t)*held : (double)*held;
        }
        return std::nullopt;
    }
    std::optional<bool> flag() const { return kind == Flag ? std::optional<bool>(bits != 0) : std::nullopt; }
    const std::vector<Value> *array() const { return kind == Array ? &items : nullptr; }
};

struct Tensor {
    Element element;
    uint64_t elements;
    uint64_t shape[4];
    uint32_t rank;
    uint64_t at;
    uint64_t bytes;
    bool operator==(const Tensor &o) const {
        return element == o.element && elements == o.elements && rank == o.rank && at == o.at && bytes == o.bytes &&
               std::equal(shape, shape + 4, o.shape);
    }
};

class Metadata {
  public:
    explicit Metadata(const std::map<std::string, Value> *held) : held_(held) {}
    bool has(const std::string &key) const { return held_->count(key) != 0; }
    const Value &value(const std::string &key) const {
        auto found = held_->find(key);
        if (found == held_->end()) panic("this gguf holds no %s", key.c_str());
        return found->second;
    }
    std::string text(const std::string &key) const {
        auto held = value(key).text();
        if (!held) panic("the %s of this gguf is %s where a string stands", key.c_str(), value(key).name());
        return *held;
    }
    bool flag(const std::string &key) const {
        auto held = value(key).flag();
        if (!held) panic("the %s of this gguf is %s where a flag stands", key.c_str(), value(key).name());
        return *held;
    }
    uint32_t word(const std::string &key) const {
        auto held = value(key).integer();
        if (!held) panic("the %s of this gguf is %s where a whole number stands", key.c_str(), value(key).name());
        if (*held > 0xffffffffull) panic("the %s of this gguf holds %llu where a word holds what fits one", key.c_str(), (unsigned long long)*held);
        return (uint32_t)*held;
    }
    float single(const std::string &key) const {
        auto held = value(key).number();
        if (!held) panic("the %s of this gguf is %s where a number stands", key.c_str(), value(key).name());
        return (float)*held;
    }
    std::optional<uint32_t> optional_word(const std::string &key) const { return has(key) ? std::optional<uint32_t>(word(key)) : std::nullopt; }
    const std::vector<Value> &array(const std::string &key) const {
        auto held = value(key).array();
        if (!held) panic("the %s of this gguf is %s where an array stands", key.c_str(), value(key).name());
        return *held;
    }

  private:
    const std::map<std::string, Value> *held_;
};

// crates/neura-source/src/lib.rs:7-22
struct Placed {
    Element element;
    uint64_t elements;
    float scale;
    uint64_t payload_bytes, table_bytes;
};

using Sink = std::function<void(const uint8_t *, size_t)>;

class Source {
  public:
    virtual ~Source() = default;
    virtual std::optional<Placed> placed(const std::string &name) const = 0;
    virtual void payload(const std::string &name, const Sink &sink) const = 0;
    virtual void table(const std::string &name, const Sink &sink) const = 0;
};

// crates/neura-gguf/src/archive.rs:3-7
class Archive {
  public:
    virtual ~Archive() = default;
    virtual Metadata metadata() const = 0;
    virtual std::optional<Tensor> tensor(const std::string &name) const = 0;
};

namespace detail {

constexpr uint64_t DEFAULT_ALIGNMENT = 32;  // crates/neura-gguf/src/header.rs:6
constexpr size_t COPY_CHUNK = 1 << 16;      // crates/neura-gguf/src/lib.rs:20
constexpr size_t HEADER_STEP = 1 << 20;     // crates/neura-gguf/src/lib.rs:21

struct Truncated {};

struct Header {
    std::map<std::string, Value> metadata;
    std::vector<std::pair<std::string, Tensor>> tensors;
    uint64_t data = 0;
};

inline const char *type_name(uint32_t kind) {  // crates/neura-gguf/src/header.rs:164-204
    static const char *names[] = {"F32", "F16", "Q4_0", "Q4_1", "removed four bit", "removed four bit", "Q5_0", "Q5_1", "Q8_0", "Q8_1",
                                  "Q2_K", "Q3_K", "Q4_K", "Q5_K", "Q6_K", "Q8_K", "IQ2_XXS", "IQ2_XS", "IQ3_XXS", "IQ1_S", "IQ4_NL",
                                  "IQ3_S", "IQ2_S", "IQ4_XS", "I8", "I16", "I32", "I64", "F64", "IQ1_M", "BF16"};
    if (kind <= 30) return names[kind];
    if (kind <= 33 || (kind >= 36 && kind <= 38)) return "removed four bit plane";
    if (kind == 34) return "TQ1_0";
    if (kind == 35) return "TQ2_0";
    if (kind == 39) return "MXFP4";
    return "unknown";
}

inline std::optional<Element> type_element(uint32_t kind) {  // crates/neura-gguf/src/header.rs:150-162
    switch (kind) {
    case 0: return Element::Single;
    case 1: return Element::Half;
    case 8: return Element::Q8_0;
    case 11: return Element::Q3K;
    case 12: return Element::Q4K;
    case 13: return Element::Q5K;
    case 14: return Element::Q6K;
    case 30: return Element::Bfloat16;
    default: return std::nullopt;
    }
}

class Reader {  // crates/neura-gguf/src/header.rs:206-299
  public:
    Reader(const uint8_t *bytes, size_t size) : bytes_(bytes), size_(size) {}
    size_t at = 0;
    const uint8_t *take(size_t count) {
        if (count > size_ - at || at > size_) throw Truncated{};
        const uint8_t *held = bytes_ + at;
        at += count;
        return held;
    }
    template <typename T>
    T plain() {
        T out;
        memcpy(&out, take(sizeof(T)), sizeof(T));
        return out;
    }
    std::string text() {
        uint64_t length = plain<uint64_t>();
        if (length > size_) throw Truncated{};
        const uint8_t *held = take((size_t)length);
        return std::string(reinterpret_cast<const char *>(held), (size_t)length);
    }
    Value value(int depth) { return body(plain<uint32_t>(), depth); }
    Value body(uint32_t kind, int depth) {
        if (depth > 8) panic("this gguf nests arrays deeper than eight deep");
        Value v;
        switch (kind) {
        case 0: v.kind = Value::Unsigned8, v.bits = plain<uint8_t>(); break;
        case 1: v.kind = Value::Signed8, v.bits = (uint64_t)(int64_t)plain<int8_t>(); break;
        case 2: v.kind = Value::Unsigned16, v.bits = plain<uint16_t>(); break;
        case 3: v.kind = Value::Signed16, v.bits = (uint64_t)(int64_t)plain<int16_t>(); break;
        case 4: v.kind = Value::Unsigned32, v.bits = plain<uint32_t>(); break;
        case 5: v.kind = Value::Signed32, v.bits = (uint64_t)(int64_t)plain<int32_t>(); break;
        case 6: v.kind = Value::Single, v.real = plain<float>(); break;
        case 7: {
            uint8_t held = plain<uint8_t>();
            if (held > 1) panic("this gguf holds %u where a flag holds zero or one", held);
            v.kind = Value::Flag, v.bits = held;
            break;
        }
        case 8: v.kind = Value::Text, v.string = text(); break;
        case 9: {
            uint32_t held = plain<uint32_t>();
            uint64_t count = plain<uint64_t>();
            v.kind = Value::Array;
            for (uint64_t i = 0; i < count; i++) v.items.push_back(body(held, depth + 1));
            break;
        }
        case 10: v.kind = Value::Unsigned64, v.bits = plain<uint64_t>(); break;
        case 11: v.kind = Value::Signed64, v.bits = (uint64_t)plain<int64_t>(); break;
        case 12: v.kind = Value::Double, v.real = plain<double>(); break;
        default: panic("this gguf holds a metadata value of type %u, and a gguf declares thirteen of them", kind);
        }
        return v;
    }

  private:
    const uint8_t *bytes_;
    size_t size_;
};

// crates/neura-gguf/src/header.rs:43-148; throws Truncated when the bytes stop inside the header
inline Header parse(const uint8_t *bytes, size_t size) {
    Reader reader(bytes, size);
    const uint8_t *magic = reader.take(4);
    if (memcmp(magic, "GGUF", 4) != 0)
        panic("this file opens with [%02x, %02x, %02x, %02x] where a gguf opens with GGUF", magic[0], magic[1], magic[2], magic[3]);
    uint32_t version = reader.plain<uint32_t>();
    if (version != 2 && version != 3)
        panic("this gguf declares version %u, and this reader holds the versions [2, 3] whose layout it follows", version);
    uint64_t tensors = reader.plain<uint64_t>(), pairs = reader.plain<uint64_t>();
    Header header;
    for (uint64_t i = 0; i < pairs; i++) {
        std::string key = reader.text();
        Value value = reader.value(0);
        if (!header.metadata.emplace(key, std::move(value)).second) panic("two entries of this gguf carry the metadata key %s", key.c_str());
    }
    uint64_t alignment = DEFAULT_ALIGNMENT;
    auto declared = header.metadata.find("general.alignment");
    if (declared != header.metadata.end()) {
        auto held = declared->second.integer();
        if (!held) panic("this gguf measures its alignment by a value that is not an integer");
        alignment = *held;
    }
    if (alignment == 0 || alignment % 8 != 0)
        panic("this gguf aligns its tensors by %llu, and a gguf aligns them by a multiple of eight", (unsigned long long)alignment);
    for (uint64_t i = 0; i < tensors; i++) {
        std::string name = reader.text();
        uint32_t rank = reader.plain<uint32_t>();
        if (rank == 0 || rank > 4) panic("the tensor %s declares %u dimensions, and a gguf tensor carries one to four", name.c_str(), rank);
        Tensor tensor{};
        tensor.rank = rank;
        tensor.elements = 1;
        for (int d = 0; d < 4; d++) tensor.shape[d] = 1;
        for (uint32_t d = 0; d < rank; d++) {
            uint64_t held = reader.plain<uint64_t>();
            tensor.shape[d] = held;
            if (held != 0 && tensor.elements > UINT64_MAX / held) panic("the tensor %s spans more numbers than a gguf counts", name.c_str());
            tensor.elements *= held;
        }
        uint32_t kind = reader.plain<uint32_t>();
        tensor.at = reader.plain<uint64_t>();
        if (tensor.at % alignment != 0)
            panic("the tensor %s begins at byte %llu of the tensor data, and a gguf aligns it by %llu", name.c_str(),
                  (unsigned long long)tensor.at, (unsigned long long)alignment);
        auto element = type_element(kind);
        if (!element)
            panic("the tensor %s holds numbers of ggml type %u (%s), which this framework does not read", name.c_str(), kind, type_name(kind));
        tensor.element = *element;
        if (auto held = block(*element)) {
            if (tensor.elements % held->elements != 0)
                panic("the tensor %s holds %llu numbers of %s storage, and a %s block packs %u of them", name.c_str(),
                      (unsigned long long)tensor.elements, neura::name(*element), neura::name(*element), held->elements);
            tensor.bytes = tensor.elements / held->elements * held->bytes;
        } else {
            uint64_t bits = 0;
            if (__builtin_mul_overflow(tensor.elements, (uint64_t)bits_per_element(*element), &bits))
                panic("the tensor %s spans more bytes than a gguf counts", name.c_str());
            tensor.bytes = bits / 8;
        }
        header.tensors.emplace_back(std::move(name), tensor);
    }
    header.data = (reader.at + alignment - 1) / alignment * alignment;
    return header;
}

inline void bounds(const Header &header, uint64_t held, const std::string &what) {  // crates/neura-gguf/src/lib.rs:225-233
    for (auto &entry : header.tensors) {
        // checked sums: an offset near 2^64 must not wrap to an end inside the file
        uint64_t start = 0, end = 0;
        const bool wraps = __builtin_add_overflow(header.data, entry.second.at, &start) || __builtin_add_overflow(start, entry.second.bytes, &end);
        if (wraps || end > held)
            panic("%s holds %llu bytes where the tensor %s runs to byte %llu", what.c_str(), (unsigned long long)held, entry.first.c_str(),
                  (unsigned long long)(wraps ? UINT64_MAX : end));
    }
}

inline std::unordered_map<std::string, size_t> index_of(const Header &header) {  // crates/neura-gguf/src/lib.rs:235-244
    std::unordered_map<std::string, size_t> index;
    for (size_t at = 0; at < header.tensors.size(); at++)
        if (!index.emplace(header.tensors[at].first, at).second)
            panic("two tensors of one gguf carry the name %s, and a name identifies one tensor", header.tensors[at].first.c_str());
    return index;
}

inline Placed placed_of(const Tensor &tensor) { return Placed{tensor.element, tensor.elements, 1.0f, tensor.bytes, 0}; }

}  // namespace detail

// A whole GGUF held in memory (crates/neura-gguf/src/lib.rs:23-91)
class Gguf : public Source, public Archive {
  public:
    static Gguf decode(const uint8_t *bytes, size_t size) {
        Gguf out;
        try {
            out.header_ = detail::parse(bytes, size);
        } catch (const detail::Truncated &) {
            panic("a gguf header runs past the bytes this file holds, and a gguf opens with its metadata and its tensor table");
        }
        detail::bounds(out.header_, size, "a gguf");
        out.index_ = detail::index_of(out.header_);
        out.bytes_.assign(bytes, bytes + size);
        return out;
    }
    static Gguf decode(const std::vector<uint8_t> &bytes) { return decode(bytes.data(), bytes.size()); }

    const std::vector<uint8_t> &bytes() const { return bytes_; }
    Metadata metadata() const override { return Metadata(&header_.metadata); }
    const Value *value(const std::string &key) const {
        auto found = header_.metadata.find(key);
        return found == header_.metadata.end() ? nullptr : &found->second;
    }
    size_t tensors() const { return header_.tensors.size(); }
    std::vector<std::string> names() const {
        std::vector<std::string> out;
        for (auto &entry : header_.tensors) out.push_back(entry.first);
        return out;
    }
    std::optional<Tensor> tensor(const std::string &name) const override {
        auto found = index_.find(name);
        if (found == index_.end()) return std::nullopt;
        return header_.tensors[found->second].second;
    }
    uint64_t data() const { return header_.data; }

    std::optional<Placed> placed(const std::string &name) const override {
        auto held = tensor(name);
        return held ? std::optional<Placed>(detail::placed_of(*held)) : std::nullopt;
    }
    void payload(const std::string &name, const Sink &sink) const override {
        auto held = tensor(name);
        if (!held) panic("this gguf holds no tensor named %s", name.c_str());
        size_t start = (size_t)(header_.data + held->at), left = (size_t)held->bytes;
        while (left) {
            size_t take = std::min(left, detail::COPY_CHUNK);
            sink(bytes_.data() + start, take);
            start += take, left -= take;
        }
    }
    void table(const std::string &name, const Sink &) const override {
        if (!index_.count(name)) panic("this gguf holds no tensor named %s", name.c_str());
    }

  private:
    std::vector<uint8_t> bytes_;
    detail::Header header_;
    std::unordered_map<std::string, size_t> index_;
};

// A GGUF read from a file: the header only, payloads streamed on demand
// (crates/neura-gguf/src/lib.rs:93-213)
class GgufFile : public Source, public Archive {
  public:
    static std::unique_ptr<GgufFile> open(const std::string &path) {
        std::unique_ptr<GgufFile> out(new GgufFile());
        out->path_ = path;
        out->file_.open(path, std::ios::binary);
        if (!out->file_) panic("a gguf at %s could not be opened: no such file or no access", path.c_str());
        out->file_.seekg(0, std::ios::end);
        uint64_t len = (uint64_t)out->file_.tellg();
        size_t held = std::min<uint64_t>(detail::HEADER_STEP, std::max<uint64_t>(len, 1));
        for (;;) {
            std::vector<uint8_t> bytes(held);
            out->read_at(0, bytes.data(), bytes.size());
            try {
                out->header_ = detail::parse(bytes.data(), bytes.size());
                break;
            } catch (const detail::Truncated &) {
                if (held >= len)
                    panic("a gguf at %s holds %llu bytes where its metadata and its tensor table run past them, and a header closes before the first tensor of a gguf",
                          path.c_str(), (unsigned long long)len);
                held = (size_t)std::min<uint64_t>((uint64_t)held * 2, len);
            } catch (const Panic &refused) {
                panic("a gguf at %s holds %s", path.c_str(), refused.what());
            }
        }
        detail::bounds(out->header_, len, "a gguf at " + path);
        out->index_ = detail::index_of(out->header_);
        return out;
    }
    uint64_t reads() const { return reads_; }
    const std::string &path() const { return path_; }
    Metadata metadata() const override { return Metadata(&header_.metadata); }
    size_t tensors() const { return header_.tensors.size(); }
    std::optional<Tensor> tensor(const std::string &name) const override {
        auto found = index_.find(name);
        if (found == index_.end()) return std::nullopt;
        return header_.tensors[found->second].second;
    }
    std::optional<Placed> placed(const std::string &name) const override {
        auto held = tensor(name);
        return held ? std::optional<Placed>(detail::placed_of(*held)) : std::nullopt;
    }
    void payload(const std::string &name, const Sink &sink) const override {
        auto held = tensor(name);
        if (!held) panic("this gguf holds no tensor named %s", name.c_str());
        uint64_t at = header_.data + held->at, left = held->bytes;
        std::vector<uint8_t> chunk;
        while (left) {
            size_t take = (size_t)std::min<uint64_t>(left, detail::COPY_CHUNK);
            chunk.resize(take);
            read_at(at, chunk.data(), take);
            reads_++;
            sink(chunk.data(), take);
            at += take, left -= take;
        }
    }
    void table(const std::string &name, const Sink &) const override {
        if (!index_.count(name)) panic("this gguf holds no tensor named %s", name.c_str());
    }

  private:
    GgufFile() = default;
    void read_at(uint64_t at, uint8_t *bytes, size_t count) const {
        file_.clear();
        file_.seekg((std::streamoff)at);
        file_.read(reinterpret_cast<char *>(bytes), (std::streamsize)count);
        if ((size_t)file_.gcount() != count) panic("a gguf at %s could not be read at %llu: the file ends early", path_.c_str(), (unsigned long long)at);
    }
    mutable std::ifstream file_;
    std::string path_;
    detail::Header header_;
    std::unordered_map<std::string, size_t> index_;
    mutable uint64_t reads_ = 0;
};

// Writes a GGUF v3 (the layout of the reference's fixture builder, crates/neura-gguf/tests/support/mod.rs:21-64)
class Writer {
  public:
    explicit Writer(uint64_t alignment = 32) : alignment_(alignment) {}
    void meta_u32(const std::string &key, uint32_t value) { key_kind(key, 4), put(value); }
    void meta_f32(const std::string &key, float value) { key_kind(key, 6), put(value); }
    void meta_text(const std::string &key, const std::string &value) { key_kind(key, 8), text(meta_, value); }
    void tensor(const std::string &name, Element element, const std::vector<uint64_t> &shape, const uint8_t *payload, size_t bytes) {
        tensors_.push_back({name, (uint32_t)element, shape, std::vector<uint8_t>(payload, payload + bytes)});
    }
    std::vector<uint8_t> bytes() const {
        std::vector<uint8_t> out;
        out.insert(out.end(), {'G', 'G', 'U', 'F'});
        append(out, (uint32_t)3), append(out, (uint64_t)tensors_.size()), append(out, (uint64_t)pairs_);
        out.insert(out.end(), meta_.begin(), meta_.end());
        uint64_t cursor = 0;
        for (auto &t : tensors_) {
            text(out, t.name);
            append(out, (uint32_t)t.shape.size());
            for (uint64_t dim : t.shape) append(out, dim);
            append(out, t.kind), append(out, cursor);
            cursor = (cursor + t.payload.size() + alignment_ - 1) / alignment_ * alignment_;
        }
        while (out.size() % alignment_) out.push_back(0);
        for (auto &t : tensors_) {
            out.insert(out.end(), t.payload.begin(), t.payload.end());
            while (out.size() % alignment_) out.push_back(0);
        }
        return out;
    }

  private:
    struct Held {
        std::string name;
        uint32_t kind;
        std::vector<uint64_t> shape;
        std::vector<uint8_t> payload;
    };
    template <typename T>
    static void append(std::vector<uint8_t> &out, T value) {
        const uint8_t *raw = reinterpret_cast<const uint8_t *>(&value);
        out.insert(out.end(), raw, raw + sizeof(T));
    }
    static void text(std::vector<uint8_t> &out, const std::string &held) {
        append(out, (uint64_t)held.size());
        out.insert(out.end(), held.begin(), held.end());
    }
    void key_kind(const std::string &key, uint32_t kind) { text(meta_, key), append(meta_, kind), pairs_++; }
    template <typename T>
    void put(T value) { append(meta_, value); }
    uint64_t alignment_;
    uint64_t pairs_ = 0;
    std::vector<uint8_t> meta_;
    std::vector<Held> tensors_;
};

}  // namespace gguf

// ---- neura-runtime: the device and the weight arena ------------------------------------------

namespace runtime {

inline void check(int32_t status) {
    if (status != NH_OK) panic("%s", nh_last_error());
}

// Runtime::open (crates/neura-runtime/src/runtime.rs:183): the only error VALUE of the reference
// is GpuUnavailable at open; here open throws Panic carrying the library's message.
class Runtime {
  public:
    explicit Runtime(int32_t index = 0) : device_(nh_open(index)) {
        if (!device_) panic("%s", nh_last_error());
    }
    ~Runtime() { nh_close(device_); }
    Runtime(const Runtime &) = delete;
    Runtime &operator=(const Runtime &) = delete;
    nh_device *device() const { return device_; }

  private:
    nh_device *device_;
};

// Runtime::load (crates/neura-runtime/src/runtime.rs:356-367): every named tensor of a Source
// poured verbatim into one arena at 256-byte aligned starts (crates/neura-plan/src/layout.rs:29-36)
class Weights {
  public:
    Weights(const Runtime &runtime, const gguf::Source &source, const std::vector<std::string> &names) {
        uint64_t total = 0;
        for (auto &name : names) {
            auto placed = source.placed(name);
            if (!placed) panic("this gguf holds no tensor named %s", name.c_str());
            offsets_[name] = total;
            placed_.emplace(name, *placed);
            total += (placed->payload_bytes + 255) / 256 * 256;
        }
        arena_ = nh_weights_create(runtime.device(), (size_t)std::max<uint64_t>(total, 256));
        if (!arena_) panic("%s", nh_last_error());
        for (auto &name : names) {
            uint64_t at = offsets_[name];
            source.payload(name, [&](const uint8_t *chunk, size_t bytes) {
                check(nh_weights_put(arena_, (size_t)at, chunk, bytes));
                at += bytes;
            });
        }
    }
    ~Weights() { nh_weights_destroy(arena_); }
    Weights(const Weights &) = delete;
    Weights &operator=(const Weights &) = delete;
    nh_weights *arena() const { return arena_; }
    uint64_t offset(const std::string &name) const {
        auto found = offsets_.find(name);
        if (found == offsets_.end()) panic("this store holds no tensor named %s", name.c_str());
        return found->second;
    }
    const gguf::Placed &placed(const std::string &name) const { return placed_.at(name); }

  private:
    nh_weights *arena_ = nullptr;
    std::map<std::string, uint64_t> offsets_;
    std::map<std::string, gguf::Placed> placed_;
};

}  // namespace runtime

// ---- neura-decoder: declarations and the KV cache ---------------------------------------------

namespace decoder {

struct Parameter {
    std::string name;
    uint32_t rows, columns;
    Element element;
};

// crates/neura-decoder/src/parameter.rs:5-15: GGUF dim0 = columns (contiguous), dim1 = rows
inline Parameter matrix(const gguf::Archive &source, const std::string &name, uint32_t rows, uint32_t columns) {
    auto held = source.tensor(name);
    if (!held) panic("this gguf holds no tensor named %s", name.c_str());
    if (!(held->rank == 2 && held->shape[0] == columns && held->shape[1] == rows))
        panic("the tensor %s of this gguf walks %u dimensions of [%llu, %llu, %llu, %llu] where %u rows of %u numbers walk [1, 1, %u, %u]", name.c_str(),
              held->rank, (unsigned long long)held->shape[0], (unsigned long long)held->shape[1], (unsigned long long)held->shape[2],
              (unsigned long long)held->shape[3], rows, columns, rows, columns);
    return Parameter{name, rows, columns, held->element};
}

// crates/neura-decoder/src/parameter.rs:17-27
inline Parameter vector(const gguf::Archive &source, const std::string &name, uint32_t width) {
    auto held = source.tensor(name);
    if (!held) panic("this gguf holds no tensor named %s", name.c_str());
    if (!(held->rank == 1 && held->shape[0] == width))
        panic("the tensor %s of this gguf walks %u dimensions of [%llu, %llu, %llu, %llu] where %u numbers walk [1, 1, 1, %u]", name.c_str(), held->rank,
              (unsigned long long)held->shape[0], (unsigned long long)held->shape[1], (unsigned long long)held->shape[2],
              (unsigned long long)held->shape[3], width, width);
    return Parameter{name, 1, width, held->element};
}

// crates/neura-decoder/src/cache.rs:19-39
struct CacheShape {
    uint32_t heads, width, capacity, window, batch, rows;
    CacheShape(uint32_t heads, uint32_t width, uint32_t capacity, uint32_t window, uint32_t batch, uint32_t rows)
        : heads(heads), width(width), capacity(capacity), window(window), batch(batch), rows(rows) {}
};

// An fp16 KV cache of one layer with the reference's write / attend / reset surface
// (crates/neura-decoder/src/cache.rs:63-65, :92-195, :223-250, :267-352, :366-406); eager: each
// call enqueues the kernels on the runtime's stream.
class Cache {
  public:
    // the constructor's refusals, callable without a device
    static void validate(const std::string &name, const CacheShape &shape, Element element) {
        NEURA_ASSERT(!name.empty(), "a cache names the state it keeps so a checkpoint can hold it");
        NEURA_ASSERT(shape.heads > 0 && shape.width > 0 && shape.batch > 0, "a cache of %u planes of %u heads of %u numbers holds no key",
                     shape.batch, shape.heads, shape.width);
        NEURA_ASSERT(shape.capacity > 0, "a cache of %u positions holds no key", shape.capacity);
        NEURA_ASSERT(shape.window > 0 && shape.window <= shape.capacity, "a cache of %u positions keeps a window of %u positions",
                     shape.capacity, shape.window);
        NEURA_ASSERT(shape.rows > 0 && shape.rows <= shape.window,
                     "a cache of a %u position window takes %u rows at a time, and a chunk of more rows than the window holds walks past the slots it fills",
                     shape.window, shape.rows);
        NEURA_ASSERT(element == Element::Single || element == Element::Half || element == Element::Bfloat16,
                     "a cache holds keys and values in single, half or bfloat16 storage, and %s storage carries another grid", neura::name(element));
    }
    // bytes of one key or value number, and the element as the C ABI names it
    static size_t width_of(Element element) { return element == Element::Single ? 4 : 2; }
    static int32_t abi(Element element) { return element == Element::Single ? NH_F32 : element == Element::Bfloat16 ? NH_BF16 : NH_F16; }
    Cache(const runtime::Runtime &runtime, const std::string &name, CacheShape shape, Element element = Element::Half, bool ring = false)
        : device_(runtime.device()), name_(name), shape_(shape), ring_(ring), element_(element) {
        validate(name, shape, element);
        size_t bytes = (size_t)shape.heads * shape.batch * shape.capacity * shape.width * width_of(element);
        keys_ = static_cast<uint8_t *>(nh_alloc(device_, bytes));
        values_ = static_cast<uint8_t *>(nh_alloc(device_, bytes));
        if (!keys_ || !values_) panic("%s", nh_last_error());
    }
    ~Cache() {
        nh_free(device_, keys_);
        nh_free(device_, values_);
    }
    Cache(const Cache &) = delete;
    Cache &operator=(const Cache &) = delete;

    // crates/neura-decoder/src/cache.rs:67-69: the window is a ring -- position p is written to slot p mod window and a
    // query weighs the last `window` positions
    static std::unique_ptr<Cache> windowed(const runtime::Runtime &runtime, const std::string &name, CacheShape shape, Element element = Element::Half) {
        return std::make_unique<Cache>(runtime, name, shape, element, true);
    }
    uint32_t rows() const { return shape_.rows; }
    uint32_t batch() const { return shape_.batch; }
    uint32_t window() const { return shape_.window; }
    bool ring() const { return ring_; }
    Element element() const { return element_; }  // cache.rs:219-221
    std::pair<void *, void *> states() const { return {keys_, values_}; }  // "{name}.key", "{name}.value", numbers of element()
    std::string key_name() const { return name_ + ".key"; }
    std::string value_name() const { return name_ + ".value"; }

    // keys / values: device fp32 [heads][batch][rows][width]; cursor: device u32 [batch]
    void write(const uint32_t *cursor, const float *keys, const float *values) { store(cursor, keys, values, nullptr); }
    void write_masked(const uint32_t *cursor, const float *keys, const float *values, const uint8_t *active) {
        NEURA_ASSERT(shape_.rows <= shape_.capacity - shape_.window,
                     "a cache of %u positions keeps a %u position window, and a masked chunk of %u rows holds only %u scratch rows", shape_.capacity,
                     shape_.window, shape_.rows, shape_.capacity - shape_.window);
        store(cursor, keys, values, active);
    }
    // query / out: device fp32 [query_heads][batch][rows][width]
    void attend(const float *query, uint32_t query_heads, const uint32_t *cursor, float scale, float *out) {
        NEURA_ASSERT(query_heads % shape_.heads == 0,
                     "a query of %u heads reads a cache of %u key heads, and every key head serves a whole group of queries", query_heads, shape_.heads);
        runtime::check(nh_attention_element(device_, query, keys_, values_, query_heads, shape_.heads, shape_.batch, shape_.rows, shape_.width,
                                            shape_.capacity, shape_.window, ring_ ? shape_.window : 0u, cursor, scale, out, abi(element_)));
    }
    // reset: host flags, one per plane; a set flag zeroes the plane's keys and values
    void reset(const std::vector<uint8_t> &reset) {
        NEURA_ASSERT(reset.size() == shape_.batch, "a cache of %u planes resets by %zu flags", shape_.batch, reset.size());
        size_t plane = (size_t)shape_.capacity * shape_.width;
        for (uint32_t head = 0; head < shape_.heads; head++)
            for (uint32_t b = 0; b < shape_.batch; b++)
                if (reset[b]) {
                    size_t at = ((size_t)head * shape_.batch + b) * plane * width_of(element_);
                    runtime::check(nh_clear(device_, keys_ + at, plane * width_of(element_)));
                    runtime::check(nh_clear(device_, values_ + at, plane * width_of(element_)));
                }
    }

  private:
    void store(const uint32_t *cursor, const float *keys, const float *values, const uint8_t *active) {
        runtime::check(nh_cache_write_element(device_, keys, values, keys_, values_, shape_.heads, shape_.batch, shape_.rows, shape_.width,
                                              shape_.capacity, shape_.window, cursor, active, ring_ ? 1 : 0, abi(element_)));
    }
    nh_device *device_;
    std::string name_;
    CacheShape shape_;
    bool ring_ = false;
    Element element_ = Element::Half;
    uint8_t *keys_ = nullptr, *values_ = nullptr;
};

}  // namespace decoder

// ---- the Qwen2-style decoder and neura-generate ------------------------------------------------

namespace generate {

// examples/qwen/config.rs:21-60 for the qwen2 architecture keys
struct Config {
    uint32_t layers, hidden, feed_forward, heads, key_heads, head_width, vocabulary, context;
    float rope_base, floor;
    static Config read(const gguf::Metadata &metadata, uint32_t vocabulary) {
        std::string arch = metadata.text("general.architecture");
        NEURA_ASSERT(arch == "qwen2",
                     "this model weighs the tensors of the qwen2 architecture, and this gguf names %s as its general.architecture", arch.c_str());
        auto key = [&](const char *suffix) { return arch + "." + suffix; };
        Config c;
        c.layers = metadata.word(key("block_count"));
        c.hidden = metadata.word(key("embedding_length"));
        c.feed_forward = metadata.word(key("feed_forward_length"));
        c.heads = metadata.word(key("attention.head_count"));
        c.key_heads = metadata.word(key("attention.head_count_kv"));
        c.head_width = metadata.optional_word(key("attention.key_length")).value_or(c.hidden / c.heads);
        c.rope_base = metadata.single(key("rope.freq_base"));
        c.context = metadata.word(key("context_length"));
        c.floor = metadata.single(key("attention.layer_norm_rms_epsilon"));
        c.vocabulary = vocabulary;
        return c;
    }
};

// crates/neura-generate/src/batch.rs:110-153 (tuning is not built: there is no compiler to tune)
// crates/neura-generate/src/sampling.rs:3-57: a batch answers with the largest logit, or draws among the `keep` largest
// cut at a cumulative mass after dividing the logits by a temperature
struct Sampling {
    bool greedy = true;
    float temperature = 1.0f;
    uint32_t keep = 1;
    float cumulative = 1.0f;
    static constexpr uint32_t CANDIDATES = 64;  // crates/neura-abi/src/lib.rs:39
    static Sampling sampled(float temperature, uint32_t keep, float cumulative) {
        check_temperature(temperature);
        NEURA_ASSERT(keep >= 1 && keep <= CANDIDATES, "a sample keeps %u candidates where a row holds between one and %u", keep, CANDIDATES);
        check_cumulative(cumulative);
        Sampling out;
        out.greedy = false, out.temperature = temperature, out.keep = keep, out.cumulative = cumulative;
        return out;
    }
    static void check_temperature(float value) {
        NEURA_ASSERT(value > 0.0f && std::isfinite(value), "a sampling temperature of %g spreads no logits", (double)value);
    }
    static void check_cumulative(float value) {
        NEURA_ASSERT(value > 0.0f && value <= 1.0f, "a cumulative mass of %g keeps no candidate or names more than every candidate", (double)value);
    }
};

struct BatchSpec {
    uint32_t context, batch;
    std::vector<uint32_t> chunks;
    Sampling sampling;
    std::optional<uint32_t> window_tokens;  // BatchSpec::window: the caches are rings of that many tokens
    bool shares = false;                    // BatchSpec::shared: the planes can start from one prefix fed once
    BatchSpec shared() const {              // crates/neura-generate/src/batch.rs:143-146
        BatchSpec out = *this;
        out.shares = true;
        return out;
    }
    BatchSpec(uint32_t context, uint32_t batch, std::vector<uint32_t> chunks) : context(context), batch(batch), chunks(std::move(chunks)) {}
    BatchSpec window(uint32_t tokens) const {  // crates/neura-generate/src/batch.rs:148-152
        NEURA_ASSERT(tokens > 0, "a batch keeps a window of no token");
        BatchSpec out = *this;
        out.window_tokens = tokens;
        return out;
    }
    BatchSpec sampled(Sampling held) const {  // crates/neura-generate/src/batch.rs:133-136
        BatchSpec out = *this;
        out.sampling = held;
        return out;
    }
};

struct Emitted {  // crates/neura-generate/src/batch.rs:155-159
    uint32_t slot, token;
    bool operator==(const Emitted &o) const { return slot == o.slot && token == o.token; }
};

// The decoder of one GGUF on one device: weights poured into an arena, nh_model above them.
class Model {
  public:
    // `cache`: what the key and value states hold (the element the model function hands Cache::new, examples/qwen/main.rs:107,
    // attention.rs:77-83): Half unless the caller names Single or Bfloat16
    Model(const runtime::Runtime &runtime, const gguf::Archive &archive, const gguf::Source &source, const Config &config, const BatchSpec &spec,
          Element cache = Element::Half)
        : config_(config), cache_(cache) {
        NEURA_ASSERT(cache == Element::Single || cache == Element::Half || cache == Element::Bfloat16,
                     "a cache holds keys and values in single, half or bfloat16 storage, and %s storage carries another grid", neura::name(cache));
        const uint32_t H = config.hidden, QW = config.heads * config.head_width, KW = config.key_heads * config.head_width, F = config.feed_forward;
        std::vector<std::string> names;
        // tensor names of a Qwen2 GGUF (the reference's qwen35 example names them alike, examples/qwen/attention.rs:40-78, mlp.rs:22-25)
        // every matrix keeps the storage the file gives it (a Q4_K_M file mixes q4_k and q6_k, a Q3_K_M file q3_k, q4_k and q5_k); the q, k and v projections of
        // Qwen2 checkpoints carry biases the reference's own example has no tensors for
        Element element = decoder::matrix(archive, "token_embd.weight", config.vocabulary, H).element;
        std::vector<int32_t> elements;
        auto declare = [&](const decoder::Parameter &parameter) {
            if (parameter.rows == 1) {
                NEURA_ASSERT(parameter.element == Element::Single, "this decoder reads norm weights and biases in single storage, and %s holds %s storage",
                             parameter.name.c_str(), name(parameter.element));
            } else {
                NEURA_ASSERT(parameter.element == Element::Q8_0 || parameter.element == Element::Q3K || parameter.element == Element::Q4K ||
                                 parameter.element == Element::Q5K || parameter.element == Element::Q6K,
                             "this decoder multiplies q8_0, q3_k, q4_k, q5_k and q6_k matrices, and %s holds %s storage", parameter.name.c_str(),
                             name(parameter.element));
                elements.push_back((int32_t)parameter.element);
            }
            names.push_back(parameter.name);
            return parameter;
        };
        declare(decoder::matrix(archive, "token_embd.weight", config.vocabulary, H));
        bool separate_head = archive.tensor("output.weight").has_value();
        if (separate_head)
            declare(decoder::matrix(archive, "output.weight", config.vocabulary, H));
        else
            elements.push_back((int32_t)element);
        declare(decoder::vector(archive, "output_norm.weight", H));
        std::vector<uint64_t> biases[3];
        for (uint32_t layer = 0; layer < config.layers; layer++) {
            auto at = [&](const char *suffix) { return "blk." + std::to_string(layer) + "." + suffix; };
            declare(decoder::matrix(archive, at("attn_q.weight"), QW, H));
            declare(decoder::matrix(archive, at("attn_k.weight"), KW, H));
            declare(decoder::matrix(archive, at("attn_v.weight"), KW, H));
            declare(decoder::matrix(archive, at("attn_output.weight"), H, QW));
            declare(decoder::matrix(archive, at("ffn_gate.weight"), F, H));
            declare(decoder::matrix(archive, at("ffn_up.weight"), F, H));
            declare(decoder::matrix(archive, at("ffn_down.weight"), H, F));
            declare(decoder::vector(archive, at("attn_norm.weight"), H));
            declare(decoder::vector(archive, at("ffn_norm.weight"), H));
            const char *projections[3] = {"attn_q.bias", "attn_k.bias", "attn_v.bias"};
            const uint32_t widths[3] = {QW, KW, KW};
            for (int s = 0; s < 3; s++)
                if (archive.tensor(at(projections[s])).has_value()) declare(decoder::vector(archive, at(projections[s]), widths[s]));
        }
        weights_ = std::make_unique<runtime::Weights>(runtime, source, names);
        std::vector<uint64_t> columns[9];
        const char *suffixes[9] = {"attn_norm", "attn_q", "attn_k", "attn_v", "attn_output", "ffn_norm", "ffn_gate", "ffn_up", "ffn_down"};
        for (uint32_t layer = 0; layer < config.layers; layer++)
            for (int s = 0; s < 9; s++) columns[s].push_back(weights_->offset("blk." + std::to_string(layer) + "." + suffixes[s] + ".weight"));
        for (uint32_t layer = 0; layer < config.layers; layer++) {
            const char *projections[3] = {"attn_q.bias", "attn_k.bias", "attn_v.bias"};
            for (int s = 0; s < 3; s++) {
                const std::string bias = "blk." + std::to_string(layer) + "." + projections[s];
                biases[s].push_back(archive.tensor(bias).has_value() ? weights_->offset(bias) : UINT64_MAX);
            }
        }
        nh_tensor_table table{};
        table.matrix_element = (int32_t)element;
        table.matrix_elements = elements.data();
        table.attn_q_bias = biases[0].data(), table.attn_k_bias = biases[1].data(), table.attn_v_bias = biases[2].data();
        table.token_embd = weights_->offset("token_embd.weight");
        table.output = separate_head ? weights_->offset("output.weight") : UINT64_MAX;
        table.output_norm = weights_->offset("output_norm.weight");
        table.attn_norm = columns[0].data(), table.attn_q = columns[1].data(), table.attn_k = columns[2].data(), table.attn_v = columns[3].data();
        table.attn_output = columns[4].data(), table.ffn_norm = columns[5].data(), table.ffn_gate = columns[6].data();
        table.ffn_up = columns[7].data(), table.ffn_down = columns[8].data();
        nh_model_config c{};
        c.layers = config.layers, c.hidden = H, c.heads = config.heads, c.kv_heads = config.key_heads, c.head_dim = config.head_width;
        c.ffn = F, c.vocab = config.vocabulary, c.context = spec.context, c.batch = spec.batch;
        c.max_rows = spec.chunks.empty() ? 1 : spec.chunks.front();
        c.window = spec.window_tokens.value_or(0);
        c.rope_base = config.rope_base, c.eps = config.floor;
        c.cache_element = decoder::Cache::abi(cache);
        model_ = nh_model_create(runtime.device(), &c, weights_->arena(), &table);
        if (!model_) panic("%s", nh_last_error());
    }
    ~Model() { nh_model_destroy(model_); }
    Model(const Model &) = delete;
    Model &operator=(const Model &) = delete;
    nh_model *handle() const { return model_; }
    const Config &config() const { return config_; }
    Element cache_element() const { return cache_; }

  private:
    Config config_;
    Element cache_ = Element::Half;
    std::unique_ptr<runtime::Weights> weights_;
    nh_model *model_ = nullptr;
};

// crates/neura-generate/src/snapshot.rs: what a batch holds between steps on the host -- planes, cursors, phases,
// seeds and draw settings -- and its wire format "NBS1": little-endian words, counted lists, floats by their bits.
struct SlotSnapshot {
    uint32_t cursor;
    uint32_t phase;  // 1 prompting (prompt tokens follow), 2 generating (the token to feed follows), 3 suspended
    std::vector<uint32_t> prompt;
    uint32_t feed;
};

struct BatchSnapshot {
    uint32_t batch = 0, context = 0, window = 0;
    bool sampled = false;
    std::optional<std::vector<uint32_t>> prefix;
    std::vector<std::optional<SlotSnapshot>> slots;
    std::vector<uint32_t> seeds;
    std::vector<float> temperatures, keeps, cumulatives;
    std::vector<std::string> state_names;
    std::vector<std::vector<float>> states;

    std::vector<uint8_t> to_bytes() const {  // snapshot.rs:47-130
        std::vector<uint8_t> bytes{'N', 'B', 'S', '1'};
        auto word = [&](uint32_t value) {
            for (int k = 0; k < 4; k++) bytes.push_back((uint8_t)(value >> (8 * k)));
        };
        auto words = [&](const std::vector<uint32_t> &values) {
            word((uint32_t)values.size());
            for (uint32_t value : values) word(value);
        };
        auto floats = [&](const std::vector<float> &values) {
            word((uint32_t)values.size());
            for (float value : values) {
                uint32_t bits;
                memcpy(&bits, &value, 4);
                word(bits);
            }
        };
        word(batch), word(context), word(window), word(sampled ? 1 : 0);
        if (prefix) word(1), words(*prefix);
        else word(0);
        word((uint32_t)slots.size());
        for (const auto &slot : slots) {
            if (!slot) {
                word(0);
                continue;
            }
            word(slot->phase), word(slot->cursor);
            if (slot->phase == 1) words(slot->prompt);
            else if (slot->phase == 2) word(slot->feed);
        }
        words(seeds);
        floats(temperatures), floats(keeps), floats(cumulatives);
        word((uint32_t)state_names.size());
        for (const std::string &name : state_names) {
            word((uint32_t)name.size());
            bytes.insert(bytes.end(), name.begin(), name.end());
        }
        word((uint32_t)states.size());
        for (const auto &values : states) floats(values);
        return bytes;
    }

    static BatchSnapshot from_bytes(const std::vector<uint8_t> &bytes) {  // snapshot.rs:132-236
        size_t at = 0;
        auto take = [&](size_t count) {
            NEURA_ASSERT(count <= bytes.size() - at, "a snapshot holds %zu bytes where its reader asks for %zu", bytes.size(), at + count);
            const uint8_t *held = bytes.data() + at;
            at += count;
            return held;
        };
        auto word = [&]() {
            const uint8_t *held = take(4);
            return (uint32_t)held[0] | ((uint32_t)held[1] << 8) | ((uint32_t)held[2] << 16) | ((uint32_t)held[3] << 24);
        };
        auto count = [&]() {
            const uint32_t held = word();
            NEURA_ASSERT(held <= bytes.size(), "a snapshot counts %u values in %zu bytes", held, bytes.size());
            return held;
        };
        auto words = [&]() {
            std::vector<uint32_t> out(count());
            for (uint32_t &value : out) value = word();
            return out;
        };
        auto floats = [&]() {
            std::vector<float> out(count());
            for (float &value : out) {
                const uint32_t bits = word();
                memcpy(&value, &bits, 4);
            }
            return out;
        };
        NEURA_ASSERT(bytes.size() >= 4 && memcmp(take(4), "NBS1", 4) == 0, "a batch snapshot opens with the four bytes NBS1");
        BatchSnapshot out;
        out.batch = word(), out.context = word(), out.window = word();
        const uint32_t sampled = word();
        NEURA_ASSERT(sampled <= 1, "a batch snapshot samples by %u", sampled);
        out.sampled = sampled == 1;
        if (word() != 0) out.prefix = words();
        const uint32_t planes = count();
        NEURA_ASSERT(planes == out.batch, "a snapshot of %u planes names %u slots", out.batch, planes);
        for (uint32_t plane = 0; plane < planes; plane++) {
            const uint32_t tag = word();
            if (tag == 0) {
                out.slots.push_back(std::nullopt);
                continue;
            }
            SlotSnapshot slot{word(), tag, {}, 0};
            if (tag == 1) slot.prompt = words();
            else if (tag == 2) slot.feed = word();
            else NEURA_ASSERT(tag == 3, "a slot snapshot holds phase %u", tag);
            out.slots.push_back(slot);
        }
        out.seeds = words();
        out.temperatures = floats(), out.keeps = floats(), out.cumulatives = floats();
        const uint32_t names = count();
        for (uint32_t i = 0; i < names; i++) {
            const uint32_t length = word();
            const uint8_t *held = take(length);
            out.state_names.emplace_back(reinterpret_cast<const char *>(held), length);
        }
        const uint32_t held = count();
        NEURA_ASSERT(held == names, "a snapshot names %u states and holds %u of them", names, held);
        for (uint32_t i = 0; i < held; i++) out.states.push_back(floats());
        NEURA_ASSERT(at == bytes.size(), "a snapshot holds %zu bytes where its reader stops at %zu", bytes.size(), at);
        NEURA_ASSERT(out.seeds.size() == out.batch, "a snapshot of %u planes carries %zu seeds", out.batch, out.seeds.size());
        for (const auto *values : {&out.temperatures, &out.keeps, &out.cumulatives})
            NEURA_ASSERT(values->size() == out.batch, "a snapshot of %u planes carries %zu values", out.batch, values->size());
        for (const auto &values : out.states)
            NEURA_ASSERT(values.size() == out.batch, "a state of %u planes carries %zu values", out.batch, values.size());
        return out;
    }
};

// The generation state machine (crates/neura-generate/src/batch.rs:279-465, :1000-1172,
// :1401-1517, :1595-1725): admit / restart / resume / suspend / finish / step with chunked
// prompt fill; greedy, or sampled with per-plane seeds, temperatures, candidate counts and nuclei
// (:643-732, :829-864).  Single threaded, one model, like `&mut Batch`.
class Batch {
  public:
    // the constructor's refusals, callable without a model
    static void validate(const BatchSpec &spec) {
        NEURA_ASSERT(spec.batch > 0, "a batch of no plane answers nothing");
        NEURA_ASSERT(spec.context > 0, "a context of no token holds no batch");
        for (size_t i = 0; i + 1 < spec.chunks.size(); i++)
            NEURA_ASSERT(spec.chunks[i] > spec.chunks[i + 1], "a batch fills the largest chunk first, and fills %u then %u", spec.chunks[i],
                         spec.chunks[i + 1]);
        for (uint32_t chunk : spec.chunks)
            NEURA_ASSERT(chunk > 1 && chunk < spec.context,
                         "a batch fills %u rows of a context of %u, and a chunk holds between two rows and the rows a prompt leaves for the answer",
                         chunk, spec.context);
        // crates/neura-generate/src/batch.rs:313-322
        const uint32_t widest = spec.chunks.empty() ? 1 : spec.chunks.front(), window = spec.window_tokens.value_or(spec.context);
        NEURA_ASSERT(window <= spec.context, "a batch keeps a window of %u tokens over a context of %u", window, spec.context);
        NEURA_ASSERT(widest <= window, "a batch fills chunks of %u rows into a window of %u tokens", widest, window);
    }
    Batch(Model &model, BatchSpec spec)
        : model_(model), batch_(spec.batch), context_(spec.context), window_(spec.window_tokens.value_or(spec.context)), chunks_(spec.chunks),
          slots_(spec.batch), shared_(spec.shares), seeded_(!spec.sampling.greedy),
          temperatures_(spec.batch, spec.sampling.temperature), keeps_(spec.batch, spec.sampling.keep), cumulatives_(spec.batch, spec.sampling.cumulative) {
        validate(spec);
        for (uint32_t slot = 0; slot < batch_; slot++) seeds_.push_back(plane_seed(0, slot));  // batch.rs:426-428
    }

    // ---- what a sampled batch draws with (crates/neura-generate/src/batch.rs:643-732, :829-864): written by the host
    // between steps, per plane or for every plane
    bool sampled() const { return seeded_; }
    uint32_t seed_of(uint32_t slot) const {
        plane(slot);
        NEURA_ASSERT(seeded_, "a greedy batch draws no seed");
        return seeds_[slot];
    }
    void set_seed(uint32_t seed) {
        NEURA_ASSERT(seeded_, "a greedy batch draws no seed");
        for (uint32_t slot = 0; slot < batch_; slot++) seeds_[slot] = plane_seed(seed, slot);
    }
    void set_seed_of(uint32_t slot, uint32_t seed) {
        plane(slot);
        NEURA_ASSERT(seeded_, "a greedy batch draws no seed");
        seeds_[slot] = seed;
    }
    void set_temperature(float value) {
        Sampling::check_temperature(value);
        NEURA_ASSERT(seeded_, "a greedy batch draws no temperature");
        std::fill(temperatures_.begin(), temperatures_.end(), value);
    }
    void set_temperature_of(uint32_t slot, float value) {
        plane(slot);
        Sampling::check_temperature(value);
        NEURA_ASSERT(seeded_, "a greedy batch draws no temperature");
        temperatures_[slot] = value;
    }
    void set_keep(uint32_t keep) {
        check_keep(keep);
        NEURA_ASSERT(seeded_, "a greedy batch draws no candidate count");
        std::fill(keeps_.begin(), keeps_.end(), keep);
    }
    void set_keep_of(uint32_t slot, uint32_t keep) {
        plane(slot);
        check_keep(keep);
        NEURA_ASSERT(seeded_, "a greedy batch draws no candidate count");
        keeps_[slot] = keep;
    }
    void set_cumulative(float value) {
        Sampling::check_cumulative(value);
        NEURA_ASSERT(seeded_, "a greedy batch draws no cumulative mass");
        std::fill(cumulatives_.begin(), cumulatives_.end(), value);
    }
    void set_cumulative_of(uint32_t slot, float value) {
        plane(slot);
        Sampling::check_cumulative(value);
        NEURA_ASSERT(seeded_, "a greedy batch draws no cumulative mass");
        cumulatives_[slot] = value;
    }
    // crates/neura-generate/src/batch.rs:1841-1847: the seed of a plane under a batch seed, and the bits a batch writes for it
    static uint32_t plane_seed(uint32_t seed, uint32_t slot) { return seed ^ ((slot + 1u) * 0x9e3779b9u); }
    static uint32_t seed_bits(uint32_t seed) { return 0x3f800000u | ((seed ^ (seed >> 23)) & 0x007fffffu); }
    uint32_t batch() const { return batch_; }
    uint32_t context() const { return context_; }
    uint32_t window() const { return window_; }  // crates/neura-generate/src/batch.rs:635-637

    uint32_t admit(const std::vector<uint32_t> &tokens) {  // batch.rs:1000-1013
        for (uint32_t slot = 0; slot < batch_; slot++)
            if (!slots_[slot]) {
                restart(slot, tokens);
                return slot;
            }
        panic("all %u planes of this batch hold a sequence", batch_);
    }
    void restart(uint32_t slot, const std::vector<uint32_t> &tokens) {  // batch.rs:1056-1105
        NEURA_ASSERT(slot < batch_, "a batch of %u planes names no plane %u", batch_, slot);
        NEURA_ASSERT(!tokens.empty(), "a batch admits a prompt of at least one token");
        NEURA_ASSERT(tokens.size() < context_, "the prompt holds %zu tokens where this batch holds %u of context", tokens.size(), context_);
        std::vector<uint8_t> reset(batch_, 0), share(batch_, 0);
        reset[slot] = 1;
        size_t fed = 0;
        if (prefix_) {  // batch.rs:1076-1093: the plane starts from the keys and values the prefix left, at the cursor behind it
            NEURA_ASSERT(tokens.size() >= prefix_->size() && std::equal(prefix_->begin(), prefix_->end(), tokens.begin()),
                         "a batch shares a prefix of %zu tokens, and this prompt does not start with it", prefix_->size());
            NEURA_ASSERT(tokens.size() > prefix_->size(), "a prompt of %zu tokens holds no token after the shared prefix of %zu tokens", tokens.size(),
                         prefix_->size());
            fed = prefix_->size(), share[slot] = 1;
        }
        if (shared_)
            runtime::check(nh_model_reset_shared(model_.handle(), reset.data(), share.data(), batch_));
        else
            runtime::check(nh_model_reset(model_.handle(), reset.data(), batch_));
        slots_[slot] = Slot{(uint32_t)fed, Prompting, std::deque<uint32_t>(tokens.begin() + (std::ptrdiff_t)fed, tokens.end()), 0};
    }
    // Batch::prefix (batch.rs:885-994): the tokens every prompt of this batch will start with, fed once -- in the largest
    // chunk while it fits, then token by token -- into the shared plane the reset copies into a plane that starts a sequence
    void prefix(const std::vector<uint32_t> &tokens) {
        NEURA_ASSERT(shared_, "a batch fills a shared prefix only when it declares one");
        for (const auto &slot : slots_) NEURA_ASSERT(!slot.has_value(), "a batch fills a shared prefix while no plane holds a sequence");
        NEURA_ASSERT(!tokens.empty(), "a shared prefix holds at least one token");
        NEURA_ASSERT(tokens.size() < context_,
                     "a shared prefix holds %zu tokens where this batch holds %u of context, and the prompt after it holds at least one token",
                     tokens.size(), context_);
        if (prefix_ && *prefix_ == tokens) return;
        // no plane holds a sequence: plane 0 stands in for the one-plane program the reference compiles for the prefix
        std::vector<uint8_t> reset(batch_, 0), mask(batch_, 0);
        reset[0] = 1, mask[0] = 1;
        runtime::check(nh_model_reset(model_.handle(), reset.data(), batch_));
        const uint32_t bulk = chunks_.empty() ? 1 : chunks_.front();
        size_t at = 0;
        std::vector<uint32_t> cursors(batch_, 0), chosen(batch_, 0);
        while (bulk > 1 && tokens.size() - at >= bulk) {
            std::vector<uint32_t> rows((size_t)bulk * batch_, 0);
            for (uint32_t row = 0; row < bulk; row++) rows[(size_t)row * batch_] = tokens[at + row];
            cursors[0] = (uint32_t)at;
            runtime::check(nh_prefill(model_.handle(), rows.data(), bulk, cursors.data(), mask.data(), batch_));
            at += bulk;
        }
        for (; at < tokens.size(); at++) {
            std::vector<uint32_t> row(batch_, 0);
            row[0] = tokens[at], cursors[0] = (uint32_t)at;
            runtime::check(nh_decode_step(model_.handle(), row.data(), cursors.data(), mask.data(), batch_, chosen.data()));
        }
        runtime::check(nh_model_keep_prefix(model_.handle(), 0));
        prefix_ = tokens;
    }
    void forget_prefix() { prefix_.reset(); }  // batch.rs:996-998
    const std::optional<std::vector<uint32_t>> &shared_prefix() const { return prefix_; }
    void resume(uint32_t slot, const std::vector<uint32_t> &tokens) {  // batch.rs:1015-1054
        auto &held = slots_.at(slot);
        NEURA_ASSERT(held.has_value(), "plane %u of this batch holds no sequence", slot);
        NEURA_ASSERT(held->phase == Suspended, "plane %u resumes only after it is suspended, and it is %s its sequence", slot,
                     held->phase == Prompting ? "still feeding" : "still answering");
        NEURA_ASSERT(!tokens.empty(), "a sequence resumes with at least one token");
        NEURA_ASSERT(held->cursor < context_, "a sequence at cursor %u of a context of %u resumes only after the application restarts or releases it",
                     held->cursor, context_);
        NEURA_ASSERT(tokens.size() < context_ - held->cursor, "a sequence at cursor %u resumes with %zu tokens where this batch holds %u of context",
                     held->cursor, tokens.size(), context_);
        held->phase = Prompting;
        held->prompt.assign(tokens.begin(), tokens.end());
    }
    void suspend(uint32_t slot) {  // batch.rs:1107-1123
        auto &held = slots_.at(slot);
        NEURA_ASSERT(held.has_value(), "plane %u of this batch holds no sequence", slot);
        if (held->phase == Prompting)
            panic("a sequence suspends after it has fed its prompt, and plane %u still holds %zu prompt tokens", slot, held->prompt.size());
        if (held->phase == Suspended) panic("plane %u of this batch is already suspended", slot);
        held->phase = Suspended;
    }
    void finish(uint32_t slot) {  // batch.rs:1137-1148
        NEURA_ASSERT(slot < batch_, "a batch of %u planes names no plane %u", batch_, slot);
        slots_[slot].reset();
    }
    std::vector<uint32_t> active() const {
        std::vector<uint32_t> out;
        for (uint32_t slot = 0; slot < batch_; slot++)
            if (slots_[slot] && slots_[slot]->phase != Suspended) out.push_back(slot);
        return out;
    }
    std::vector<uint32_t> occupied() const {
        std::vector<uint32_t> out;
        for (uint32_t slot = 0; slot < batch_; slot++)
            if (slots_[slot]) out.push_back(slot);
        return out;
    }
    std::optional<uint32_t> cursor(uint32_t slot) const { return slots_.at(slot) ? std::optional<uint32_t>(slots_[slot]->cursor) : std::nullopt; }
    std::optional<uint32_t> remaining(uint32_t slot) const {
        auto held = cursor(slot);
        return held ? std::optional<uint32_t>(context_ - *held) : std::nullopt;
    }

    // ---- what a batch holds between steps (crates/neura-generate/src/batch.rs:484-628) ----------------------------
    BatchSnapshot snapshot() const {
        BatchSnapshot out;
        out.batch = batch_, out.context = context_, out.window = window_, out.sampled = seeded_;
        out.prefix = prefix_;
        for (const auto &slot : slots_) {
            if (!slot) {
                out.slots.push_back(std::nullopt);
                continue;
            }
            out.slots.push_back(SlotSnapshot{slot->cursor, slot->phase == Prompting ? 1u : slot->phase == Generating ? 2u : 3u,
                                             std::vector<uint32_t>(slot->prompt.begin(), slot->prompt.end()), slot->feed});
        }
        out.seeds = seeds_, out.temperatures = temperatures_, out.cumulatives = cumulatives_;
        for (uint32_t keep : keeps_) out.keeps.push_back((float)keep);
        return out;
    }
    void restore(const BatchSnapshot &snapshot) {
        NEURA_ASSERT(snapshot.batch == batch_, "a batch of %u planes restores a snapshot of %u planes", batch_, snapshot.batch);
        NEURA_ASSERT(snapshot.context == context_, "a batch of %u tokens of context restores a snapshot of %u", context_, snapshot.context);
        NEURA_ASSERT(snapshot.window == window_, "a batch of a %u token window restores a snapshot of a %u token window", window_, snapshot.window);
        NEURA_ASSERT(snapshot.sampled == seeded_, "a batch draws %s restores a snapshot of a batch that draws %s", seeded_ ? "true" : "false",
                     snapshot.sampled ? "true" : "false");
        NEURA_ASSERT(snapshot.slots.size() == batch_, "a snapshot of %u planes holds %zu slots", batch_, snapshot.slots.size());
        NEURA_ASSERT(!snapshot.prefix || shared_, "a snapshot holds a shared prefix where this batch declares none");
        NEURA_ASSERT(snapshot.state_names.empty(), "a snapshot names %zu states where this batch registers 0", snapshot.state_names.size());
        NEURA_ASSERT(snapshot.states.size() == snapshot.state_names.size(), "a snapshot names %zu states and holds %zu of them",
                     snapshot.state_names.size(), snapshot.states.size());
        NEURA_ASSERT(snapshot.seeds.size() == batch_, "a batch of %u planes restores %zu seeds", batch_, snapshot.seeds.size());
        NEURA_ASSERT(snapshot.temperatures.size() == batch_, "a batch of %u planes restores %zu temperatures", batch_, snapshot.temperatures.size());
        NEURA_ASSERT(snapshot.keeps.size() == batch_, "a batch of %u planes restores %zu keeps", batch_, snapshot.keeps.size());
        NEURA_ASSERT(snapshot.cumulatives.size() == batch_, "a batch of %u planes restores %zu cumulatives", batch_, snapshot.cumulatives.size());
        for (uint32_t slot = 0; slot < batch_; slot++) {
            const auto &held = snapshot.slots[slot];
            if (!held) {
                slots_[slot].reset();
                continue;
            }
            slots_[slot] = Slot{held->cursor, held->phase == 1 ? Prompting : held->phase == 2 ? Generating : Suspended,
                                std::deque<uint32_t>(held->prompt.begin(), held->prompt.end()), held->feed};
        }
        seeds_ = snapshot.seeds, temperatures_ = snapshot.temperatures, cumulatives_ = snapshot.cumulatives;
        for (uint32_t slot = 0; slot < batch_; slot++) keeps_[slot] = (uint32_t)snapshot.keeps[slot];
        prefix_ = snapshot.prefix;  // batch.rs:621
    }
    // The device side of a batch between steps: the key and value states of every layer, written as the container the
    // reference's Runtime::save_state writes (crates/neura-runtime/src/checkpoint/container.rs:129-246: an 8-byte
    // length, a JSON header padded with blanks to a multiple of 8, then the tensors back to back in header order --
    // the layout of a safetensors file).  States are named as the decoder's caches name them (blk.N.cache.key / .value,
    // crates/neura-decoder/src/cache.rs:136-137) and shaped [key heads, planes, capacity, width] in half storage.
    void save_state(const std::string &path) const {
        const std::vector<State> states = device_states();
        const Element stored = model_.cache_element();
        const size_t wide = decoder::Cache::width_of(stored);
        const char *dtype = stored == Element::Single ? "F32" : stored == Element::Bfloat16 ? "BF16" : "F16";
        std::string header = "{";
        size_t at = 0;
        for (size_t i = 0; i < states.size(); i++) {
            if (i) header += ',';
            header += '"' + states[i].name + "\":{\"dtype\":\"" + dtype + "\",\"shape\":" + states[i].shape + ",\"data_offsets\":[" + std::to_string(at) + ',';
            at += states[i].elements * wide;
            header += std::to_string(at) + "]}";
        }
        header += '}';
        header.resize((header.size() + 7) / 8 * 8, ' ');
        std::ofstream out(path, std::ios::binary);
        if (!out) panic("a container at %s could not be created", path.c_str());
        const uint64_t length = header.size();
        for (int k = 0; k < 8; k++) out.put((char)(length >> (8 * k)));
        out.write(header.data(), (std::streamsize)header.size());
        std::vector<uint8_t> held;
        for (const State &state : states) {
            held.resize(state.elements * wide);
            if (state.shared)
                runtime::check(nh_model_shared_read(model_.handle(), state.layer, state.value ? 1 : 0, held.data()));
            else
                runtime::check(nh_model_cache_read(model_.handle(), state.layer, state.value ? 1 : 0, held.data()));
            out.write(reinterpret_cast<const char *>(held.data()), (std::streamsize)(state.elements * wide));
        }
        out.flush();
        if (!out) panic("a container at %s could not be written", path.c_str());
    }
    // Batch::restore_state (batch.rs:519-532): the device states out of a container, then the host bookkeeping
    void restore_state(const std::string &path, const BatchSnapshot &snapshot) {
        std::ifstream in(path, std::ios::binary);
        if (!in) panic("a container at %s could not be opened", path.c_str());
        uint8_t framed[8];
        in.read(reinterpret_cast<char *>(framed), 8);
        NEURA_ASSERT(in.gcount() == 8, "a container at %s holds no header length", path.c_str());
        uint64_t length = 0;
        for (int k = 0; k < 8; k++) length |= (uint64_t)framed[k] << (8 * k);
        NEURA_ASSERT(length > 0 && length < (1ull << 26), "a container at %s frames a header of %llu bytes", path.c_str(), (unsigned long long)length);
        std::string header(length, ' ');
        in.read(header.data(), (std::streamsize)length);
        NEURA_ASSERT((uint64_t)in.gcount() == length, "a container at %s ends inside its header", path.c_str());
        const Element stored = model_.cache_element();
        const size_t wide = decoder::Cache::width_of(stored);
        const std::string dtype = std::string("\"dtype\":\"") + (stored == Element::Single ? "F32" : stored == Element::Bfloat16 ? "BF16" : "F16") + "\"";
        std::vector<uint8_t> held;
        for (const State &state : device_states()) {
            const std::string &name = state.name;
            const size_t elements = state.elements;
            const size_t found = header.find('"' + name + "\":{");
            NEURA_ASSERT(found != std::string::npos, "the container at %s holds no state named %s", path.c_str(), name.c_str());
            const size_t close = header.find('}', found);
            const std::string entry = compact(header.substr(found, close - found));
            NEURA_ASSERT(entry.find(dtype) != std::string::npos, "state %s of the container at %s is not in %s storage", name.c_str(),
                         path.c_str(), neura::name(stored));
            NEURA_ASSERT(entry.find("\"shape\":" + state.shape) != std::string::npos, "state %s of the container at %s is not shaped %s", name.c_str(),
                         path.c_str(), state.shape.c_str());
            const size_t offsets = entry.find("\"data_offsets\":[");
            NEURA_ASSERT(offsets != std::string::npos, "state %s of the container at %s names no bytes", name.c_str(), path.c_str());
            const uint64_t begin = std::stoull(entry.substr(offsets + 16));
            const uint64_t end = std::stoull(entry.substr(entry.find(',', offsets + 16) + 1));
            NEURA_ASSERT(end - begin == elements * wide, "state %s of the container at %s holds %llu bytes where the cache holds %zu", name.c_str(),
                         path.c_str(), (unsigned long long)(end - begin), elements * wide);
            held.resize(elements * wide);
            in.seekg((std::streamoff)(8 + length + begin));
            in.read(reinterpret_cast<char *>(held.data()), (std::streamsize)(elements * wide));
            NEURA_ASSERT((size_t)in.gcount() == elements * wide, "the container at %s ends inside state %s", path.c_str(), name.c_str());
            if (state.shared)
                runtime::check(nh_model_shared_write(model_.handle(), state.layer, state.value ? 1 : 0, held.data()));
            else
                runtime::check(nh_model_cache_write(model_.handle(), state.layer, state.value ? 1 : 0, held.data()));
        }
        restore(snapshot);
    }

    std::vector<Emitted> step() {  // batch.rs:1125-1135
        if (active().empty()) return {};
        prefill();
        return answer();
    }

  private:
    enum Phase { Prompting, Generating, Suspended };
    struct Slot {
        uint32_t cursor;
        Phase phase;
        std::deque<uint32_t> prompt;
        uint32_t feed;
    };

    // batch.rs:1401-1432: the first (largest) chunk some prompt still exceeds, and the planes it serves
    bool next_fill(size_t &index, std::vector<uint32_t> &group) const {
        std::vector<std::vector<uint32_t>> groups(chunks_.size());
        for (uint32_t slot = 0; slot < batch_; slot++) {
            if (!slots_[slot] || slots_[slot]->phase != Prompting) continue;
            size_t left = slots_[slot]->prompt.size();
            if (left <= 1) continue;
            NEURA_ASSERT(slots_[slot]->cursor < context_, "a sequence at cursor %u of a context of %u no longer reaches the prompt it holds",
                         slots_[slot]->cursor, context_);
            for (size_t i = 0; i < chunks_.size(); i++)
                if (chunks_[i] < left) {
                    groups[i].push_back(slot);
                    break;
                }
        }
        for (size_t i = 0; i < groups.size(); i++)
            if (!groups[i].empty()) {
                index = i, group = groups[i];
                return true;
            }
        return false;
    }
    void prefill() {  // batch.rs:1595-1599, :1434-1501
        size_t index;
        std::vector<uint32_t> group;
        while (next_fill(index, group)) {
            const uint32_t rows = chunks_[index];
            std::vector<uint32_t> tokens((size_t)rows * batch_, 0), cursors(batch_, 0);
            std::vector<uint8_t> mask(batch_, 0);
            for (uint32_t slot : group) {
                auto &held = *slots_[slot];
                cursors[slot] = held.cursor, mask[slot] = 1;
                for (uint32_t row = 0; row < rows; row++) tokens[(size_t)row * batch_ + slot] = held.prompt[row];
            }
            runtime::check(nh_prefill(model_.handle(), tokens.data(), rows, cursors.data(), mask.data(), batch_));
            for (uint32_t slot : group) {
                auto &held = *slots_[slot];
                held.cursor += rows;
                held.prompt.erase(held.prompt.begin(), held.prompt.begin() + rows);
            }
        }
    }
    std::vector<Emitted> answer() {  // batch.rs:1601-1644, :1681-1725
        std::vector<uint32_t> tokens(batch_, 0), cursors(batch_, 0), chosen(batch_, 0);
        std::vector<uint8_t> mask(batch_, 0);
        for (uint32_t slot = 0; slot < batch_; slot++) {
            if (!slots_[slot] || slots_[slot]->phase == Suspended) continue;
            auto &held = *slots_[slot];
            NEURA_ASSERT(held.cursor < context_, "a sequence at cursor %u of a context of %u no longer %s", held.cursor, context_,
                         held.phase == Prompting ? "feeds the prompt it holds" : "answers; suspend or release it");
            tokens[slot] = held.phase == Prompting ? held.prompt.front() : held.feed;
            cursors[slot] = held.cursor, mask[slot] = 1;
        }
        if (seeded_) {
            std::vector<nh_draw> draws(batch_);
            for (uint32_t slot = 0; slot < batch_; slot++)
                draws[slot] = nh_draw{seed_bits(seeds_[slot]), temperatures_[slot], keeps_[slot], cumulatives_[slot]};
            runtime::check(nh_decode_step_sampled(model_.handle(), tokens.data(), cursors.data(), mask.data(), batch_, draws.data(), chosen.data()));
        } else {
            runtime::check(nh_decode_step(model_.handle(), tokens.data(), cursors.data(), mask.data(), batch_, chosen.data()));
        }
        std::vector<Emitted> emitted;
        for (uint32_t slot = 0; slot < batch_; slot++) {
            if (!slots_[slot]) continue;
            auto &held = *slots_[slot];
            // a plane draws when it answers: on the last token of its prompt and on every token after (batch.rs:1688-1709)
            const bool drew = held.phase == Generating || (held.phase == Prompting && held.prompt.size() == 1);
            if (drew) seeds_[slot] += 1u;
            if (held.phase == Prompting) {
                held.prompt.pop_front();
                if (held.prompt.empty()) held.phase = Generating, held.feed = chosen[slot];
            } else if (held.phase == Generating) {
                emitted.push_back(Emitted{slot, held.feed});  // a token is emitted on the step after it was chosen
                held.feed = chosen[slot];
            }
            if (held.phase != Suspended) held.cursor += 1;
        }
        return emitted;
    }

    void plane(uint32_t slot) const { NEURA_ASSERT(slot < batch_, "a batch of %u planes names no plane %u", batch_, slot); }
    // the device states of this batch in the order a container holds them (one storage width: by name): blk.N.cache.key / .value,
    // and blk.N.cache.shared.key / .value of one plane where the batch declares a shared prefix (cache.rs:136-137, :140-143)
    struct State {
        std::string name, shape;
        uint32_t layer;
        bool value, shared;
        size_t elements;
    };
    std::vector<State> device_states() const {
        const Config &c = model_.config();
        const uint32_t capacity = nh_model_capacity(model_.handle());
        std::vector<State> out;
        for (uint32_t layer = 0; layer < c.layers; layer++)
            for (int shared = 0; shared < (shared_ ? 2 : 1); shared++)
                for (int value = 0; value < 2; value++) {
                    const uint32_t planes = shared ? 1 : batch_;
                    out.push_back(State{"blk." + std::to_string(layer) + ".cache." + (shared ? "shared." : "") + (value ? "value" : "key"),
                                        "[" + std::to_string(c.key_heads) + ',' + std::to_string(planes) + ',' + std::to_string(capacity) + ',' +
                                            std::to_string(c.head_width) + "]",
                                        layer, value != 0, shared != 0, (size_t)c.key_heads * planes * capacity * c.head_width});
                }
        std::sort(out.begin(), out.end(), [](const State &a, const State &b) { return a.name < b.name; });
        return out;
    }
    static std::string compact(const std::string &text) {  // a header entry without the blanks a writer may have put between its parts
        std::string out;
        for (char held : text)
            if (held != ' ' && held != '\n' && held != '\t') out.push_back(held);
        return out;
    }
    static void check_keep(uint32_t keep) {
        NEURA_ASSERT(keep >= 1 && keep <= Sampling::CANDIDATES, "a batch keeps %u candidates where a row holds between one and %u", keep,
                     Sampling::CANDIDATES);
    }

    Model &model_;
    uint32_t batch_, context_, window_;
    std::vector<uint32_t> chunks_;
    std::vector<std::optional<Slot>> slots_;
    bool shared_ = false;
    std::optional<std::vector<uint32_t>> prefix_;
    bool seeded_;
    std::vector<uint32_t> seeds_;
    std::vector<float> temperatures_;
    std::vector<uint32_t> keeps_;
    std::vector<float> cumulatives_;
};

}  // namespace generate
}  // namespace neura
