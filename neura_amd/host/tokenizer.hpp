// Byte-level BPE as a GGUF of the gpt2 kind holds it, and the split rule of Qwen2's tokenizer: the host-side mirror of
// crates/neura-tokenizer (Rule, Vocabulary, Tokenizer, Text) and of the rule the reference's qwen example passes in
// (examples/qwen/text/qwen.rs).  Token ids in, token ids out: nothing here touches the device.
#pragma once
#include <string_view>
#include <unordered_set>

#include "neura.hpp"
#include "unicode_tables.hpp"

namespace neura {
namespace tokenizer {

// ---- UTF-8 ------------------------------------------------------------------------------------------------------------
inline void push_utf8(std::string &out, uint32_t point) {
    if (point < 0x80) {
        out.push_back((char)point);
    } else if (point < 0x800) {
        out.push_back((char)(0xc0 | (point >> 6)));
        out.push_back((char)(0x80 | (point & 0x3f)));
    } else if (point < 0x10000) {
        out.push_back((char)(0xe0 | (point >> 12)));
        out.push_back((char)(0x80 | ((point >> 6) & 0x3f)));
        out.push_back((char)(0x80 | (point & 0x3f)));
    } else {
        out.push_back((char)(0xf0 | (point >> 18)));
        out.push_back((char)(0x80 | ((point >> 12) & 0x3f)));
        out.push_back((char)(0x80 | ((point >> 6) & 0x3f)));
        out.push_back((char)(0x80 | (point & 0x3f)));
    }
}

// One step of a strict UTF-8 reader over bytes[at .. size): the width of the character that starts there (its code point
// in `point`), 0 when the bytes run out inside a character that is well formed so far, or minus the count of bytes that
// cannot start a character (the maximal ill-formed prefix, as Rust's Utf8Error::error_len counts it).
inline int utf8_step(const uint8_t *bytes, size_t size, size_t at, uint32_t &point) {
    const uint8_t lead = bytes[at];
    if (lead < 0x80) return point = lead, 1;
    int width;
    uint8_t low = 0x80, high = 0xbf;
    if (lead >= 0xc2 && lead <= 0xdf) width = 2;
    else if (lead >= 0xe0 && lead <= 0xef) width = 3, low = lead == 0xe0 ? 0xa0 : 0x80, high = lead == 0xed ? 0x9f : 0xbf;
    else if (lead >= 0xf0 && lead <= 0xf4) width = 4, low = lead == 0xf0 ? 0x90 : 0x80, high = lead == 0xf4 ? 0x8f : 0xbf;
    else return -1;
    point = lead & (width == 2 ? 0x1f : width == 3 ? 0x0f : 0x07);
    for (int k = 1; k < width; k++) {
        if (at + k >= size) return 0;
        const uint8_t next = bytes[at + k];
        if (next < (k == 1 ? low : 0x80) || next > (k == 1 ? high : 0xbf)) return -k;
        point = (point << 6) | (next & 0x3f);
    }
    return width;
}

// the code points of a text that is UTF-8 already, and the byte each starts at (one more entry: the text's end)
inline void code_points(std::string_view text, std::vector<uint32_t> &points, std::vector<size_t> &offsets) {
    const uint8_t *bytes = reinterpret_cast<const uint8_t *>(text.data());
    size_t at = 0;
    while (at < text.size()) {
        uint32_t point = 0;
        const int width = utf8_step(bytes, text.size(), at, point);
        NEURA_ASSERT(width > 0, "a tokenizer reads text, and byte %zu of this one starts no character", at);
        points.push_back(point), offsets.push_back(at);
        at += (size_t)width;
    }
    offsets.push_back(text.size());
}

// crates/neura-tokenizer/src/text.rs: bytes of generated pieces in, the text they spell out as soon as whole characters
// stand; ill-formed bytes read as U+FFFD
class Text {
  public:
    std::string push(const std::vector<uint8_t> &piece) {
        held_.insert(held_.end(), piece.begin(), piece.end());
        std::string out;
        size_t at = 0;
        while (at < held_.size()) {
            uint32_t point = 0;
            const int width = utf8_step(held_.data(), held_.size(), at, point);
            if (width == 0) break;  // the character may still arrive
            if (width > 0) out.append(reinterpret_cast<const char *>(held_.data() + at), (size_t)width), at += (size_t)width;
            else out += "\xef\xbf\xbd", at += (size_t)(-width);
        }
        held_.erase(held_.begin(), held_.begin() + (std::ptrdiff_t)at);
        return out;
    }
    std::string flush() {
        std::string out;
        size_t at = 0;
        while (at < held_.size()) {
            uint32_t point = 0;
            const int width = utf8_step(held_.data(), held_.size(), at, point);
            if (width > 0) {
                out.append(reinterpret_cast<const char *>(held_.data() + at), (size_t)width), at += (size_t)width;
            } else {  // an ill-formed prefix, or the start of a character that never came whole: one replacement each
                out += "\xef\xbf\xbd";
                at = width == 0 ? held_.size() : at + (size_t)(-width);
            }
        }
        held_.clear();
        return out;
    }

  private:
    std::vector<uint8_t> held_;
};

// crates/neura-tokenizer/src/rule.rs: where a text splits before its pieces merge
struct Rule {
    virtual ~Rule() = default;
    virtual std::vector<std::string_view> pieces(std::string_view text) const = 0;
};

// crates/neura-tokenizer/src/vocabulary.rs
class Vocabulary {
  public:
    struct Part {
        bool token;
        uint32_t id;
        std::string_view text;
    };

    static Vocabulary read(const gguf::Archive &source) {
        const gguf::Metadata metadata = source.metadata();
        const std::string model = metadata.text("tokenizer.ggml.model");
        NEURA_ASSERT(model == "gpt2",
                     "this tokenizer reads the byte level bpe a gpt2 gguf holds, and this gguf names %s as its tokenizer.ggml.model", model.c_str());
        Vocabulary out;
        for (const gguf::Value &value : metadata.array("tokenizer.ggml.tokens")) {
            auto held = value.text();
            if (!held) panic("the tokenizer.ggml.tokens of this gguf holds %s where a string stands", value.name());
            out.tokens_.push_back(*held);
        }
        std::vector<uint32_t> kinds;
        for (const gguf::Value &value : metadata.array("tokenizer.ggml.token_type")) {
            auto held = value.integer();
            if (!held) panic("the tokenizer.ggml.token_type of this gguf holds %s where a whole number stands", value.name());
            if (*held > 0xffffffffull)
                panic("the tokenizer.ggml.token_type of this gguf holds %llu where a word holds what fits one", (unsigned long long)*held);
            kinds.push_back((uint32_t)*held);
        }
        for (size_t at = 0; at < out.tokens_.size(); at++) {
            out.ids_[out.tokens_[at]] = (uint32_t)at;
            const bool held = at < kinds.size() && kinds[at] >= 2 && kinds[at] <= 4;  // unknown, control, user defined
            out.special_.push_back(held);
            if (held) out.control_.push_back({out.tokens_[at], (uint32_t)at});
        }
        std::stable_sort(out.control_.begin(), out.control_.end(), [](const auto &a, const auto &b) { return a.first.size() > b.first.size(); });
        uint32_t rank = 0;
        for (const gguf::Value &value : metadata.array("tokenizer.ggml.merges")) {
            auto held = value.text();
            if (!held) panic("the tokenizer.ggml.merges of this gguf holds %s where a string stands", value.name());
            const size_t space = held->find(' ');
            if (space == std::string::npos) panic("the merge %s of this gguf names two pieces where it splits on no space", held->c_str());
            out.ranks_[pair_key(held->substr(0, space), held->substr(space + 1))] = rank++;
        }
        // the byte alphabet of gpt2: printable bytes spell themselves, the others the code points from 256 up
        uint32_t extra = 0;
        for (uint32_t byte = 0; byte < 256; byte++) {
            const bool printable = (byte >= 0x21 && byte <= 0x7e) || (byte >= 0xa1 && byte <= 0xac) || (byte >= 0xae && byte <= 0xff);
            out.alphabet_[byte] = printable ? byte : 256 + extra++;
            out.bytes_[out.alphabet_[byte]] = (uint8_t)byte;
        }
        return out;
    }

    size_t len() const { return tokens_.size(); }
    bool is_empty() const { return tokens_.empty(); }
    std::optional<uint32_t> id(const std::string &token) const {
        auto found = ids_.find(token);
        return found == ids_.end() ? std::nullopt : std::optional<uint32_t>(found->second);
    }
    // a piece of text in the byte alphabet
    std::string spell(std::string_view text) const {
        std::string out;
        for (unsigned char byte : text) push_utf8(out, alphabet_[byte]);
        return out;
    }
    // the ids of a spelled piece: the lowest ranked neighbouring pair joins first, the leftmost of equals
    std::vector<uint32_t> merge(const std::string &piece) const {
        if (auto whole = id(piece)) return {*whole};
        std::vector<uint32_t> points;
        std::vector<size_t> offsets;
        code_points(piece, points, offsets);
        std::vector<std::string> parts;
        for (size_t at = 0; at < points.size(); at++) parts.push_back(piece.substr(offsets[at], offsets[at + 1] - offsets[at]));
        for (;;) {
            std::optional<std::pair<uint32_t, size_t>> best;
            for (size_t at = 0; at + 1 < parts.size(); at++) {
                auto found = ranks_.find(pair_key(parts[at], parts[at + 1]));
                if (found != ranks_.end() && (!best || found->second < best->first)) best = std::make_pair(found->second, at);
            }
            if (!best) break;
            parts[best->second] += parts[best->second + 1];
            parts.erase(parts.begin() + (std::ptrdiff_t)best->second + 1);
        }
        std::vector<uint32_t> out;
        for (const std::string &part : parts) {
            auto held = id(part);
            if (!held) panic("this vocabulary holds no piece %s", part.c_str());
            out.push_back(*held);
        }
        return out;
    }
    // the text cut at its special tokens, the longest names first
    std::vector<Part> parted(std::string_view text) const {
        std::vector<Part> parts{Part{false, 0, text}};
        for (const auto &[token, id] : control_) {
            std::vector<Part> next;
            for (const Part &part : parts) {
                if (part.token) {
                    next.push_back(part);
                    continue;
                }
                const std::string_view held = part.text;
                size_t at = 0;
                for (;;) {
                    const size_t found = token.empty() ? std::string_view::npos : held.find(token, at);
                    if (found == std::string_view::npos) break;
                    if (found > at) next.push_back(Part{false, 0, held.substr(at, found - at)});
                    next.push_back(Part{true, id, {}});
                    at = found + token.size();
                }
                if (at < held.size()) next.push_back(Part{false, 0, held.substr(at)});
            }
            parts = std::move(next);
        }
        return parts;
    }
    // the bytes token `id` stands for
    std::vector<uint8_t> piece(uint32_t id) const {
        if (id >= tokens_.size()) panic("this vocabulary holds no token %u of %zu tokens", id, tokens_.size());
        const std::string &held = tokens_[id];
        if (special_[id]) return std::vector<uint8_t>(held.begin(), held.end());
        std::vector<uint32_t> points;
        std::vector<size_t> offsets;
        code_points(held, points, offsets);
        std::vector<uint8_t> out;
        for (uint32_t point : points) {
            auto found = bytes_.find(point);
            if (found == bytes_.end()) panic("the token %s holds a character no byte of it stands behind", held.c_str());
            out.push_back(found->second);
        }
        return out;
    }

  private:
    static std::string pair_key(const std::string &left, const std::string &right) {
        std::string key = left;
        key.push_back('\0');
        return key += right;
    }
    std::vector<std::string> tokens_;
    std::vector<bool> special_;
    std::unordered_map<std::string, uint32_t> ids_, ranks_;
    std::vector<std::pair<std::string, uint32_t>> control_;
    uint32_t alphabet_[256] = {};
    std::unordered_map<uint32_t, uint8_t> bytes_;
};

// crates/neura-tokenizer/src/tokenizer.rs
class Tokenizer {
  public:
    Tokenizer(Vocabulary vocabulary, std::unique_ptr<Rule> rule) : vocabulary_(std::move(vocabulary)), rule_(std::move(rule)) {}
    size_t vocabulary() const { return vocabulary_.len(); }
    std::optional<uint32_t> id(const std::string &token) const { return vocabulary_.id(token); }
    std::vector<uint32_t> encode(std::string_view text) const {
        std::vector<uint32_t> ids;
        for (const Vocabulary::Part &part : vocabulary_.parted(text)) {
            if (part.token) {
                ids.push_back(part.id);
                continue;
            }
            for (std::string_view piece : rule_->pieces(part.text)) {
                NEURA_ASSERT(!piece.empty(), "a split rule names the pieces of the text it reads, and one of them holds no character");
                for (uint32_t id : vocabulary_.merge(vocabulary_.spell(piece))) ids.push_back(id);
            }
        }
        return ids;
    }
    std::vector<uint8_t> piece(uint32_t id) const { return vocabulary_.piece(id); }

  private:
    Vocabulary vocabulary_;
    std::unique_ptr<Rule> rule_;
};

// ---- rules -------------------------------------------------------------------------------------------------------------
inline bool in_ranges(const uint32_t (*table)[2], size_t count, uint32_t point) {
    size_t low = 0, high = count;
    while (low < high) {
        const size_t middle = (low + high) / 2;
        if (point < table[middle][0]) high = middle;
        else if (point > table[middle][1]) low = middle + 1;
        else return true;
    }
    return false;
}
inline bool is_letter(uint32_t point) { return in_ranges(unicode::LETTERS, sizeof(unicode::LETTERS) / sizeof(unicode::LETTERS[0]), point); }
inline bool is_number(uint32_t point) { return in_ranges(unicode::NUMBERS, sizeof(unicode::NUMBERS) / sizeof(unicode::NUMBERS[0]), point); }
inline bool is_space(uint32_t point) { return in_ranges(unicode::WHITE_SPACE, sizeof(unicode::WHITE_SPACE) / sizeof(unicode::WHITE_SPACE[0]), point); }

// The split of Qwen2's pre-tokenizer, its published pattern read alternative by alternative, the first that matches at a
// position winning (examples/qwen/text/qwen.rs walks the same pattern):
//   (?i:'s|'t|'re|'ve|'m|'ll|'d) | [^\r\n\p{L}\p{N}]?\p{L}+ | \p{N} | ?[^\s\p{L}\p{N}]+[\r\n]* | \s*[\r\n]+ | \s+(?!\S) | \s+
struct Qwen : Rule {
    std::vector<std::string_view> pieces(std::string_view text) const override {
        std::vector<uint32_t> held;
        std::vector<size_t> offsets;
        code_points(text, held, offsets);
        const size_t count = held.size();
        auto at_or = [&](size_t at) { return at < count ? held[at] : 0xffffffffu; };
        auto lower = [&](size_t at) {
            const uint32_t point = at_or(at);
            return point >= 'A' && point <= 'Z' ? point + 32 : point;
        };
        auto letter = [&](size_t at) { return at < count && is_letter(held[at]); };
        auto space = [&](size_t at) { return at < count && is_space(held[at]); };
        auto other = [&](size_t at) { return at < count && !is_space(held[at]) && !is_letter(held[at]) && !is_number(held[at]); };
        auto newline = [&](size_t at) { return at < count && (held[at] == '\r' || held[at] == '\n'); };
        std::vector<std::string_view> out;
        size_t at = 0;
        auto take = [&](size_t end) {
            out.push_back(text.substr(offsets[at], offsets[end] - offsets[at]));
            at = end;
        };
        while (at < count) {
            const uint32_t point = held[at];
            if (point == '\'') {  // a contraction
                const uint32_t one = lower(at + 1), two = lower(at + 2);
                if (one == 's' || one == 't') { take(at + 2); continue; }
                if ((one == 'r' && two == 'e') || (one == 'v' && two == 'e')) { take(at + 3); continue; }
                if (one == 'm') { take(at + 2); continue; }
                if (one == 'l' && two == 'l') { take(at + 3); continue; }
                if (one == 'd') { take(at + 2); continue; }
            }
            // letters, with at most one character ahead of them that is no letter, number or line break
            if (letter(at) || (!newline(at) && !is_number(point) && letter(at + 1))) {
                size_t end = at + 1;
                while (letter(end)) end++;
                take(end);
                continue;
            }
            if (is_number(point)) { take(at + 1); continue; }  // one digit a piece
            // what is neither space, letter nor number, after at most one blank, with the line breaks that follow
            if (other(at) || (point == ' ' && other(at + 1))) {
                size_t end = at + (point == ' ' ? 1 : 0);
                while (other(end)) end++;
                while (newline(end)) end++;
                take(end);
                continue;
            }
            // a run of whitespace: up to its last line break; else all but its last character when text follows; else all
            size_t run = 0, last_break = 0;
            while (space(at + run)) {
                if (newline(at + run)) last_break = at + run + 1;
                run++;
            }
            if (last_break) { take(last_break); continue; }
            if (run > 1 && at + run < count) { take(at + run - 1); continue; }
            if (run > 0) { take(at + run); continue; }
            take(at + 1);
        }
        return out;
    }
};

// the three rules of the reference's own tokenizer tests (crates/neura-tokenizer/tests/tokenizer.rs:9-38)
struct PerCharacter : Rule {
    std::vector<std::string_view> pieces(std::string_view text) const override {
        std::vector<uint32_t> held;
        std::vector<size_t> offsets;
        code_points(text, held, offsets);
        std::vector<std::string_view> out;
        for (size_t at = 0; at < held.size(); at++) out.push_back(text.substr(offsets[at], offsets[at + 1] - offsets[at]));
        return out;
    }
};
struct PerSpace : Rule {
    std::vector<std::string_view> pieces(std::string_view text) const override {
        std::vector<std::string_view> out;
        size_t at = 0;
        for (;;) {
            const size_t found = text.find(' ', at);
            out.push_back(text.substr(at, found == std::string_view::npos ? std::string_view::npos : found - at));
            if (found == std::string_view::npos) break;
            at = found + 1;
        }
        return out;
    }
};
struct Whole : Rule {
    std::vector<std::string_view> pieces(std::string_view text) const override { return {text}; }
};

}  // namespace tokenizer
}  // namespace neura
