// template.hpp -- the chat template engine: the subset of Jinja a GGUF's `tokenizer.chat_template` is written in.
//
// Mirrors crates/neura-template (lexer.rs, parser.rs, render.rs, value.rs, template.rs): Template::parse / read / render,
// Message, Value, with the reference's panics as neura::Panic carrying the same sentences.  What it reads: bodies, {{ prints }},
// {% if / elif / else %}, {% for x in .. %} with `loop`, {% set x = .. %} and {% set ns.x = .. %}, {% macro %}, {# comments #},
// `-` whitespace control; expressions with or / and / not, comparisons, in / not in, is [not] <test>, + - ~, filters
// (trim, string, safe, length, tojson), attributes, subscripts, slices, calls (macros, namespace(..), raise_exception(..)),
// string methods (split, strip, lstrip, rstrip, startswith, endswith), `x if c else y`.
#pragma once

#include "neura.hpp"

#include <charconv>

namespace neura {
namespace chat {

// whether the character at `at` is white space (char::is_whitespace), and the bytes it takes
inline bool space_at(const std::string &source, size_t at, size_t &wide) {
    const unsigned char c = (unsigned char)source[at];
    wide = 1;
    if (c < 0x80) return std::isspace(c) != 0;
    wide = c >= 0xf0 ? 4 : c >= 0xe0 ? 3 : c >= 0xc0 ? 2 : 1;
    uint32_t code = c >= 0xf0 ? c & 7u : c >= 0xe0 ? c & 15u : c & 31u;
    for (size_t k = 1; k < wide && at + k < source.size(); k++) code = code << 6 | ((unsigned char)source[at + k] & 63u);
    // the White_Space characters past ASCII
    return code == 0x85 || code == 0xa0 || code == 0x1680 || (code >= 0x2000 && code <= 0x200a) || code == 0x2028 || code == 0x2029 || code == 0x202f ||
           code == 0x205f || code == 0x3000;
}

// ---- values (crates/neura-template/src/value.rs) ------------------------------------------------
struct Value {
    enum Kind { Missing, Empty, Flag, Integer, Number, Text, List, Map, Namespace };
    using Entries = std::vector<std::pair<std::string, Value>>;
    Kind kind = Missing;
    bool flag = false;
    int64_t integer = 0;
    double number = 0.0;
    std::string string;
    std::vector<Value> items;
    Entries entries;
    std::shared_ptr<Entries> space;  // a namespace is shared by every copy of the value

    Value() = default;
    static Value missing() { return Value(); }
    static Value empty() { Value v; v.kind = Empty; return v; }
    static Value of(bool held) { Value v; v.kind = Flag, v.flag = held; return v; }
    static Value of(int64_t held) { Value v; v.kind = Integer, v.integer = held; return v; }
    static Value of(double held) { Value v; v.kind = Number, v.number = held; return v; }
    static Value of(std::string held) { Value v; v.kind = Text, v.string = std::move(held); return v; }
    static Value of(const char *held) { return of(std::string(held)); }
    static Value list(std::vector<Value> held) { Value v; v.kind = List, v.items = std::move(held); return v; }
    static Value map(Entries held) { Value v; v.kind = Map, v.entries = std::move(held); return v; }
    static Value names(Entries held) { Value v; v.kind = Namespace, v.space = std::make_shared<Entries>(std::move(held)); return v; }

    const Entries &fields() const { return kind == Namespace ? *space : entries; }

    bool truth() const {  // value.rs:18-30
        switch (kind) {
        case Missing: case Empty: return false;
        case Flag: return flag;
        case Integer: return integer != 0;
        case Number: return number != 0.0;
        case Text: return !string.empty();
        case List: return !items.empty();
        default: return !fields().empty();
        }
    }
    const char *kind_name() const {  // value.rs:50-62
        static const char *names[] = {"what the template leaves undefined", "none", "a flag", "a whole number", "a number", "a string", "a list", "a mapping",
                                      "a namespace"};
        return names[kind];
    }
    // the shortest digits that read back as the number, never in exponent form
    static std::string digits(double held) {
        if (std::isnan(held)) return "NaN";
        if (std::isinf(held)) return held < 0 ? "-inf" : "inf";
        char room[400];
        auto done = std::to_chars(room, room + sizeof(room), held, std::chars_format::fixed);
        return std::string(room, done.ptr);
    }
    std::string text() const {  // value.rs:32-48
        switch (kind) {
        case Missing: return "";
        case Empty: return "None";
        case Flag: return flag ? "True" : "False";
        case Integer: return std::to_string(integer);
        case Number: {
            std::string held = digits(number);
            if (std::isfinite(number) && number == std::trunc(number) && held.find('.') == std::string::npos) held += ".0";
            return held;
        }
        case Text: return string;
        default: return repr();
        }
    }
    std::string repr() const {  // value.rs:64-85
        switch (kind) {
        case Text: {
            std::string out = "'";
            for (char c : string) {
                if (c == '\\') out += "\\\\";
                else if (c == '\'') out += "\\'";
                else out += c;
            }
            return out + "'";
        }
        case List: {
            std::string out = "[";
            for (size_t i = 0; i < items.size(); i++) out += (i ? ", " : "") + items[i].repr();
            return out + "]";
        }
        case Map: case Namespace: {
            std::string out = "{";
            const Entries &held = fields();
            for (size_t i = 0; i < held.size(); i++) out += (i ? ", " : "") + of(held[i].first).repr() + ": " + held[i].second.repr();
            return out + "}";
        }
        default: return text();
        }
    }
    bool equals(const Value &other) const {  // value.rs:87-122
        if (kind == Missing || other.kind == Missing) return kind == Missing && other.kind == Missing;
        if (kind == Empty || other.kind == Empty) return kind == Empty && other.kind == Empty;
        const bool numeric = (kind == Integer || kind == Number) && (other.kind == Integer || other.kind == Number);
        if (numeric) {
            if (kind == Integer && other.kind == Integer) return integer == other.integer;
            return (kind == Integer ? (double)integer : number) == (other.kind == Integer ? (double)other.integer : other.number);
        }
        if (kind != other.kind) return false;
        switch (kind) {
        case Flag: return flag == other.flag;
        case Text: return string == other.string;
        case List:
            if (items.size() != other.items.size()) return false;
            for (size_t i = 0; i < items.size(); i++)
                if (!items[i].equals(other.items[i])) return false;
            return true;
        case Map:
            if (entries.size() != other.entries.size()) return false;
            for (const auto &entry : entries) {
                auto found = std::find_if(other.entries.begin(), other.entries.end(), [&](const auto &held) { return held.first == entry.first; });
                if (found == other.entries.end() || !entry.second.equals(found->second)) return false;
            }
            return true;
        case Namespace: return space == other.space;
        default: return false;
        }
    }
    bool greater(const Value &other) const {  // value.rs:124-137
        const bool numeric = (kind == Integer || kind == Number) && (other.kind == Integer || other.kind == Number);
        if (numeric) {
            if (kind == Integer && other.kind == Integer) return integer > other.integer;
            return (kind == Integer ? (double)integer : number) > (other.kind == Integer ? (double)other.integer : other.number);
        }
        if (kind == Text && other.kind == Text) return string > other.string;
        panic("a template weighs %s against %s where no order stands", kind_name(), other.kind_name());
    }
    Value add(const Value &other) const {  // value.rs:139-153
        if (kind == Text && other.kind == Text) return of(string + other.string);
        if (kind == Integer && other.kind == Integer) {
            int64_t sum;
            if (__builtin_add_overflow(integer, other.integer, &sum))
                panic("a template adds %lld to %lld where no whole number holds the sum", (long long)integer, (long long)other.integer);
            return of(sum);
        }
        const bool numeric = (kind == Integer || kind == Number) && (other.kind == Integer || other.kind == Number);
        if (numeric) return of((kind == Integer ? (double)integer : number) + (other.kind == Integer ? (double)other.integer : other.number));
        panic("a template adds %s to %s", other.kind_name(), kind_name());
    }
    Value attribute(const std::string &name) const {  // value.rs:159-174
        if (kind == Missing) return missing();
        if (kind != Map && kind != Namespace) panic("a template reads the attribute %s of %s", name.c_str(), kind_name());
        for (const auto &entry : fields())
            if (entry.first == name) return entry.second;
        return missing();
    }
    void assign(const std::string &name, Value value) const {  // value.rs:176-188
        if (kind != Namespace) panic("a template writes the attribute %s of %s", name.c_str(), kind_name());
        for (auto &entry : *space)
            if (entry.first == name) {
                entry.second = std::move(value);
                return;
            }
        space->emplace_back(name, std::move(value));
    }
    // characters of a string, as UTF-8 pieces
    static std::vector<std::string> characters(const std::string &held) {
        std::vector<std::string> out;
        for (size_t at = 0; at < held.size();) {
            size_t wide = 1;
            const unsigned char lead = (unsigned char)held[at];
            if (lead >= 0xf0) wide = 4;
            else if (lead >= 0xe0) wide = 3;
            else if (lead >= 0xc0) wide = 2;
            out.push_back(held.substr(at, wide));
            at += wide;
        }
        return out;
    }
    static size_t within(int64_t at, size_t len) {  // value.rs:366-373
        const int64_t held = at < 0 ? at + (int64_t)len : at;
        if (held < 0 || held >= (int64_t)len) panic("a template reads the element %lld of a list of %zu elements", (long long)at, len);
        return (size_t)held;
    }
    Value subscript(const Value &key) const {  // value.rs:190-215
        if (kind == List && key.kind == Integer) return items[within(key.integer, items.size())];
        if ((kind == Map || kind == Namespace) && key.kind == Text) return attribute(key.string);
        if (kind == Text && key.kind == Integer) {
            auto held = characters(string);
            return of(held[within(key.integer, held.size())]);
        }
        panic("a template reads the %s of %s", key.kind_name(), kind_name());
    }
    Value slice(std::optional<int64_t> start, std::optional<int64_t> stop, std::optional<int64_t> step_held) const {  // value.rs:217-249
        if (kind != List) panic("a template slices %s where a list stands", kind_name());
        const int64_t step = step_held.value_or(1);
        NEURA_ASSERT(step != 0, "a template slices a list by no step at all");
        const int64_t len = (int64_t)items.size();
        auto bound = [len](int64_t at) { return at < 0 ? at + len : at; };
        auto clamp = [](int64_t v, int64_t low, int64_t high) { return v < low ? low : v > high ? high : v; };
        std::vector<Value> out;
        if (step > 0) {
            const int64_t first = start ? clamp(bound(*start), 0, len) : 0, last = stop ? clamp(bound(*stop), 0, len) : len;
            for (int64_t at = first; at < last; at += step) out.push_back(items[(size_t)at]);
        } else {
            const int64_t first = start ? clamp(bound(*start), -1, len - 1) : len - 1, last = stop ? bound(*stop) : -len - 1;
            for (int64_t at = first; at > last; at += step)
                if (at >= 0 && at < len) out.push_back(items[(size_t)at]);
        }
        return list(std::move(out));
    }
    bool contains(const Value &other) const {  // value.rs:251-266
        if (kind == Text && other.kind == Text) return string.find(other.string) != std::string::npos;
        if (kind == List) return std::any_of(items.begin(), items.end(), [&](const Value &item) { return item.equals(other); });
        if ((kind == Map || kind == Namespace) && other.kind == Text)
            return std::any_of(fields().begin(), fields().end(), [&](const auto &entry) { return entry.first == other.string; });
        panic("a template asks whether %s holds %s", kind_name(), other.kind_name());
    }
    size_t length() const {  // value.rs:268-277
        switch (kind) {
        case Missing: return 0;
        case Text: return characters(string).size();
        case List: return items.size();
        case Map: case Namespace: return fields().size();
        default: panic("a template measures the length of %s", kind_name());
        }
    }
    // str.strip / lstrip / rstrip: whitespace, or the characters of `set`
    static std::string stripped(const std::string &held, const std::vector<std::string> *set, bool left, bool right) {
        auto pieces = characters(held);
        auto drops = [&](const std::string &piece) {
            if (set) return std::find(set->begin(), set->end(), piece) != set->end();
            size_t wide;
            return space_at(piece, 0, wide);
        };
        size_t first = 0, last = pieces.size();
        while (left && first < last && drops(pieces[first])) first++;
        while (right && last > first && drops(pieces[last - 1])) last--;
        std::string out;
        for (size_t i = first; i < last; i++) out += pieces[i];
        return out;
    }
    Value method(const std::string &name, const std::vector<Value> &arguments) const {  // value.rs:279-325
        if (kind != Text) panic("a template calls %s on %s", name.c_str(), kind_name());
        auto first = [&]() {
            if (arguments.empty()) panic("a template calls %s with no argument", name.c_str());
            return arguments.front().text();
        };
        if (name == "split") {
            const std::string by = first();
            std::vector<Value> out;
            if (by.empty()) {  // str::split("") yields the empty ends and every character between
                out.push_back(of(""));
                for (const auto &piece : characters(string)) out.push_back(of(piece));
                out.push_back(of(""));
                return list(std::move(out));
            }
            size_t at = 0;
            for (;;) {
                const size_t found = string.find(by, at);
                out.push_back(of(string.substr(at, found == std::string::npos ? std::string::npos : found - at)));
                if (found == std::string::npos) break;
                at = found + by.size();
            }
            return list(std::move(out));
        }
        if (name == "strip" || name == "lstrip" || name == "rstrip") {
            std::vector<std::string> set;
            if (!arguments.empty()) set = characters(first());
            return of(stripped(string, arguments.empty() ? nullptr : &set, name != "rstrip", name != "lstrip"));
        }
        if (name == "startswith") {
            const std::string with = first();
            return of(string.size() >= with.size() && string.compare(0, with.size(), with) == 0);
        }
        if (name == "endswith") {
            const std::string with = first();
            return of(string.size() >= with.size() && string.compare(string.size() - with.size(), with.size(), with) == 0);
        }
        panic("a template calls %s on a string, and this renderer reads no such method", name.c_str());
    }
    std::string json() const {  // value.rs:327-385
        switch (kind) {
        case Missing: case Empty: return "null";
        case Flag: return flag ? "true" : "false";
        case Integer: return std::to_string(integer);
        case Number: return digits(number);
        case Text: {
            std::string out = "\"";
            char room[16];
            for (size_t at = 0; at < string.size();) {
                // one character: its code point
                const unsigned char lead = (unsigned char)string[at];
                uint32_t code = lead;
                size_t wide = 1;
                if (lead >= 0xf0) code = lead & 7u, wide = 4;
                else if (lead >= 0xe0) code = lead & 15u, wide = 3;
                else if (lead >= 0xc0) code = lead & 31u, wide = 2;
                for (size_t k = 1; k < wide && at + k < string.size(); k++) code = code << 6 | ((unsigned char)string[at + k] & 63u);
                at += wide;
                switch (code) {
                case '"': out += "\\\""; break;
                case '\\': out += "\\\\"; break;
                case '\n': out += "\\n"; break;
                case '\r': out += "\\r"; break;
                case '\t': out += "\\t"; break;
                case '<': out += "\\u003c"; break;
                case '>': out += "\\u003e"; break;
                case '&': out += "\\u0026"; break;
                case '\'': out += "\\u0027"; break;
                default:
                    if (code >= 0x20 && code <= 0x7e) {
                        out += (char)code;
                    } else if (code <= 0xffff) {
                        snprintf(room, sizeof(room), "\\u%04x", code);
                        out += room;
                    } else {
                        const uint32_t held = code - 0x10000;
                        snprintf(room, sizeof(room), "\\u%04x\\u%04x", 0xd800 + (held >> 10), 0xdc00 + (held & 0x3ff));
                        out += room;
                    }
                }
            }
            return out + "\"";
        }
        case List: {
            std::string out = "[";
            for (size_t i = 0; i < items.size(); i++) out += (i ? ", " : "") + items[i].json();
            return out + "]";
        }
        default: {
            Entries sorted = fields();
            std::stable_sort(sorted.begin(), sorted.end(), [](const auto &left, const auto &right) { return left.first < right.first; });
            std::string out = "{";
            for (size_t i = 0; i < sorted.size(); i++) out += (i ? ", " : "") + of(sorted[i].first).json() + ": " + sorted[i].second.json();
            return out + "}";
        }
        }
    }
};

// ---- tokens (crates/neura-template/src/lexer.rs) ------------------------------------------------
struct Token {
    enum Kind { Body, Print, Block, Close, Name, Text, Whole, Decimal, Symbol };
    Kind kind;
    std::string text;
    int64_t whole = 0;
    double decimal = 0.0;
    std::string shown() const {
        switch (kind) {
        case Body: return "Body(" + Value::of(text).repr() + ")";
        case Print: return "Print";
        case Block: return "Block";
        case Close: return "Close";
        case Name: return "Name(\"" + text + "\")";
        case Text: return "Text(\"" + text + "\")";
        case Whole: return "Whole(" + std::to_string(whole) + ")";
        case Decimal: return "Decimal(" + Value::digits(decimal) + ")";
        default: return "Symbol(\"" + text + "\")";
        }
    }
};

// the words of a tag: names, quoted strings, numbers, symbols (lexer.rs:104-154)
inline void words(const std::string &source, std::vector<Token> &held) {
    static const char *doubles[] = {"**", "//", "==", "!=", "<=", ">="};
    for (size_t at = 0; at < source.size();) {
        size_t wide;
        if (space_at(source, at, wide)) {
            at += wide;
            continue;
        }
        const char character = source[at];
        if (character == '\'' || character == '"') {  // lexer.rs:156-184
            std::string text;
            size_t cursor = at + 1;
            bool closed = false;
            while (cursor < source.size()) {
                const char c = source[cursor++];
                if (c == character) {
                    closed = true;
                    break;
                }
                if (c != '\\') {
                    text += c;
                    continue;
                }
                if (cursor >= source.size()) panic("a template ends a string with a backslash that escapes nothing");
                const char escaped = source[cursor++];
                text += escaped == 'n' ? '\n' : escaped == 't' ? '\t' : escaped == 'r' ? '\r' : escaped == '0' ? '\0' : escaped;
            }
            if (!closed) panic("a template opens the string %s and holds no %c that closes it", Value::of(text).repr().c_str(), character);
            held.push_back({Token::Text, text});
            at = cursor;
            continue;
        }
        if (std::isdigit((unsigned char)character)) {  // lexer.rs:186-220
            size_t cursor = at;
            bool decimal = false;
            while (cursor < source.size() && (std::isdigit((unsigned char)source[cursor]) || (source[cursor] == '.' && !decimal))) {
                decimal |= source[cursor] == '.';
                cursor++;
            }
            const std::string digits = source.substr(at, cursor - at);
            Token token{decimal ? Token::Decimal : Token::Whole, digits};
            try {
                if (decimal) token.decimal = std::stod(digits);
                else token.whole = std::stoll(digits);
            } catch (const std::exception &) {
                panic(decimal ? "a template holds %s where a number stands" : "a template holds %s where a whole number stands", digits.c_str());
            }
            held.push_back(token);
            at = cursor;
            continue;
        }
        if (std::isalpha((unsigned char)character) || character == '_' || (unsigned char)character >= 0x80) {
            size_t cursor = at;
            while (cursor < source.size() && (std::isalnum((unsigned char)source[cursor]) || source[cursor] == '_' || (unsigned char)source[cursor] >= 0x80)) cursor++;
            held.push_back({Token::Name, source.substr(at, cursor - at)});
            at = cursor;
            continue;
        }
        bool found = false;
        for (const char *symbol : doubles)
            if (source.compare(at, 2, symbol) == 0) {
                held.push_back({Token::Symbol, symbol});
                at += 2, found = true;
                break;
            }
        if (found) continue;
        if (std::strchr("+-*/%~=,.:|()[]<>", character) == nullptr)
            panic("a tag of a template holds the character %c where this renderer reads no part of an expression", character);
        held.push_back({Token::Symbol, std::string(1, character)});
        at++;
    }
}

inline std::vector<Token> lex(const std::string &source) {  // lexer.rs:30-102
    std::vector<Token> held;
    std::string body;
    bool trim = false;
    size_t at = 0;
    while (at < source.size()) {
        const bool print = source.compare(at, 2, "{{") == 0, block = source.compare(at, 2, "{%") == 0, comment = source.compare(at, 2, "{#") == 0;
        if (!print && !block && !comment) {
            size_t wide;
            const bool blank = space_at(source, at, wide);
            if (trim && blank) {
                at += wide;
                continue;
            }
            trim = false;
            body.append(source, at, wide);
            at += wide;
            continue;
        }
        at += 2;
        const bool left = at < source.size() && source[at] == '-';
        if (left) at++;
        const char *closer = print ? "}}" : block ? "%}" : "#}";
        const size_t end = source.find(closer, at);
        if (end == std::string::npos) panic("a template opens a tag at byte %zu and holds no %s that closes it", at, closer);
        std::string inner = source.substr(at, end - at);
        const bool right = !inner.empty() && inner.back() == '-';
        if (right) inner.pop_back();
        at = end + 2;
        if (left) body = Value::stripped(body, nullptr, false, true);
        if (!body.empty()) {
            held.push_back({Token::Body, body});
            body.clear();
        }
        trim = right;
        if (comment) continue;
        held.push_back({print ? Token::Print : Token::Block, ""});
        words(inner, held);
        held.push_back({Token::Close, ""});
    }
    if (!body.empty()) held.push_back({Token::Body, body});
    return held;
}

// ---- syntax (crates/neura-template/src/syntax.rs) -----------------------------------------------
struct Expression;
using Held = std::unique_ptr<Expression>;
struct Expression {
    enum Kind { Literal, Name, Attribute, Index, Slice, Call, Filter, Test, Conditional, Negate, Not, And, Or, Compare, Add, Subtract, Concat };
    enum Comparison { Equal, NotEqual, Less, LessEqual, Greater, GreaterEqual, In, NotIn };
    Kind kind;
    Value value;        // Literal
    std::string name;   // Name, Attribute, Filter, Test
    Held a, b, c, d;    // operands: base / left / accept, key / right / condition, reject / stop, step
    std::vector<Held> positional;
    std::vector<std::pair<std::string, Held>> keywords;
    Comparison comparison = Equal;
    bool negated = false;
    explicit Expression(Kind kind) : kind(kind) {}
};
struct Statement {
    enum Kind { Body, Print, If, For, Set, Macro };
    Kind kind;
    std::string text, name, attribute;  // Body; For / Set / Macro names; Set's attribute ("" = none)
    Held expression;                    // Print, For source, Set value
    std::vector<std::pair<Held, std::vector<Statement>>> arms;  // If
    std::vector<Statement> body;        // For, Macro; If's otherwise
    std::vector<std::pair<std::string, Held>> parameters;       // Macro
    explicit Statement(Kind kind) : kind(kind) {}
};

// ---- parser (crates/neura-template/src/parser.rs) -----------------------------------------------
class Parser {
  public:
    explicit Parser(std::vector<Token> tokens) : tokens_(std::move(tokens)) {}
    std::vector<Statement> program() {
        auto held = statements({});
        if (peek()) panic("a template holds %s where its end stands", peek()->shown().c_str());
        return held;
    }

  private:
    std::vector<Statement> statements(const std::vector<std::string> &ends) {
        std::vector<Statement> held;
        while (const Token *token = peek()) {
            if (token->kind == Token::Body) {
                Statement body(Statement::Body);
                body.text = token->text;
                at_++;
                held.push_back(std::move(body));
            } else if (token->kind == Token::Print) {
                at_++;
                Statement print(Statement::Print);
                print.expression = expression();
                close();
                held.push_back(std::move(print));
            } else if (token->kind == Token::Block) {
                const std::string name = tag_name();
                if (std::find(ends.begin(), ends.end(), name) != ends.end()) return held;
                held.push_back(statement(name));
            } else {
                panic("a template holds %s where a body stands", token->shown().c_str());
            }
        }
        if (!ends.empty()) {
            std::string joined;
            for (size_t i = 0; i < ends.size(); i++) joined += (i ? " or " : "") + ends[i];
            panic("a template ends where its %s stands", joined.c_str());
        }
        return held;
    }
    Statement statement(const std::string &name) {
        if (name == "if") return if_statement();
        if (name == "for") return for_statement();
        if (name == "set") return set_statement();
        if (name == "macro") return macro_statement();
        panic("a template holds the %s tag, and this renderer reads no such tag", name.c_str());
    }
    Statement if_statement() {  // parser.rs:66-107
        Statement held(Statement::If);
        open("if");
        for (;;) {
            Held condition = expression();
            close();
            held.arms.emplace_back(std::move(condition), statements({"elif", "else", "endif"}));
            const std::string name = tag_name();
            if (name == "elif") {
                open("elif");
                continue;
            }
            if (name == "else") {
                open("else");
                close();
                held.body = statements({"endif"});
            } else if (name != "endif") {
                panic("a template holds the %s tag where an if ends", name.c_str());
            }
            open("endif");
            close();
            return held;
        }
    }
    Statement for_statement() {  // parser.rs:109-120
        Statement held(Statement::For);
        open("for");
        held.name = name();
        expect_name("in");
        held.expression = expression();
        close();
        held.body = statements({"endfor"});
        open("endfor");
        close();
        return held;
    }
    Statement set_statement() {  // parser.rs:122-139
        Statement held(Statement::Set);
        open("set");
        held.name = name();
        if (take_symbol(".")) held.attribute = name();
        expect_symbol("=");
        held.expression = expression();
        close();
        return held;
    }
    Statement macro_statement() {  // parser.rs:141-168
        Statement held(Statement::Macro);
        open("macro");
        held.name = name();
        expect_symbol("(");
        while (!take_symbol(")")) {
            std::string parameter = name();
            Held fallback;
            if (take_symbol("=")) fallback = expression();
            held.parameters.emplace_back(std::move(parameter), std::move(fallback));
            if (!take_symbol(",")) {
                expect_symbol(")");
                break;
            }
        }
        close();
        held.body = statements({"endmacro"});
        open("endmacro");
        close();
        return held;
    }

    static Held make(Expression::Kind kind, Held a = nullptr, Held b = nullptr) {
        auto held = std::make_unique<Expression>(kind);
        held->a = std::move(a), held->b = std::move(b);
        return held;
    }
    Held expression() { return conditional(); }
    Held conditional() {  // parser.rs:174-187
        Held accept = either();
        if (!take_name("if")) return accept;
        Held condition = either();
        expect_name("else");
        auto held = make(Expression::Conditional, std::move(accept), std::move(condition));
        held->c = conditional();
        return held;
    }
    Held either() {
        Held held = both();
        while (take_name("or")) held = make(Expression::Or, std::move(held), both());
        return held;
    }
    Held both() {
        Held held = negation();
        while (take_name("and")) held = make(Expression::And, std::move(held), negation());
        return held;
    }
    Held negation() {
        if (take_name("not")) return make(Expression::Not, negation());
        return comparison();
    }
    Held comparison() {  // parser.rs:212-260
        Held held = addition();
        for (;;) {
            Expression::Comparison compare;
            if (take_symbol("==")) compare = Expression::Equal;
            else if (take_symbol("!=")) compare = Expression::NotEqual;
            else if (take_symbol("<=")) compare = Expression::LessEqual;
            else if (take_symbol(">=")) compare = Expression::GreaterEqual;
            else if (take_symbol("<")) compare = Expression::Less;
            else if (take_symbol(">")) compare = Expression::Greater;
            else if (take_name("in")) compare = Expression::In;
            else if (at_name("not") && at_name_at(1, "in")) at_ += 2, compare = Expression::NotIn;
            else if (take_name("is")) {
                auto test = make(Expression::Test, std::move(held));
                test->negated = take_name("not");
                test->name = name();
                if (take_symbol("(")) arguments(*test, false);
                held = std::move(test);
                continue;
            } else {
                break;
            }
            auto compared = make(Expression::Compare, std::move(held), addition());
            compared->comparison = compare;
            held = std::move(compared);
        }
        return held;
    }
    Held addition() {
        Held held = concat();
        for (;;) {
            if (take_symbol("+")) held = make(Expression::Add, std::move(held), concat());
            else if (take_symbol("-")) held = make(Expression::Subtract, std::move(held), concat());
            else return held;
        }
    }
    Held concat() {
        Held held = filtered();
        while (take_symbol("~")) held = make(Expression::Concat, std::move(held), filtered());
        return held;
    }
    Held filtered() {  // parser.rs:284-301
        Held held = postfix();
        while (take_symbol("|")) {
            auto filter = make(Expression::Filter, std::move(held));
            filter->name = name();
            if (take_symbol("(")) arguments(*filter, false);
            held = std::move(filter);
        }
        return held;
    }
    Held postfix() {  // parser.rs:303-323
        Held held = primary();
        for (;;) {
            if (take_symbol(".")) {
                auto attribute = make(Expression::Attribute, std::move(held));
                attribute->name = name();
                held = std::move(attribute);
            } else if (take_symbol("[")) {
                held = subscript(std::move(held));
            } else if (take_symbol("(")) {
                auto call = make(Expression::Call, std::move(held));
                arguments(*call, true);
                held = std::move(call);
            } else {
                return held;
            }
        }
    }
    Held subscript(Held base) {  // parser.rs:325-357
        Held start;
        if (!at_symbol(":")) start = expression();
        if (!take_symbol(":")) {
            expect_symbol("]");
            if (!start) panic("a template reads the element of a list no index names");
            return make(Expression::Index, std::move(base), std::move(start));
        }
        auto slice = make(Expression::Slice, std::move(base), std::move(start));
        if (!at_symbol(":") && !at_symbol("]")) slice->c = expression();
        if (take_symbol(":")) slice->d = expression();
        expect_symbol("]");
        return slice;
    }
    // the arguments of a call, a filter or a test, behind their "(" (parser.rs:359-380); filters and tests read no keywords
    void arguments(Expression &into, bool keywords) {
        if (take_symbol(")")) return;
        for (;;) {
            const bool keyword = peek() && peek()->kind == Token::Name && at_symbol_at(1, "=");
            if (keyword) {
                std::string key = name();
                expect_symbol("=");
                Held value = expression();
                if (keywords) into.keywords.emplace_back(std::move(key), std::move(value));
            } else {
                into.positional.push_back(expression());
            }
            if (take_symbol(",")) continue;
            expect_symbol(")");
            return;
        }
    }
    Held primary() {  // parser.rs:382-423
        const Token *token = peek();
        if (!token) panic("a template ends where an expression stands");
        auto literal = [&](Value value) {
            at_++;
            auto held = make(Expression::Literal);
            held->value = std::move(value);
            return held;
        };
        switch (token->kind) {
        case Token::Name: {
            if (token->text == "true") return literal(Value::of(true));
            if (token->text == "false") return literal(Value::of(false));
            if (token->text == "none") return literal(Value::empty());
            auto held = make(Expression::Name);
            held->name = token->text;
            at_++;
            return held;
        }
        case Token::Text: return literal(Value::of(token->text));
        case Token::Whole: return literal(Value::of(token->whole));
        case Token::Decimal: return literal(Value::of(token->decimal));
        case Token::Symbol:
            if (token->text == "-") {
                at_++;
                return make(Expression::Negate, negation());
            }
            if (token->text == "+") {
                at_++;
                return negation();
            }
            if (token->text == "(") {
                at_++;
                Held held = expression();
                expect_symbol(")");
                return held;
            }
            [[fallthrough]];
        default: panic("a template holds %s where an expression stands", token->shown().c_str());
        }
    }

    const Token *peek(size_t skip = 0) const { return at_ + skip < tokens_.size() ? &tokens_[at_ + skip] : nullptr; }
    static std::string shown(const Token *token) { return token ? "Some(" + token->shown() + ")" : "None"; }
    std::string tag_name() const {
        if (!peek() || peek()->kind != Token::Block) panic("a template holds %s where a tag stands", shown(peek()).c_str());
        if (!peek(1) || peek(1)->kind != Token::Name) panic("a template holds %s where a tag names itself", shown(peek(1)).c_str());
        return peek(1)->text;
    }
    void open(const char *tag) {
        const std::string held = tag_name();
        if (held != tag) panic("a template closes the %s tag with %s", tag, held.c_str());
        at_++;
        expect_name(tag);
    }
    void close() {
        if (!peek() || peek()->kind != Token::Close) panic("a template holds %s where a tag ends", shown(peek()).c_str());
        at_++;
    }
    std::string name() {
        if (!peek() || peek()->kind != Token::Name) panic("a template holds %s where a name stands", shown(peek()).c_str());
        return tokens_[at_++].text;
    }
    void expect_name(const char *wanted) {
        const std::string held = name();
        if (held != wanted) panic("a template holds %s where %s stands", held.c_str(), wanted);
    }
    bool at_name(const char *wanted) const { return at_name_at(0, wanted); }
    bool at_name_at(size_t skip, const char *wanted) const { return peek(skip) && peek(skip)->kind == Token::Name && peek(skip)->text == wanted; }
    bool take_name(const char *wanted) { return at_name(wanted) ? (at_++, true) : false; }
    bool at_symbol(const char *wanted) const { return at_symbol_at(0, wanted); }
    bool at_symbol_at(size_t skip, const char *wanted) const { return peek(skip) && peek(skip)->kind == Token::Symbol && peek(skip)->text == wanted; }
    bool take_symbol(const char *wanted) { return at_symbol(wanted) ? (at_++, true) : false; }
    void expect_symbol(const char *wanted) {
        if (!peek() || peek()->kind != Token::Symbol) panic("a template holds %s where %s stands", shown(peek()).c_str(), wanted);
        if (peek()->text != wanted) panic("a template holds %s where %s stands", peek()->text.c_str(), wanted);
        at_++;
    }
    std::vector<Token> tokens_;
    size_t at_ = 0;
};

// ---- messages and the template (crates/neura-template/src/template.rs) ---------------------------
class Message {
  public:
    Message(std::string role, Value content) : role_(std::move(role)), content_(std::move(content)) {}
    Message with(const std::string &name, Value value) && {
        NEURA_ASSERT(name != "role" && name != "content", "a message walks under its role and its content, and %s names one of them", name.c_str());
        held_.emplace_back(name, std::move(value));
        return std::move(*this);
    }
    const std::string &role() const { return role_; }
    const Value &content() const { return content_; }
    const Value::Entries &held() const { return held_; }

  private:
    std::string role_;
    Value content_;
    Value::Entries held_;
};

// ---- renderer (crates/neura-template/src/render.rs) ---------------------------------------------
class Renderer {
  public:
    static std::string render(const std::vector<Statement> &body, const std::vector<Message> &messages, const Value::Entries &values) {
        Renderer held;
        held.scopes_.emplace_back();
        std::vector<Value> walked;
        for (const Message &message : messages) {
            Value::Entries entries = {{"role", Value::of(message.role())}, {"content", message.content()}};
            entries.insert(entries.end(), message.held().begin(), message.held().end());
            walked.push_back(Value::map(std::move(entries)));
        }
        held.bind("messages", Value::list(std::move(walked)));
        for (const auto &entry : values) held.bind(entry.first, entry.second);
        held.run(body);
        return held.out_;
    }

  private:
    void run(const std::vector<Statement> &body) {
        for (const Statement &held : body) statement(held);
    }
    void statement(const Statement &held) {
        switch (held.kind) {
        case Statement::Body: out_ += held.text; return;
        case Statement::Print: out_ += evaluate(*held.expression).text(); return;
        case Statement::If:
            for (const auto &arm : held.arms)
                if (evaluate(*arm.first).truth()) return run(arm.second);
            return run(held.body);
        case Statement::For: {  // render.rs:68-96
            Value walked = evaluate(*held.expression);
            std::vector<Value> items;
            if (walked.kind == Value::List) items = std::move(walked.items);
            else if (walked.kind == Value::Map)
                for (const auto &entry : walked.entries) items.push_back(Value::of(entry.first));
            else if (walked.kind == Value::Text)
                for (const auto &piece : Value::characters(walked.string)) items.push_back(Value::of(piece));
            else panic("a template walks %s where a list stands", walked.kind_name());
            for (size_t at = 0; at < items.size(); at++) {
                const int64_t length = (int64_t)items.size();
                Value loop = Value::map({{"index0", Value::of((int64_t)at)}, {"index", Value::of((int64_t)at + 1)}, {"first", Value::of(at == 0)},
                                         {"last", Value::of(at + 1 == items.size())}, {"length", Value::of(length)},
                                         {"previtem", at == 0 ? Value::missing() : items[at - 1]},
                                         {"nextitem", at + 1 == items.size() ? Value::missing() : items[at + 1]}});
                scopes_.push_back({{held.name, items[at]}, {"loop", std::move(loop)}});
                run(held.body);
                scopes_.pop_back();
            }
            return;
        }
        case Statement::Set: {
            Value value = evaluate(*held.expression);
            if (held.attribute.empty()) bind(held.name, std::move(value));
            else lookup(held.name).assign(held.attribute, std::move(value));
            return;
        }
        case Statement::Macro: macros_.push_back(&held); return;
        }
    }
    static double real(const Value &held) { return held.kind == Value::Integer ? (double)held.integer : held.number; }
    Value evaluate(const Expression &held) {
        switch (held.kind) {
        case Expression::Literal: return held.value;
        case Expression::Name: return lookup(held.name);
        case Expression::Attribute: return evaluate(*held.a).attribute(held.name);
        case Expression::Index: {
            const Value base = evaluate(*held.a), key = evaluate(*held.b);
            return base.subscript(key);
        }
        case Expression::Slice: {
            const Value base = evaluate(*held.a);
            auto whole = [&](const Held &part) -> std::optional<int64_t> {
                if (!part) return std::nullopt;
                const Value value = evaluate(*part);
                if (value.kind != Value::Integer) panic("a template slices a list by %s", value.kind_name());
                return value.integer;
            };
            const auto start = whole(held.b), stop = whole(held.c), step = whole(held.d);
            return base.slice(start, stop, step);
        }
        case Expression::Call: {
            std::vector<Value> positional;
            for (const Held &argument : held.positional) positional.push_back(evaluate(*argument));
            Value::Entries keywords;
            for (const auto &argument : held.keywords) keywords.emplace_back(argument.first, evaluate(*argument.second));
            return call(*held.a, positional, keywords);
        }
        case Expression::Filter: {
            Value input = evaluate(*held.a);
            if (!held.positional.empty())
                panic("the template filters a value through the %s filter, and this renderer reads no argument of it", held.name.c_str());
            if (held.name == "trim") return Value::of(Value::stripped(input.text(), nullptr, true, true));
            if (held.name == "string") return Value::of(input.text());
            if (held.name == "safe") return input;
            if (held.name == "length") return Value::of((int64_t)input.length());
            if (held.name == "tojson") return Value::of(input.json());
            panic("the template filters a value through %s, and this renderer reads no such filter", held.name.c_str());
        }
        case Expression::Test: {
            const Value input = evaluate(*held.a);
            const bool answer = holds(input, held.name, !held.positional.empty());
            return Value::of(held.negated ? !answer : answer);
        }
        case Expression::Conditional: return evaluate(*held.b).truth() ? evaluate(*held.a) : evaluate(*held.c);
        case Expression::Negate: {
            const Value value = evaluate(*held.a);
            if (value.kind == Value::Integer) return Value::of(-value.integer);
            if (value.kind == Value::Number) return Value::of(-value.number);
            panic("a template negates %s", value.kind_name());
        }
        case Expression::Not: return Value::of(!evaluate(*held.a).truth());
        case Expression::And: {
            Value left = evaluate(*held.a);
            return left.truth() ? evaluate(*held.b) : left;
        }
        case Expression::Or: {
            Value left = evaluate(*held.a);
            return left.truth() ? left : evaluate(*held.b);
        }
        case Expression::Compare: {  // render.rs:322-333
            const Value left = evaluate(*held.a), right = evaluate(*held.b);
            switch (held.comparison) {
            case Expression::Equal: return Value::of(left.equals(right));
            case Expression::NotEqual: return Value::of(!left.equals(right));
            case Expression::Less: return Value::of(right.greater(left));
            case Expression::LessEqual: return Value::of(!left.greater(right));
            case Expression::Greater: return Value::of(left.greater(right));
            case Expression::GreaterEqual: return Value::of(!right.greater(left));
            case Expression::In: return Value::of(right.contains(left));
            default: return Value::of(!right.contains(left));
            }
        }
        case Expression::Add: {
            const Value left = evaluate(*held.a), right = evaluate(*held.b);
            return left.add(right);
        }
        case Expression::Subtract: {  // render.rs:335-343
            const Value left = evaluate(*held.a), right = evaluate(*held.b);
            const bool numeric = (left.kind == Value::Integer || left.kind == Value::Number) && (right.kind == Value::Integer || right.kind == Value::Number);
            if (!numeric) panic("a template takes %s from %s", right.kind_name(), left.kind_name());
            if (left.kind == Value::Integer && right.kind == Value::Integer) return Value::of(left.integer - right.integer);
            return Value::of(real(left) - real(right));
        }
        case Expression::Concat: {
            const Value left = evaluate(*held.a), right = evaluate(*held.b);
            return Value::of(left.text() + right.text());
        }
        }
        return Value::missing();
    }
    Value call(const Expression &callee, const std::vector<Value> &positional, const Value::Entries &keywords) {  // render.rs:241-262
        if (callee.kind == Expression::Attribute) return evaluate(*callee.a).method(callee.name, positional);
        if (callee.kind != Expression::Name)
            panic("a template calls a value this renderer reads no callee of, and it calls macros and functions by name");
        if (callee.name == "namespace") return Value::names(keywords);
        if (callee.name == "raise_exception") panic("the template raises %s", positional.empty() ? "an exception" : positional.front().text().c_str());
        return invoke(callee.name, positional, keywords);
    }
    Value invoke(const std::string &name, const std::vector<Value> &positional, const Value::Entries &keywords) {  // render.rs:264-303
        const Statement *macro = nullptr;
        for (auto held = macros_.rbegin(); held != macros_.rend() && !macro; ++held)
            if ((*held)->name == name) macro = *held;
        if (!macro) panic("a template calls %s, and this renderer reads no such macro or function", name.c_str());
        const auto &parameters = macro->parameters;
        bool fits = positional.size() <= parameters.size();
        for (const auto &keyword : keywords)
            fits = fits && std::any_of(parameters.begin(), parameters.end(), [&](const auto &parameter) { return parameter.first == keyword.first; });
        if (!fits) panic("the template calls the macro %s with an argument it names no parameter for", name.c_str());
        Value::Entries scope;
        for (size_t at = 0; at < parameters.size(); at++) {
            Value value = Value::missing();
            auto named = std::find_if(keywords.begin(), keywords.end(), [&](const auto &keyword) { return keyword.first == parameters[at].first; });
            if (at < positional.size()) value = positional[at];
            else if (named != keywords.end()) value = named->second;
            else if (parameters[at].second) value = evaluate(*parameters[at].second);
            scope.emplace_back(parameters[at].first, std::move(value));
        }
        scopes_.push_back(std::move(scope));
        std::string saved;
        saved.swap(out_);
        run(macro->body);
        saved.swap(out_);
        scopes_.pop_back();
        return Value::of(saved);
    }
    static bool holds(const Value &value, const std::string &name, bool with_arguments) {  // render.rs:396-423
        if (with_arguments) panic("the template weighs a value against the %s test, and this renderer reads no argument of it", name.c_str());
        if (name == "defined") return value.kind != Value::Missing;
        if (name == "undefined") return value.kind == Value::Missing;
        if (name == "none") return value.kind == Value::Empty;
        if (name == "string") return value.kind == Value::Text;
        if (name == "number") return value.kind == Value::Integer || value.kind == Value::Number;
        if (name == "integer") return value.kind == Value::Integer;
        if (name == "boolean") return value.kind == Value::Flag;
        if (name == "true") return value.kind == Value::Flag && value.flag;
        if (name == "false") return value.kind == Value::Flag && !value.flag;
        if (name == "iterable") return value.kind == Value::Text || value.kind == Value::List || value.kind == Value::Map;
        if (name == "mapping") return value.kind == Value::Map || value.kind == Value::Namespace;
        if (name == "sequence") return value.kind == Value::Text || value.kind == Value::List;
        panic("the template weighs a value against the %s test, and this renderer reads no such test", name.c_str());
    }
    void bind(const std::string &name, Value value) {
        for (auto &entry : scopes_.back())
            if (entry.first == name) {
                entry.second = std::move(value);
                return;
            }
        scopes_.back().emplace_back(name, std::move(value));
    }
    Value lookup(const std::string &name) const {
        for (auto scope = scopes_.rbegin(); scope != scopes_.rend(); ++scope)
            for (const auto &entry : *scope)
                if (entry.first == name) return entry.second;
        return Value::missing();
    }
    std::vector<Value::Entries> scopes_;
    std::vector<const Statement *> macros_;
    std::string out_;
};

class Template {
  public:
    // crates/neura-template/src/template.rs:13-15: the template a GGUF carries
    static Template read(const gguf::Archive &source) { return parse(source.metadata().text("tokenizer.chat_template")); }
    static Template parse(const std::string &source) { return Template(Parser(lex(source)).program()); }
    std::string render(const std::vector<Message> &messages, const Value::Entries &values = {}) const { return Renderer::render(body_, messages, values); }

  private:
    explicit Template(std::vector<Statement> body) : body_(std::move(body)) {}
    std::vector<Statement> body_;
};

}  // namespace chat
}  // namespace neura
