// capi.cpp -- a flat C surface over neura.hpp so the host layer can be driven from scripts and
// tests without a C++ compiler in the loop.  Every call that can be refused returns a status
// (0 done, -1 refused) or a null handle, and nhost_last_error() then holds the sentence the
// reference would have panicked with.
#include "neura.hpp"
#include "template.hpp"
#include "tokenizer.hpp"

#include <cstdlib>

using namespace neura;

namespace {
thread_local std::string last_error;

template <typename F>
auto guarded(F &&body, decltype(body()) refused) -> decltype(body()) {
    try {
        return body();
    } catch (const std::exception &held) {
        last_error = held.what();
        return refused;
    }
}

struct Opened {
    std::unique_ptr<gguf::Gguf> whole;
    std::unique_ptr<gguf::GgufFile> file;
    const gguf::Archive &archive() const { return whole ? static_cast<const gguf::Archive &>(*whole) : *file; }
    const gguf::Source &source() const { return whole ? static_cast<const gguf::Source &>(*whole) : *file; }
};

struct Loaded {
    std::unique_ptr<generate::Model> model;
    std::unique_ptr<generate::Batch> batch;
};

std::unique_ptr<tokenizer::Rule> rule_named(const std::string &name) {
    if (name == "qwen") return std::make_unique<tokenizer::Qwen>();
    if (name == "per_character") return std::make_unique<tokenizer::PerCharacter>();
    if (name == "per_space") return std::make_unique<tokenizer::PerSpace>();
    if (name == "whole") return std::make_unique<tokenizer::Whole>();
    panic("no split rule is named %s", name.c_str());
}
}  // namespace

namespace {
// what a script hands the template engine: JSON text into chat::Value (objects keep their order; a number without a
// fraction or exponent is a whole number)
struct Json {
    const std::string &text;
    size_t at = 0;
    void blanks() {
        while (at < text.size() && std::isspace((unsigned char)text[at])) at++;
    }
    char next() {
        blanks();
        if (at >= text.size()) panic("the json handed to a template ends early");
        return text[at];
    }
    void expect(char wanted) {
        if (next() != wanted) panic("the json handed to a template holds %c where %c stands", text[at], wanted);
        at++;
    }
    static void put(std::string &out, uint32_t code) {
        if (code < 0x80) out += (char)code;
        else if (code < 0x800) out += (char)(0xc0 | code >> 6), out += (char)(0x80 | (code & 63));
        else if (code < 0x10000) out += (char)(0xe0 | code >> 12), out += (char)(0x80 | ((code >> 6) & 63)), out += (char)(0x80 | (code & 63));
        else out += (char)(0xf0 | code >> 18), out += (char)(0x80 | ((code >> 12) & 63)), out += (char)(0x80 | ((code >> 6) & 63)), out += (char)(0x80 | (code & 63));
    }
    uint32_t hex4() {
        if (at + 4 > text.size()) panic("the json handed to a template ends inside an escape");
        const uint32_t code = (uint32_t)std::stoul(text.substr(at, 4), nullptr, 16);
        at += 4;
        return code;
    }
    std::string string() {
        expect('"');
        std::string out;
        while (at < text.size() && text[at] != '"') {
            char c = text[at++];
            if (c != '\\') {
                out += c;
                continue;
            }
            c = text[at++];
            switch (c) {
            case 'n': out += '\n'; break;
            case 't': out += '\t'; break;
            case 'r': out += '\r'; break;
            case 'b': out += '\b'; break;
            case 'f': out += '\f'; break;
            case 'u': {
                uint32_t code = hex4();
                if (code >= 0xd800 && code < 0xdc00 && text.compare(at, 2, "\\u") == 0) {
                    at += 2;
                    code = 0x10000 + ((code - 0xd800) << 10) + (hex4() - 0xdc00);
                }
                put(out, code);
                break;
            }
            default: out += c;
            }
        }
        expect('"');
        return out;
    }
    chat::Value value() {
        const char c = next();
        if (c == '"') return chat::Value::of(string());
        if (c == '{') {
            at++;
            chat::Value::Entries entries;
            if (next() == '}') return at++, chat::Value::map({});
            for (;;) {
                std::string key = string();
                expect(':');
                entries.emplace_back(std::move(key), value());
                if (next() == ',') {
                    at++;
                    continue;
                }
                expect('}');
                return chat::Value::map(std::move(entries));
            }
        }
        if (c == '[') {
            at++;
            std::vector<chat::Value> items;
            if (next() == ']') return at++, chat::Value::list({});
            for (;;) {
                items.push_back(value());
                if (next() == ',') {
                    at++;
                    continue;
                }
                expect(']');
                return chat::Value::list(std::move(items));
            }
        }
        if (text.compare(at, 4, "true") == 0) return at += 4, chat::Value::of(true);
        if (text.compare(at, 5, "false") == 0) return at += 5, chat::Value::of(false);
        if (text.compare(at, 4, "null") == 0) return at += 4, chat::Value::empty();
        size_t end = at;
        bool real = false;
        while (end < text.size() && (std::isdigit((unsigned char)text[end]) || std::strchr("+-.eE", text[end]))) real |= std::strchr(".eE", text[end]) != nullptr, end++;
        if (end == at) panic("the json handed to a template holds %c where a value stands", c);
        const std::string digits = text.substr(at, end - at);
        at = end;
        return real ? chat::Value::of(std::stod(digits)) : chat::Value::of((int64_t)std::stoll(digits));
    }
};

int64_t rendered(const chat::Template &held, const char *messages_json, const char *values_json, char *out, size_t room) {
    const std::string messages_text = messages_json ? messages_json : "[]", values_text = values_json ? values_json : "{}";
    const chat::Value listed = Json{messages_text}.value(), named = Json{values_text}.value();
    if (listed.kind != chat::Value::List || named.kind != chat::Value::Map) panic("a template renders a list of messages and a mapping of values");
    std::vector<chat::Message> messages;
    for (const chat::Value &entry : listed.items) {
        if (entry.kind != chat::Value::Map) panic("a message handed to a template is a mapping");
        chat::Message message(entry.attribute("role").text(), entry.attribute("content"));
        for (const auto &field : entry.entries)
            if (field.first != "role" && field.first != "content") message = std::move(message).with(field.first, field.second);
        messages.push_back(std::move(message));
    }
    const std::string text = held.render(messages, named.entries);
    for (size_t i = 0; i < text.size() && i < room; i++) out[i] = text[i];
    return (int64_t)text.size();
}
}  // namespace

struct nhost_tensor {
    int32_t element;
    uint32_t rank;
    uint64_t elements, shape[4], at, bytes;
};

extern "C" {

const char *nhost_last_error(void) { return last_error.c_str(); }

// ---- GGUF ---------------------------------------------------------------------------------------
void *nhost_gguf_decode(const uint8_t *bytes, size_t size) {
    return guarded([&]() -> void * {
        auto out = std::make_unique<Opened>();
        out->whole = std::make_unique<gguf::Gguf>(gguf::Gguf::decode(bytes, size));
        return out.release();
    }, nullptr);
}
void *nhost_gguf_open(const char *path) {
    return guarded([&]() -> void * {
        auto out = std::make_unique<Opened>();
        out->file = gguf::GgufFile::open(path);
        return out.release();
    }, nullptr);
}
void nhost_gguf_close(void *held) { delete static_cast<Opened *>(held); }
uint64_t nhost_gguf_tensors(void *held) {
    auto *opened = static_cast<Opened *>(held);
    return opened->whole ? opened->whole->tensors() : opened->file->tensors();
}
uint64_t nhost_gguf_reads(void *held) {
    auto *opened = static_cast<Opened *>(held);
    return opened->file ? opened->file->reads() : 0;
}
// 1 found, 0 absent
int32_t nhost_gguf_tensor(void *held, const char *name, nhost_tensor *out) {
    auto found = static_cast<Opened *>(held)->archive().tensor(name);
    if (!found) return 0;
    out->element = (int32_t)found->element, out->rank = found->rank, out->elements = found->elements;
    for (int d = 0; d < 4; d++) out->shape[d] = found->shape[d];
    out->at = found->at, out->bytes = found->bytes;
    return 1;
}
int32_t nhost_gguf_has(void *held, const char *key) { return static_cast<Opened *>(held)->archive().metadata().has(key); }
int32_t nhost_gguf_word(void *held, const char *key, uint32_t *out) {
    return guarded([&] { return *out = static_cast<Opened *>(held)->archive().metadata().word(key), 0; }, -1);
}
int32_t nhost_gguf_single(void *held, const char *key, float *out) {
    return guarded([&] { return *out = static_cast<Opened *>(held)->archive().metadata().single(key), 0; }, -1);
}
int32_t nhost_gguf_flag(void *held, const char *key, int32_t *out) {
    return guarded([&] { return *out = static_cast<Opened *>(held)->archive().metadata().flag(key), 0; }, -1);
}
// the bytes of the string, at most `room` of them; returns its length or -1
int64_t nhost_gguf_text(void *held, const char *key, char *out, size_t room) {
    return guarded([&]() -> int64_t {
        std::string text = static_cast<Opened *>(held)->archive().metadata().text(key);
        memcpy(out, text.data(), std::min(room, text.size()));
        return (int64_t)text.size();
    }, -1);
}
// integer(): 1 and *out when the value is a whole number, 0 when it is another type, -1 absent
int32_t nhost_gguf_integer(void *held, const char *key, uint64_t *out) {
    return guarded([&] {
        auto found = static_cast<Opened *>(held)->archive().metadata().value(key).integer();
        if (found) *out = *found;
        return found ? 1 : 0;
    }, -1);
}
// length of an array value and, for arrays of strings, the text of entry `index`
int64_t nhost_gguf_array_len(void *held, const char *key) {
    return guarded([&]() -> int64_t { return (int64_t) static_cast<Opened *>(held)->archive().metadata().array(key).size(); }, -1);
}
int64_t nhost_gguf_array_text(void *held, const char *key, uint64_t index, char *out, size_t room) {
    return guarded([&]() -> int64_t {
        auto &items = static_cast<Opened *>(held)->archive().metadata().array(key);
        auto text = items.at(index).text();
        if (!text) panic("entry %llu of the %s of this gguf is %s where a string stands", (unsigned long long)index, key, items.at(index).name());
        memcpy(out, text->data(), std::min(room, text->size()));
        return (int64_t)text->size();
    }, -1);
}
int64_t nhost_gguf_array_number(void *held, const char *key, uint64_t index, double *out) {
    return guarded([&]() -> int64_t {
        auto number = static_cast<Opened *>(held)->archive().metadata().array(key).at(index).number();
        if (!number) return 0;
        *out = *number;
        return 1;
    }, -1);
}
// Source::placed + Source::payload: streams the tensor into out (room bytes), returns its bytes
int64_t nhost_gguf_payload(void *held, const char *name, uint8_t *out, size_t room) {
    return guarded([&]() -> int64_t {
        auto &source = static_cast<Opened *>(held)->source();
        size_t at = 0;
        source.payload(name, [&](const uint8_t *chunk, size_t bytes) {
            if (at + bytes <= room) memcpy(out + at, chunk, bytes);
            at += bytes;
        });
        return (int64_t)at;
    }, -1);
}
int32_t nhost_gguf_placed(void *held, const char *name, int32_t *element, uint64_t *elements, float *scale, uint64_t *payload, uint64_t *table) {
    auto found = static_cast<Opened *>(held)->source().placed(name);
    if (!found) return 0;
    *element = (int32_t)found->element, *elements = found->elements, *scale = found->scale;
    *payload = found->payload_bytes, *table = found->table_bytes;
    return 1;
}

// ---- writer -------------------------------------------------------------------------------------
void *nhost_writer_new(uint64_t alignment) { return new gguf::Writer(alignment); }
void nhost_writer_free(void *writer) { delete static_cast<gguf::Writer *>(writer); }
void nhost_writer_u32(void *writer, const char *key, uint32_t value) { static_cast<gguf::Writer *>(writer)->meta_u32(key, value); }
void nhost_writer_f32(void *writer, const char *key, float value) { static_cast<gguf::Writer *>(writer)->meta_f32(key, value); }
void nhost_writer_text(void *writer, const char *key, const char *value) { static_cast<gguf::Writer *>(writer)->meta_text(key, value); }
void nhost_writer_tensor(void *writer, const char *name, int32_t element, const uint64_t *shape, uint32_t rank, const uint8_t *payload, size_t bytes) {
    static_cast<gguf::Writer *>(writer)->tensor(name, (Element)element, std::vector<uint64_t>(shape, shape + rank), payload, bytes);
}
int32_t nhost_writer_save(void *writer, const char *path) {
    return guarded([&] {
        auto bytes = static_cast<gguf::Writer *>(writer)->bytes();
        std::ofstream out(path, std::ios::binary);
        out.write(reinterpret_cast<const char *>(bytes.data()), (std::streamsize)bytes.size());
        if (!out) panic("a gguf could not be written at %s", path);
        return 0;
    }, -1);
}

// ---- decoder declarations -----------------------------------------------------------------------
int32_t nhost_matrix(void *held, const char *name, uint32_t rows, uint32_t columns, int32_t *element) {
    return guarded([&] { return *element = (int32_t)decoder::matrix(static_cast<Opened *>(held)->archive(), name, rows, columns).element, 0; }, -1);
}
int32_t nhost_vector(void *held, const char *name, uint32_t width, int32_t *element) {
    return guarded([&] { return *element = (int32_t)decoder::vector(static_cast<Opened *>(held)->archive(), name, width).element, 0; }, -1);
}
int32_t nhost_cache_validate(const char *name, uint32_t heads, uint32_t width, uint32_t capacity, uint32_t window, uint32_t batch, uint32_t rows,
                             int32_t element) {
    return guarded([&] { return decoder::Cache::validate(name, decoder::CacheShape(heads, width, capacity, window, batch, rows), (Element)element), 0; }, -1);
}
uint64_t nhost_payload_bytes(int32_t element, uint64_t elements) { return payload_bytes((Element)element, elements); }

// ---- neura-precision --------------------------------------------------------------------------------
// precision::pack: the bytes `count` numbers pack into (out, at most room); returns their count, or -1 refused
int64_t nhost_pack(int32_t element, float quantum, const float *values, size_t count, uint8_t *out, size_t room) {
    return guarded([&]() -> int64_t {
        auto packed = precision::pack((Element)element, quantum, values, count);
        for (size_t i = 0; i < packed.size() && i < room; i++) out[i] = packed[i];
        return (int64_t)packed.size();
    }, -1);
}
// precision::unpack: `elements` numbers out of `size` bytes; 0 done, -1 refused
int32_t nhost_unpack(int32_t element, size_t elements, const uint8_t *bytes, size_t size, float *out) {
    return guarded([&] {
        auto values = precision::unpack((Element)element, elements, bytes, size);
        for (size_t i = 0; i < values.size(); i++) out[i] = values[i];
        return 0;
    }, -1);
}
uint32_t nhost_half_bits(float value) { return precision::half_bits(value); }
float nhost_half_value(uint32_t bits) { return precision::half_value((uint16_t)bits); }

// ---- neura-template -----------------------------------------------------------------------------------
// Template::parse(source).render(messages, values): messages and values as JSON text; the rendered bytes (out, at most room);
// returns their count, or -1 refused
int64_t nhost_template_render(const char *source, const char *messages_json, const char *values_json, char *out, size_t room) {
    return guarded([&]() -> int64_t { return rendered(chat::Template::parse(source), messages_json, values_json, out, room); }, -1);
}
// Template::read(archive): the template the GGUF carries under tokenizer.chat_template
int64_t nhost_template_render_gguf(void *held, const char *messages_json, const char *values_json, char *out, size_t room) {
    return guarded([&]() -> int64_t {
        return rendered(chat::Template::read(static_cast<Opened *>(held)->archive()), messages_json, values_json, out, room);
    }, -1);
}

// ---- runtime, model, batch ----------------------------------------------------------------------
void *nhost_runtime_open(int32_t index) {
    return guarded([&]() -> void * { return new runtime::Runtime(index); }, nullptr);
}
void nhost_runtime_close(void *runtime) { delete static_cast<runtime::Runtime *>(runtime); }

// BatchSpec::new(context, batch, chunks), and .window(window) when window is not 0
static generate::BatchSpec spec_of(uint32_t context, uint32_t batch, const uint32_t *chunks, uint32_t count, uint32_t window, int32_t shared = 0) {
    generate::BatchSpec spec(context, batch, std::vector<uint32_t>(chunks, chunks + count));
    if (shared) spec = spec.shared();
    return window ? spec.window(window) : spec;
}
// a Qwen2 GGUF (whole or file) becomes a model and a greedy batch over it
void *nhost_batch_open(void *runtime, void *held, uint32_t vocabulary, uint32_t context, uint32_t batch, const uint32_t *chunks, uint32_t count,
                       uint32_t window, int32_t shared) {
    return guarded([&]() -> void * {
        auto *opened = static_cast<Opened *>(held);
        generate::BatchSpec spec = spec_of(context, batch, chunks, count, window, shared);
        auto config = generate::Config::read(opened->archive().metadata(), vocabulary);
        auto out = std::make_unique<Loaded>();
        out->model = std::make_unique<generate::Model>(*static_cast<runtime::Runtime *>(runtime), opened->archive(), opened->source(), config, spec);
        out->batch = std::make_unique<generate::Batch>(*out->model, spec);
        return out.release();
    }, nullptr);
}
// the same with the key and value states in `cache_element` (Element::Single, Half or Bfloat16)
void *nhost_batch_open_element(void *runtime, void *held, uint32_t vocabulary, uint32_t context, uint32_t batch, const uint32_t *chunks,
                               uint32_t count, uint32_t window, int32_t shared, int32_t cache_element) {
    return guarded([&]() -> void * {
        auto *opened = static_cast<Opened *>(held);
        generate::BatchSpec spec = spec_of(context, batch, chunks, count, window, shared);
        auto config = generate::Config::read(opened->archive().metadata(), vocabulary);
        auto out = std::make_unique<Loaded>();
        out->model = std::make_unique<generate::Model>(*static_cast<runtime::Runtime *>(runtime), opened->archive(), opened->source(), config, spec,
                                                       (Element)cache_element);
        out->batch = std::make_unique<generate::Batch>(*out->model, spec);
        return out.release();
    }, nullptr);
}
// the same with a sampled answer (BatchSpec::sampled(Sampling::sampled(temperature, keep, cumulative)))
void *nhost_batch_open_sampled(void *runtime, void *held, uint32_t vocabulary, uint32_t context, uint32_t batch, const uint32_t *chunks, uint32_t count,
                               float temperature, uint32_t keep, float cumulative, uint32_t window, int32_t shared) {
    return guarded([&]() -> void * {
        auto *opened = static_cast<Opened *>(held);
        generate::BatchSpec spec = spec_of(context, batch, chunks, count, window, shared).sampled(generate::Sampling::sampled(temperature, keep, cumulative));
        auto config = generate::Config::read(opened->archive().metadata(), vocabulary);
        auto out = std::make_unique<Loaded>();
        out->model = std::make_unique<generate::Model>(*static_cast<runtime::Runtime *>(runtime), opened->archive(), opened->source(), config, spec);
        out->batch = std::make_unique<generate::Batch>(*out->model, spec);
        return out.release();
    }, nullptr);
}
// Sampling::sampled's refusals alone, with no device
int32_t nhost_sampling_check(float temperature, uint32_t keep, float cumulative) {
    return guarded([&] { return generate::Sampling::sampled(temperature, keep, cumulative), 0; }, -1);
}
uint32_t nhost_plane_seed(uint32_t seed, uint32_t slot) { return generate::Batch::plane_seed(seed, slot); }
uint32_t nhost_seed_bits(uint32_t seed) { return generate::Batch::seed_bits(seed); }
// what a sampled batch draws with; slot < 0 names every plane
int32_t nhost_batch_set_seed(void *held, int32_t slot, uint32_t seed) {
    return guarded([&] {
        auto &batch = *static_cast<Loaded *>(held)->batch;
        if (slot < 0) batch.set_seed(seed);
        else batch.set_seed_of((uint32_t)slot, seed);
        return 0;
    }, -1);
}
int64_t nhost_batch_seed_of(void *held, uint32_t slot) {
    return guarded([&]() -> int64_t { return (int64_t) static_cast<Loaded *>(held)->batch->seed_of(slot); }, -1);
}
int32_t nhost_batch_set_temperature(void *held, int32_t slot, float value) {
    return guarded([&] {
        auto &batch = *static_cast<Loaded *>(held)->batch;
        if (slot < 0) batch.set_temperature(value);
        else batch.set_temperature_of((uint32_t)slot, value);
        return 0;
    }, -1);
}
int32_t nhost_batch_set_keep(void *held, int32_t slot, uint32_t keep) {
    return guarded([&] {
        auto &batch = *static_cast<Loaded *>(held)->batch;
        if (slot < 0) batch.set_keep(keep);
        else batch.set_keep_of((uint32_t)slot, keep);
        return 0;
    }, -1);
}
int32_t nhost_batch_set_cumulative(void *held, int32_t slot, float value) {
    return guarded([&] {
        auto &batch = *static_cast<Loaded *>(held)->batch;
        if (slot < 0) batch.set_cumulative(value);
        else batch.set_cumulative_of((uint32_t)slot, value);
        return 0;
    }, -1);
}
// BatchSpec's refusals alone, with no device: a batch over no model
int32_t nhost_batch_spec_check(uint32_t context, uint32_t batch, const uint32_t *chunks, uint32_t count, uint32_t window) {
    return guarded([&] {
        generate::Batch::validate(spec_of(context, batch, chunks, count, window));
        return 0;
    }, -1);
}
// BatchSpec::window's own refusal
int32_t nhost_batch_window_check(uint32_t window) {
    return guarded([&] { return generate::BatchSpec(8, 1, {}).window(window), 0; }, -1);
}
// Batch::prefix / forget_prefix (crates/neura-generate/src/batch.rs:885-998)
int32_t nhost_batch_prefix(void *held, const uint32_t *tokens, uint32_t count) {
    return guarded([&] { return static_cast<Loaded *>(held)->batch->prefix(std::vector<uint32_t>(tokens, tokens + count)), 0; }, -1);
}
int32_t nhost_batch_forget_prefix(void *held) {
    return guarded([&] { return static_cast<Loaded *>(held)->batch->forget_prefix(), 0; }, -1);
}
int64_t nhost_batch_window(void *held) {
    return guarded([&]() -> int64_t { return (int64_t) static_cast<Loaded *>(held)->batch->window(); }, -1);
}
void nhost_batch_close(void *held) { delete static_cast<Loaded *>(held); }
int32_t nhost_batch_admit(void *held, const uint32_t *tokens, uint32_t count) {
    return guarded([&] { return (int32_t) static_cast<Loaded *>(held)->batch->admit(std::vector<uint32_t>(tokens, tokens + count)); }, -1);
}
int32_t nhost_batch_restart(void *held, uint32_t slot, const uint32_t *tokens, uint32_t count) {
    return guarded([&] { return static_cast<Loaded *>(held)->batch->restart(slot, std::vector<uint32_t>(tokens, tokens + count)), 0; }, -1);
}
int32_t nhost_batch_resume(void *held, uint32_t slot, const uint32_t *tokens, uint32_t count) {
    return guarded([&] { return static_cast<Loaded *>(held)->batch->resume(slot, std::vector<uint32_t>(tokens, tokens + count)), 0; }, -1);
}
int32_t nhost_batch_suspend(void *held, uint32_t slot) {
    return guarded([&] { return static_cast<Loaded *>(held)->batch->suspend(slot), 0; }, -1);
}
int32_t nhost_batch_finish(void *held, uint32_t slot) {
    return guarded([&] { return static_cast<Loaded *>(held)->batch->finish(slot), 0; }, -1);
}
// emitted pairs (slot, token) into out, at most `room` pairs; returns their count or -1
int32_t nhost_batch_step(void *held, uint32_t *out, uint32_t room) {
    return guarded([&] {
        auto emitted = static_cast<Loaded *>(held)->batch->step();
        for (size_t i = 0; i < emitted.size() && i < room; i++) out[2 * i] = emitted[i].slot, out[2 * i + 1] = emitted[i].token;
        return (int32_t)emitted.size();
    }, -1);
}
// -1 when the plane holds no sequence
int64_t nhost_batch_cursor(void *held, uint32_t slot) {
    return guarded([&]() -> int64_t {
        auto at = static_cast<Loaded *>(held)->batch->cursor(slot);
        return at ? (int64_t)*at : -1;
    }, -2);
}
int64_t nhost_batch_remaining(void *held, uint32_t slot) {
    return guarded([&]() -> int64_t {
        auto left = static_cast<Loaded *>(held)->batch->remaining(slot);
        return left ? (int64_t)*left : -1;
    }, -2);
}
// bit i set: plane i is active (low word) / occupied (high word)
uint64_t nhost_batch_planes(void *held) {
    auto &batch = *static_cast<Loaded *>(held)->batch;
    uint64_t out = 0;
    for (uint32_t slot : batch.active()) out |= 1ull << slot;
    for (uint32_t slot : batch.occupied()) out |= 1ull << (32 + slot);
    return out;
}
int32_t nhost_batch_logits(void *held, float *out) {
    return guarded([&] { return runtime::check(nh_model_logits(static_cast<Loaded *>(held)->model->handle(), out)), 0; }, -1);
}

// ---- snapshots --------------------------------------------------------------------------------------
// BatchSnapshot::from_bytes then to_bytes: the bytes a reader that accepts them would write back (out, at most room);
// returns their count, or -1 refused
int64_t nhost_snapshot_round_trip(const uint8_t *bytes, size_t size, uint8_t *out, size_t room) {
    return guarded([&]() -> int64_t {
        auto written = generate::BatchSnapshot::from_bytes(std::vector<uint8_t>(bytes, bytes + size)).to_bytes();
        for (size_t i = 0; i < written.size() && i < room; i++) out[i] = written[i];
        return (int64_t)written.size();
    }, -1);
}
int64_t nhost_batch_snapshot(void *held, uint8_t *out, size_t room) {
    return guarded([&]() -> int64_t {
        auto written = static_cast<Loaded *>(held)->batch->snapshot().to_bytes();
        for (size_t i = 0; i < written.size() && i < room; i++) out[i] = written[i];
        return (int64_t)written.size();
    }, -1);
}
int32_t nhost_batch_restore(void *held, const uint8_t *bytes, size_t size) {
    return guarded([&] {
        return static_cast<Loaded *>(held)->batch->restore(generate::BatchSnapshot::from_bytes(std::vector<uint8_t>(bytes, bytes + size))), 0;
    }, -1);
}
int32_t nhost_batch_save_state(void *held, const char *path) {
    return guarded([&] { return static_cast<Loaded *>(held)->batch->save_state(path), 0; }, -1);
}
int32_t nhost_batch_restore_state(void *held, const char *path, const uint8_t *bytes, size_t size) {
    return guarded([&] {
        return static_cast<Loaded *>(held)->batch->restore_state(path, generate::BatchSnapshot::from_bytes(std::vector<uint8_t>(bytes, bytes + size))), 0;
    }, -1);
}

// ---- tokenizer ------------------------------------------------------------------------------------
// the byte level bpe of a gguf under a split rule: "qwen", or the rules of the reference's own tests
void *nhost_tokenizer_open(void *held, const char *rule) {
    return guarded([&]() -> void * {
        return new tokenizer::Tokenizer(tokenizer::Vocabulary::read(static_cast<Opened *>(held)->archive()), rule_named(rule));
    }, nullptr);
}
void nhost_tokenizer_close(void *held) { delete static_cast<tokenizer::Tokenizer *>(held); }
uint64_t nhost_tokenizer_vocabulary(void *held) { return static_cast<tokenizer::Tokenizer *>(held)->vocabulary(); }
// -1 when no token is spelled so
int64_t nhost_tokenizer_id(void *held, const char *token) {
    auto id = static_cast<tokenizer::Tokenizer *>(held)->id(token);
    return id ? (int64_t)*id : -1;
}
// the ids of `size` bytes of text into out (at most `room`); returns their count, or -1 refused
int64_t nhost_tokenizer_encode(void *held, const char *text, size_t size, uint32_t *out, size_t room) {
    return guarded([&]() -> int64_t {
        auto ids = static_cast<tokenizer::Tokenizer *>(held)->encode(std::string_view(text, size));
        for (size_t i = 0; i < ids.size() && i < room; i++) out[i] = ids[i];
        return (int64_t)ids.size();
    }, -1);
}
// the bytes of token `id` into out (at most `room`); returns their count, or -1 refused
int64_t nhost_tokenizer_piece(void *held, uint32_t id, uint8_t *out, size_t room) {
    return guarded([&]() -> int64_t {
        auto bytes = static_cast<tokenizer::Tokenizer *>(held)->piece(id);
        for (size_t i = 0; i < bytes.size() && i < room; i++) out[i] = bytes[i];
        return (int64_t)bytes.size();
    }, -1);
}
// the ends of the pieces a rule cuts `size` bytes of text into (byte offsets, at most `room`); returns their count
int64_t nhost_rule_pieces(const char *rule, const char *text, size_t size, uint64_t *ends, size_t room) {
    return guarded([&]() -> int64_t {
        std::string_view held(text, size);
        auto pieces = rule_named(rule)->pieces(held);
        for (size_t i = 0; i < pieces.size() && i < room; i++) ends[i] = (uint64_t)(pieces[i].data() + pieces[i].size() - held.data());
        return (int64_t)pieces.size();
    }, -1);
}
void *nhost_text_open(void) { return new tokenizer::Text(); }
void nhost_text_close(void *held) { delete static_cast<tokenizer::Text *>(held); }
// feeds `size` bytes (flush: size 0 and flush != 0) and copies the text that became whole into out; returns its length
int64_t nhost_text_push(void *held, const uint8_t *bytes, size_t size, int32_t flush, char *out, size_t room) {
    auto *text = static_cast<tokenizer::Text *>(held);
    const std::string whole = flush ? text->flush() : text->push(std::vector<uint8_t>(bytes, bytes + size));
    for (size_t i = 0; i < whole.size() && i < room; i++) out[i] = whole[i];
    return (int64_t)whole.size();
}

}  // extern "C"
