// Saving and loading a VariableEnvironment in the reference's on-disk format
// (src/variable.rs:470-480 the serialised struct, :549-554 save, :556-563 deserialize,
// :565-588 load_internal, :590-598 prepare_for_serde).
//
// The reference writes `serde_json::to_writer` of
//     { "array_list": [ <array>, ... ], "name_to_id": { "<namespace>\u0001<name>": <id>, ... } }
// where every <array> is ndarray's serde form {"v":1,"dim":[extents...],"data":[elements in row-major
// order...]} (Cargo.toml:18, ndarray's `serde` feature; format version 1) and <id> is the index into
// array_list (VariableID is a newtype over usize, src/variable.rs:90-94).  serde_json prints an f32 with
// the shortest digits that read back to the same value, always with ".0" or an exponent, and prints
// `null` for a value that is not finite.  This file writes the same text and reads any JSON that
// serde_json would accept for those types.
//
// The text stage works on host memory only (SavedEnvironment), so it can be used and tested without
// a device; VariableEnvironment::save/load/initialize move the arrays between it and device memory.
#include <cctype>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <sstream>

#include "ag_host.hpp"

namespace ag {
namespace host {

// ---------------------------------------------------------------------------------------------
// writing
// ---------------------------------------------------------------------------------------------
namespace {

// Shortest decimal digits that read back as `v`, laid out the way serde_json prints an f32:
// plain notation while the decimal point stays within 13 digits to the right and 5 zeros to the
// left of the digits, otherwise d.ddde±x.
void append_f32(std::string &out, float v)
{
    if (!std::isfinite(v)) {
        out += "null";
        return;
    }
    if (std::signbit(v)) out += '-';
    const float a = std::fabs(v);
    if (a == 0.f) {
        out += "0.0";
        return;
    }
    char buf[40];
    for (int digits = 1; digits <= 9; ++digits) {
        std::snprintf(buf, sizeof buf, "%.*e", digits - 1, (double)a);
        if (std::strtof(buf, nullptr) == a) break;
    }
    // buf = d[.ddd]e±xx
    std::string digits;
    const char *p = buf;
    for (; *p && *p != 'e'; ++p)
        if (*p != '.') digits += *p;
    const int exp10 = std::atoi(p + 1);
    while (digits.size() > 1 && digits.back() == '0') digits.pop_back();
    const int length = (int)digits.size();
    const int kk = exp10 + 1;       // 10^(kk-1) <= a < 10^kk
    const int k = kk - length;      // a = digits * 10^k
    if (0 <= k && kk <= 13) {       // 1234e7 -> 12340000000.0
        out += digits;
        out.append((size_t)k, '0');
        out += ".0";
    } else if (0 < kk && kk <= 13) {  // 1234e-2 -> 12.34
        out.append(digits, 0, (size_t)kk);
        out += '.';
        out.append(digits, (size_t)kk, std::string::npos);
    } else if (-6 < kk && kk <= 0) {  // 1234e-6 -> 0.001234
        out += "0.";
        out.append((size_t)(-kk), '0');
        out += digits;
    } else {  // 1e30, 1.234e33
        out += digits[0];
        if (length > 1) {
            out += '.';
            out.append(digits, 1, std::string::npos);
        }
        out += 'e';
        out += std::to_string(kk - 1);
    }
}

void append_string(std::string &out, const std::string &s)
{
    out += '"';
    for (const char ch : s) {
        const unsigned char c = (unsigned char)ch;
        switch (c) {
            case '"': out += "\\\""; break;
            case '\\': out += "\\\\"; break;
            case '\b': out += "\\b"; break;
            case '\f': out += "\\f"; break;
            case '\n': out += "\\n"; break;
            case '\r': out += "\\r"; break;
            case '\t': out += "\\t"; break;
            default:
                if (c < 0x20) {
                    char esc[8];
                    std::snprintf(esc, sizeof esc, "\\u%04x", c);
                    out += esc;
                } else {
                    out += ch;
                }
        }
    }
    out += '"';
}

}  // namespace

std::string to_json(const SavedEnvironment &env)
{
    std::string out;
    size_t elements = 0;
    for (const SavedArray &a : env.array_list) elements += a.data.size();
    out.reserve(64 + elements * 12);
    out += "{\"array_list\":[";
    for (size_t i = 0; i < env.array_list.size(); ++i) {
        const SavedArray &a = env.array_list[i];
        if (i) out += ',';
        out += "{\"v\":1,\"dim\":[";
        for (size_t d = 0; d < a.dim.size(); ++d) {
            if (d) out += ',';
            out += std::to_string(a.dim[d]);
        }
        out += "],\"data\":[";
        for (size_t e = 0; e < a.data.size(); ++e) {
            if (e) out += ',';
            append_f32(out, a.data[e]);
        }
        out += "]}";
    }
    out += "],\"name_to_id\":{";
    bool first = true;
    for (const auto &kv : env.name_to_id) {
        if (!first) out += ',';
        first = false;
        append_string(out, kv.first);
        out += ':';
        out += std::to_string(kv.second);
    }
    out += "}}";
    return out;
}

// ---------------------------------------------------------------------------------------------
// reading
// ---------------------------------------------------------------------------------------------
namespace {

class Reader {
  public:
    explicit Reader(const std::string &text) : s_(text) {}

    [[noreturn]] void fail(const std::string &what) const
    {
        size_t line = 1, col = 1;
        for (size_t i = 0; i < pos_ && i < s_.size(); ++i) {
            if (s_[i] == '\n') {
                ++line;
                col = 1;
            } else {
                ++col;
            }
        }
        throw PersistError(what + " at line " + std::to_string(line) + " column " + std::to_string(col));
    }

    void skip_ws()
    {
        while (pos_ < s_.size() && (s_[pos_] == ' ' || s_[pos_] == '\t' || s_[pos_] == '\n' || s_[pos_] == '\r')) ++pos_;
    }
    char peek()
    {
        skip_ws();
        if (pos_ >= s_.size()) fail("EOF while parsing a value");
        return s_[pos_];
    }
    bool consume(char c)
    {
        if (peek() != c) return false;
        ++pos_;
        return true;
    }
    void expect(char c)
    {
        if (!consume(c)) fail(std::string("expected `") + c + "`");
    }
    void end()
    {
        skip_ws();
        if (pos_ != s_.size()) fail("trailing characters");
    }

    std::string string()
    {
        expect('"');
        std::string out;
        for (;;) {
            if (pos_ >= s_.size()) fail("EOF while parsing a string");
            const char c = s_[pos_++];
            if (c == '"') return out;
            if ((unsigned char)c < 0x20) fail("control character (\\u0000-\\u001F) found while parsing a string");
            if (c != '\\') {
                out += c;
                continue;
            }
            if (pos_ >= s_.size()) fail("EOF while parsing a string");
            const char e = s_[pos_++];
            switch (e) {
                case '"': out += '"'; break;
                case '\\': out += '\\'; break;
                case '/': out += '/'; break;
                case 'b': out += '\b'; break;
                case 'f': out += '\f'; break;
                case 'n': out += '\n'; break;
                case 'r': out += '\r'; break;
                case 't': out += '\t'; break;
                case 'u': {
                    unsigned cp = hex4();
                    if (cp >= 0xD800 && cp < 0xDC00) {  // surrogate pair
                        if (pos_ + 1 >= s_.size() || s_[pos_] != '\\' || s_[pos_ + 1] != 'u') fail("unexpected end of hex escape");
                        pos_ += 2;
                        const unsigned lo = hex4();
                        if (lo < 0xDC00 || lo > 0xDFFF) fail("lone leading surrogate in hex escape");
                        cp = 0x10000 + ((cp - 0xD800) << 10) + (lo - 0xDC00);
                    } else if (cp >= 0xDC00 && cp < 0xE000) {
                        fail("lone trailing surrogate in hex escape");
                    }
                    utf8(out, cp);
                    break;
                }
                default: fail("invalid escape");
            }
        }
    }

    // Any JSON number, read the way serde_json reads an f32: as f64, then narrowed.
    float number_f32()
    {
        const std::string tok = number_token();
        return (float)std::strtod(tok.c_str(), nullptr);
    }
    // A non-negative integer (usize in the reference).
    int64_t number_usize(const char *what)
    {
        const std::string tok = number_token();
        if (tok.find_first_of(".eE") != std::string::npos) fail(std::string("invalid type: floating point, expected ") + what);
        if (tok[0] == '-') fail(std::string("invalid value: negative integer, expected ") + what);
        if (tok.size() > 18) fail(std::string("number out of range, expected ") + what);
        return std::strtoll(tok.c_str(), nullptr, 10);
    }

    void skip_value()
    {
        const char c = peek();
        if (c == '"') {
            string();
        } else if (c == '{') {
            ++pos_;
            if (consume('}')) return;
            do {
                string();
                expect(':');
                skip_value();
            } while (consume(','));
            expect('}');
        } else if (c == '[') {
            ++pos_;
            if (consume(']')) return;
            do skip_value();
            while (consume(','));
            expect(']');
        } else if (c == 't') {
            literal("true");
        } else if (c == 'f') {
            literal("false");
        } else if (c == 'n') {
            literal("null");
        } else {
            number_token();
        }
    }

  private:
    void literal(const char *word)
    {
        const size_t n = std::strlen(word);
        if (s_.compare(pos_, n, word) != 0) fail("expected ident");
        pos_ += n;
    }
    unsigned hex4()
    {
        if (pos_ + 4 > s_.size()) fail("EOF while parsing a string");
        unsigned v = 0;
        for (int i = 0; i < 4; ++i) {
            const char c = s_[pos_++];
            v <<= 4;
            if (c >= '0' && c <= '9') v |= (unsigned)(c - '0');
            else if (c >= 'a' && c <= 'f') v |= (unsigned)(c - 'a' + 10);
            else if (c >= 'A' && c <= 'F') v |= (unsigned)(c - 'A' + 10);
            else fail("invalid escape");
        }
        return v;
    }
    static void utf8(std::string &out, unsigned cp)
    {
        if (cp < 0x80) {
            out += (char)cp;
        } else if (cp < 0x800) {
            out += (char)(0xC0 | (cp >> 6));
            out += (char)(0x80 | (cp & 0x3F));
        } else if (cp < 0x10000) {
            out += (char)(0xE0 | (cp >> 12));
            out += (char)(0x80 | ((cp >> 6) & 0x3F));
            out += (char)(0x80 | (cp & 0x3F));
        } else {
            out += (char)(0xF0 | (cp >> 18));
            out += (char)(0x80 | ((cp >> 12) & 0x3F));
            out += (char)(0x80 | ((cp >> 6) & 0x3F));
            out += (char)(0x80 | (cp & 0x3F));
        }
    }
    // JSON grammar: -? (0 | [1-9][0-9]*) (. [0-9]+)? ([eE] [+-]? [0-9]+)?
    std::string number_token()
    {
        const char c = peek();
        if (c == 'n') fail("invalid type: null, expected a number");
        const size_t start = pos_;
        if (s_[pos_] == '-') ++pos_;
        if (pos_ >= s_.size() || !std::isdigit((unsigned char)s_[pos_])) fail("expected value");
        if (s_[pos_] == '0') {
            ++pos_;
        } else {
            while (pos_ < s_.size() && std::isdigit((unsigned char)s_[pos_])) ++pos_;
        }
        if (pos_ < s_.size() && s_[pos_] == '.') {
            ++pos_;
            if (pos_ >= s_.size() || !std::isdigit((unsigned char)s_[pos_])) fail("invalid number");
            while (pos_ < s_.size() && std::isdigit((unsigned char)s_[pos_])) ++pos_;
        }
        if (pos_ < s_.size() && (s_[pos_] == 'e' || s_[pos_] == 'E')) {
            ++pos_;
            if (pos_ < s_.size() && (s_[pos_] == '+' || s_[pos_] == '-')) ++pos_;
            if (pos_ >= s_.size() || !std::isdigit((unsigned char)s_[pos_])) fail("invalid number");
            while (pos_ < s_.size() && std::isdigit((unsigned char)s_[pos_])) ++pos_;
        }
        return s_.substr(start, pos_ - start);
    }

    const std::string &s_;
    size_t pos_ = 0;
};

// ndarray's serde form: exactly the fields v, dim, data, in any order.
SavedArray read_array(Reader &r)
{
    SavedArray a;
    bool has_v = false, has_dim = false, has_data = false;
    r.expect('{');
    if (!r.consume('}')) {
        do {
            const std::string key = r.string();
            r.expect(':');
            if (key == "v") {
                if (has_v) r.fail("duplicate field `v`");
                has_v = true;
                const int64_t v = r.number_usize("u8");
                if (v != 1) r.fail("unknown array version: " + std::to_string(v));
            } else if (key == "dim") {
                if (has_dim) r.fail("duplicate field `dim`");
                has_dim = true;
                r.expect('[');
                if (!r.consume(']')) {
                    do a.dim.push_back(r.number_usize("usize"));
                    while (r.consume(','));
                    r.expect(']');
                }
            } else if (key == "data") {
                if (has_data) r.fail("duplicate field `data`");
                has_data = true;
                r.expect('[');
                if (!r.consume(']')) {
                    do a.data.push_back(r.number_f32());
                    while (r.consume(','));
                    r.expect(']');
                }
            } else {
                r.fail("unknown field `" + key + "`, expected one of `v`, `dim`, `data`");
            }
        } while (r.consume(','));
        r.expect('}');
    }
    if (!has_v) r.fail("missing field `v`");
    if (!has_data) r.fail("missing field `data`");
    if (!has_dim) r.fail("missing field `dim`");
    size_t len = 1;
    for (const int64_t d : a.dim) len *= (size_t)d;
    if (len != a.data.size()) r.fail("data and dimension must match in size");
    return a;
}

}  // namespace

SavedEnvironment from_json(const std::string &text)
{
    SavedEnvironment env;
    Reader r(text);
    bool has_list = false, has_names = false;
    r.expect('{');
    if (!r.consume('}')) {
        do {
            const std::string key = r.string();
            r.expect(':');
            if (key == "array_list") {
                if (has_list) r.fail("duplicate field `array_list`");
                has_list = true;
                r.expect('[');
                if (!r.consume(']')) {
                    do env.array_list.push_back(read_array(r));
                    while (r.consume(','));
                    r.expect(']');
                }
            } else if (key == "name_to_id") {
                if (has_names) r.fail("duplicate field `name_to_id`");
                has_names = true;
                r.expect('{');
                if (!r.consume('}')) {
                    do {
                        const std::string name = r.string();
                        r.expect(':');
                        env.name_to_id[name] = (VariableID)r.number_usize("usize");  // a repeated key keeps the last value
                    } while (r.consume(','));
                    r.expect('}');
                }
            } else {
                r.skip_value();  // fields the struct does not have are ignored
            }
        } while (r.consume(','));
        r.expect('}');
    }
    r.end();
    if (!has_list) r.fail("missing field `array_list`");
    if (!has_names) r.fail("missing field `name_to_id`");
    return env;
}

// ---------------------------------------------------------------------------------------------
// files
// ---------------------------------------------------------------------------------------------
SavedEnvironment read_saved_environment(const std::string &path)
{
    std::ifstream f(path, std::ios::binary);
    if (!f) throw PersistError("cannot open " + path + ": " + std::strerror(errno));
    std::ostringstream ss;
    ss << f.rdbuf();
    return from_json(ss.str());
}

void write_saved_environment(const SavedEnvironment &env, const std::string &path)
{
    std::ofstream f(path, std::ios::binary | std::ios::trunc);  // File::create truncates
    if (!f) throw PersistError("cannot create " + path + ": " + std::strerror(errno));
    const std::string text = to_json(env);
    f.write(text.data(), (std::streamsize)text.size());
    f.close();
    if (!f) throw PersistError("cannot write " + path);
}

// ---------------------------------------------------------------------------------------------
// VariableEnvironment                                               src/variable.rs:483-500, 549-588
// ---------------------------------------------------------------------------------------------
void VariableEnvironment::save(const std::string &path) const
{
    SavedEnvironment s;
    for (const NdArray &a : arrays_) {
        SavedArray sa;
        sa.dim = a.shape();
        sa.data = a.to_host();
        s.array_list.push_back(std::move(sa));
    }
    s.name_to_id = name_to_id_;
    write_saved_environment(s, path);
}

void VariableEnvironment::initialize(const std::string &path)
{
    const SavedEnvironment s = read_saved_environment(path);
    // load_internal (src/variable.rs:568-582) takes the first two \u0001-separated parts of every key
    // and panics when there is no separator
    std::map<std::string, VariableID> names;
    for (const auto &kv : s.name_to_id) {
        const size_t sep = kv.first.find('\x01');
        if (sep == std::string::npos) throw Panic("saved variable name has no namespace separator: " + kv.first);
        const size_t sep2 = kv.first.find('\x01', sep + 1);
        names[kv.first.substr(0, sep2)] = kv.second;
    }
    std::vector<NdArray> arrays;
    for (const SavedArray &a : s.array_list) arrays.push_back(NdArray::from_host(a.dim, a.data.data()));
    arrays_ = std::move(arrays);
    name_to_id_ = std::move(names);
}

VariableEnvironment VariableEnvironment::load(const std::string &path)
{
    VariableEnvironment env;
    env.initialize(path);
    return env;
}

}  // namespace host
}  // namespace ag
