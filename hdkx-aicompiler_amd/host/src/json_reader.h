// json_reader.h -- a small JSON value and recursive-descent reader for the files this layer reads back
// (execution plans it wrote itself).  Numbers are kept as doubles plus their integer value.
#pragma once

#include <cstdlib>
#include <map>
#include <memory>
#include <stdexcept>
#include <string>
#include <vector>

namespace kxc {
namespace json {

struct Value {
    enum Kind { kNull, kBool, kNumber, kString, kArray, kObject } kind = kNull;
    bool boolean = false;
    double number = 0.0;
    long long integer = 0;
    std::string string;
    std::vector<Value> array;
    std::map<std::string, Value> object;

    const Value& at(const std::string& key) const {
        auto it = object.find(key);
        if (kind != kObject || it == object.end()) throw std::runtime_error("JSON: missing key '" + key + "'");
        return it->second;
    }
    bool has(const std::string& key) const { return kind == kObject && object.count(key) != 0; }
};

class Reader {
public:
    explicit Reader(const std::string& text) : s_(text) {}
    Value Parse() {
        Value v = ParseValue();
        SkipSpace();
        if (pos_ != s_.size()) Fail("trailing characters");
        return v;
    }

private:
    [[noreturn]] void Fail(const std::string& what) const {
        throw std::runtime_error("JSON: " + what + " at offset " + std::to_string(pos_));
    }
    void SkipSpace() {
        while (pos_ < s_.size() && (s_[pos_] == ' ' || s_[pos_] == '\n' || s_[pos_] == '\t' || s_[pos_] == '\r')) ++pos_;
    }
    bool Match(const char* word) {
        const size_t n = std::char_traits<char>::length(word);
        if (s_.compare(pos_, n, word) != 0) return false;
        pos_ += n;
        return true;
    }
    Value ParseValue() {
        SkipSpace();
        if (pos_ >= s_.size()) Fail("unexpected end");
        const char c = s_[pos_];
        Value v;
        if (c == '{') {
            v.kind = Value::kObject;
            ++pos_;
            SkipSpace();
            if (pos_ < s_.size() && s_[pos_] == '}') { ++pos_; return v; }
            for (;;) {
                SkipSpace();
                if (pos_ >= s_.size() || s_[pos_] != '"') Fail("expected a key");
                std::string key = ParseString();
                SkipSpace();
                if (pos_ >= s_.size() || s_[pos_] != ':') Fail("expected ':'");
                ++pos_;
                v.object[key] = ParseValue();
                SkipSpace();
                if (pos_ < s_.size() && s_[pos_] == ',') { ++pos_; continue; }
                if (pos_ < s_.size() && s_[pos_] == '}') { ++pos_; return v; }
                Fail("expected ',' or '}'");
            }
        }
        if (c == '[') {
            v.kind = Value::kArray;
            ++pos_;
            SkipSpace();
            if (pos_ < s_.size() && s_[pos_] == ']') { ++pos_; return v; }
            for (;;) {
                v.array.push_back(ParseValue());
                SkipSpace();
                if (pos_ < s_.size() && s_[pos_] == ',') { ++pos_; continue; }
                if (pos_ < s_.size() && s_[pos_] == ']') { ++pos_; return v; }
                Fail("expected ',' or ']'");
            }
        }
        if (c == '"') { v.kind = Value::kString; v.string = ParseString(); return v; }
        if (Match("true")) { v.kind = Value::kBool; v.boolean = true; return v; }
        if (Match("false")) { v.kind = Value::kBool; return v; }
        if (Match("null")) return v;
        const char* begin = s_.c_str() + pos_;
        char* end = nullptr;
        v.number = std::strtod(begin, &end);
        if (end == begin) Fail("unexpected character");
        v.kind = Value::kNumber;
        v.integer = static_cast<long long>(v.number);
        pos_ += static_cast<size_t>(end - begin);
        return v;
    }
    std::string ParseString() {
        std::string out;
        ++pos_;   // opening quote
        while (pos_ < s_.size() && s_[pos_] != '"') {
            char c = s_[pos_++];
            if (c != '\\') { out += c; continue; }
            if (pos_ >= s_.size()) Fail("bad escape");
            c = s_[pos_++];
            switch (c) {
                case 'n': out += '\n'; break;
                case 't': out += '\t'; break;
                case 'r': out += '\r'; break;
                case 'b': out += '\b'; break;
                case 'f': out += '\f'; break;
                case 'u': {
                    if (pos_ + 4 > s_.size()) Fail("bad \\u escape");
                    const unsigned code = static_cast<unsigned>(std::strtoul(s_.substr(pos_, 4).c_str(), nullptr, 16));
                    pos_ += 4;
                    if (code < 0x80) out += static_cast<char>(code);
                    else if (code < 0x800) { out += static_cast<char>(0xC0 | (code >> 6)); out += static_cast<char>(0x80 | (code & 0x3F)); }
                    else { out += static_cast<char>(0xE0 | (code >> 12)); out += static_cast<char>(0x80 | ((code >> 6) & 0x3F)); out += static_cast<char>(0x80 | (code & 0x3F)); }
                    break;
                }
                default: out += c;   // \" \\ \/
            }
        }
        if (pos_ >= s_.size()) Fail("unterminated string");
        ++pos_;   // closing quote
        return out;
    }

    const std::string& s_;
    size_t pos_ = 0;
};

inline std::string Escape(const std::string& in) {
    std::string out;
    for (unsigned char ch : in) {
        switch (ch) {
            case '"': out += "\\\""; break;
            case '\\': out += "\\\\"; break;
            case '\n': out += "\\n"; break;
            case '\r': out += "\\r"; break;
            case '\t': out += "\\t"; break;
            default:
                if (ch < 0x20) { char b[8]; std::snprintf(b, sizeof(b), "\\u%04x", ch); out += b; }
                else out += static_cast<char>(ch);
        }
    }
    return out;
}

}  // namespace json
}  // namespace kxc
