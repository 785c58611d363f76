#include "json.h"

#include <cmath>
#include <cstdio>
#include <cstdlib>

namespace minillm {

class JsonParser {
public:
    explicit JsonParser(const std::string& t) : t_(t) {}
    Json run() {
        Json v = value();
        ws();
        if (i_ != t_.size()) bad("text after the value");
        return v;
    }

private:
    [[noreturn]] void bad(const char* what) const {
        throw JsonError("JSON: " + std::string(what) + " at offset " + std::to_string(i_));
    }
    void ws() {
        while (i_ < t_.size() && (t_[i_] == ' ' || t_[i_] == '\n' || t_[i_] == '\t' || t_[i_] == '\r')) ++i_;
    }
    bool take(const char* lit) {
        size_t n = 0;
        while (lit[n]) ++n;
        if (t_.compare(i_, n, lit) == 0) { i_ += n; return true; }
        return false;
    }
    static void utf8(std::string& out, unsigned cp) {
        if (cp < 0x80) out += static_cast<char>(cp);
        else if (cp < 0x800) { out += static_cast<char>(0xC0 | (cp >> 6)); out += static_cast<char>(0x80 | (cp & 0x3F)); }
        else if (cp < 0x10000) {
            out += static_cast<char>(0xE0 | (cp >> 12)); out += static_cast<char>(0x80 | ((cp >> 6) & 0x3F));
            out += static_cast<char>(0x80 | (cp & 0x3F));
        } else {
            out += static_cast<char>(0xF0 | (cp >> 18)); out += static_cast<char>(0x80 | ((cp >> 12) & 0x3F));
            out += static_cast<char>(0x80 | ((cp >> 6) & 0x3F)); out += static_cast<char>(0x80 | (cp & 0x3F));
        }
    }
    unsigned hex4() {
        if (i_ + 4 > t_.size()) bad("short \\u escape");
        unsigned v = 0;
        for (int k = 0; k < 4; ++k) {
            const char c = t_[i_++];
            v <<= 4;
            if (c >= '0' && c <= '9') v |= c - '0';
            else if (c >= 'a' && c <= 'f') v |= c - 'a' + 10;
            else if (c >= 'A' && c <= 'F') v |= c - 'A' + 10;
            else bad("bad \\u escape");
        }
        return v;
    }
    std::string str() {
        if (t_[i_] != '"') bad("expected a string");
        ++i_;
        std::string out;
        while (true) {
            if (i_ >= t_.size()) bad("unterminated string");
            const char c = t_[i_++];
            if (c == '"') break;
            if (c != '\\') { out += c; continue; }
            if (i_ >= t_.size()) bad("unterminated escape");
            const char e = t_[i_++];
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
                    if (cp >= 0xD800 && cp < 0xDC00 && take("\\u")) {
                        const unsigned lo = hex4();
                        cp = 0x10000 + ((cp - 0xD800) << 10) + (lo - 0xDC00);
                    }
                    utf8(out, cp);
                    break;
                }
                default: bad("unknown escape");
            }
        }
        return out;
    }
    // Nesting deeper than any configuration or safetensors header goes is refused: the parser recurses once
    // per level, and a text of a million '[' must end in an error, not in a stack overflow.
    static constexpr int MAX_DEPTH = 64;
    struct Level {
        explicit Level(JsonParser& p) : p_(p) { if (++p_.depth_ > MAX_DEPTH) p_.bad("nested deeper than 64 levels"); }
        ~Level() { --p_.depth_; }
        JsonParser& p_;
    };
    Json value() {
        const Level level(*this);
        ws();
        if (i_ >= t_.size()) bad("unexpected end");
        const char c = t_[i_];
        if (c == '{') {
            ++i_;
            Json j = Json::object();
            ws();
            if (i_ < t_.size() && t_[i_] == '}') { ++i_; return j; }
            while (true) {
                ws();
                std::string key = str();
                ws();
                if (i_ >= t_.size() || t_[i_] != ':') bad("expected ':'");
                ++i_;
                j.obj_.emplace_back(std::move(key), value());
                ws();
                if (i_ < t_.size() && t_[i_] == ',') { ++i_; continue; }
                if (i_ < t_.size() && t_[i_] == '}') { ++i_; break; }
                bad("expected ',' or '}'");
            }
            return j;
        }
        if (c == '[') {
            ++i_;
            Json j;
            j.kind_ = Json::Array;
            ws();
            if (i_ < t_.size() && t_[i_] == ']') { ++i_; return j; }
            while (true) {
                j.arr_.push_back(value());
                ws();
                if (i_ < t_.size() && t_[i_] == ',') { ++i_; continue; }
                if (i_ < t_.size() && t_[i_] == ']') { ++i_; break; }
                bad("expected ',' or ']'");
            }
            return j;
        }
        if (c == '"') return Json::of(str());
        if (take("true")) return Json::of(true);
        if (take("false")) return Json::of(false);
        if (take("null")) return Json();
        // number
        const size_t start = i_;
        if (t_[i_] == '-') ++i_;
        bool integral = true;
        while (i_ < t_.size() && ((t_[i_] >= '0' && t_[i_] <= '9') || t_[i_] == '.' || t_[i_] == 'e' || t_[i_] == 'E' ||
                                  t_[i_] == '+' || t_[i_] == '-')) {
            if (t_[i_] == '.' || t_[i_] == 'e' || t_[i_] == 'E') integral = false;
            ++i_;
        }
        if (i_ == start) bad("unexpected character");
        const std::string num = t_.substr(start, i_ - start);
        char* end = nullptr;
        const double v = std::strtod(num.c_str(), &end);
        if (end == nullptr || *end != '\0') bad("bad number");
        Json j = Json::of(v);
        j.integral_ = integral && std::fabs(v) < 9.0e15;
        return j;
    }
    const std::string& t_;
    size_t i_ = 0;
    int depth_ = 0;
};

Json Json::parse(const std::string& text) { return JsonParser(text).run(); }

bool Json::has(const std::string& key) const { return find(key) != nullptr; }

const Json* Json::find(const std::string& key) const {
    if (kind_ != Object) return nullptr;
    for (const auto& kv : obj_)
        if (kv.first == key) return &kv.second;
    return nullptr;
}

const Json& Json::at(const std::string& key) const {
    const Json* j = find(key);
    if (j == nullptr) throw JsonError("key '" + key + "' is missing");
    return *j;
}

void Json::set(const std::string& key, Json v) {
    need(Object, "an object");
    for (auto& kv : obj_)
        if (kv.first == key) { kv.second = std::move(v); return; }
    obj_.emplace_back(key, std::move(v));
}

static void dump_string(std::string& out, const std::string& s) {
    out += '"';
    for (const char c : s) {
        switch (c) {
            case '"': out += "\\\""; break;
            case '\\': out += "\\\\"; break;
            case '\n': out += "\\n"; break;
            case '\r': out += "\\r"; break;
            case '\t': out += "\\t"; break;
            default:
                if (static_cast<unsigned char>(c) < 0x20) {
                    char buf[8];
                    std::snprintf(buf, sizeof buf, "\\u%04x", c);
                    out += buf;
                } else {
                    out += c;
                }
        }
    }
    out += '"';
}

std::string Json::dump() const {
    std::string out;
    switch (kind_) {
        case Null: return "null";
        case Bool: return bool_ ? "true" : "false";
        case Number: {
            char buf[40];
            if (integral_) std::snprintf(buf, sizeof buf, "%lld", static_cast<long long>(num_));
            else std::snprintf(buf, sizeof buf, "%.17g", num_);
            return buf;
        }
        case String: dump_string(out, str_); return out;
        case Array:
            out = "[";
            for (size_t i = 0; i < arr_.size(); ++i) out += (i ? "," : "") + arr_[i].dump();
            return out + "]";
        case Object:
            out = "{";
            for (size_t i = 0; i < obj_.size(); ++i) {
                if (i) out += ",";
                dump_string(out, obj_[i].first);
                out += ":" + obj_[i].second.dump();
            }
            return out + "}";
    }
    return out;
}

}  // namespace minillm
