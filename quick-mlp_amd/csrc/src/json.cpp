#include <qmlp/json.h>

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>

namespace qmlp {

namespace {

class Parser
{
    const std::string& s_;
    size_t p_ = 0;

    [[noreturn]] void error(const std::string& what) const
    {
        throw json::parse_error("JSON parse error at offset " + std::to_string(p_) + ": " + what);
    }
    void skipWs()
    {
        while (p_ < s_.size()) {
            char c = s_[p_];
            if (c == ' ' || c == '\t' || c == '\n' || c == '\r') { ++p_; continue; }
            // tolerate // and /* */ comments in hand-written configuration files
            if (c == '/' && p_ + 1 < s_.size() && s_[p_ + 1] == '/') {
                while (p_ < s_.size() && s_[p_] != '\n') ++p_;
                continue;
            }
            if (c == '/' && p_ + 1 < s_.size() && s_[p_ + 1] == '*') {
                size_t e = s_.find("*/", p_ + 2);
                if (e == std::string::npos) error("unterminated comment");
                p_ = e + 2;
                continue;
            }
            break;
        }
    }
    char peek()
    {
        skipWs();
        if (p_ >= s_.size()) error("unexpected end of input");
        return s_[p_];
    }
    void expect(char c)
    {
        if (peek() != c) error(std::string("expected '") + c + "' but found '" + s_[p_] + "'");
        ++p_;
    }
    static void appendUtf8(std::string& out, unsigned cp)
    {
        if (cp < 0x80) out += static_cast<char>(cp);
        else if (cp < 0x800) { out += static_cast<char>(0xC0 | (cp >> 6)); out += static_cast<char>(0x80 | (cp & 0x3F)); }
        else if (cp < 0x10000) {
            out += static_cast<char>(0xE0 | (cp >> 12));
            out += static_cast<char>(0x80 | ((cp >> 6) & 0x3F));
            out += static_cast<char>(0x80 | (cp & 0x3F));
        } else {
            out += static_cast<char>(0xF0 | (cp >> 18));
            out += static_cast<char>(0x80 | ((cp >> 12) & 0x3F));
            out += static_cast<char>(0x80 | ((cp >> 6) & 0x3F));
            out += static_cast<char>(0x80 | (cp & 0x3F));
        }
    }
    unsigned hex4()
    {
        if (p_ + 4 > s_.size()) error("truncated \\u escape");
        unsigned v = 0;
        for (int i = 0; i < 4; ++i) {
            char c = s_[p_++];
            v <<= 4;
            if (c >= '0' && c <= '9') v |= c - '0';
            else if (c >= 'a' && c <= 'f') v |= c - 'a' + 10;
            else if (c >= 'A' && c <= 'F') v |= c - 'A' + 10;
            else error("invalid \\u escape");
        }
        return v;
    }
    std::string parseString()
    {
        expect('"');
        std::string out;
        while (true) {
            if (p_ >= s_.size()) error("unterminated string");
            char c = s_[p_++];
            if (c == '"') break;
            if (c == '\\') {
                if (p_ >= s_.size()) error("unterminated escape");
                char e = s_[p_++];
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
                    if (cp >= 0xD800 && cp <= 0xDBFF && p_ + 1 < s_.size() && s_[p_] == '\\' && s_[p_ + 1] == 'u') {
                        p_ += 2;
                        unsigned lo = hex4();
                        cp = 0x10000 + ((cp - 0xD800) << 10) + (lo - 0xDC00);
                    }
                    appendUtf8(out, cp);
                    break;
                }
                default: error("invalid escape character");
                }
            } else {
                out += c;
            }
        }
        return out;
    }
    json parseNumber()
    {
        size_t start = p_;
        bool isFloat = false;
        if (s_[p_] == '-' || s_[p_] == '+') ++p_;
        while (p_ < s_.size()) {
            char c = s_[p_];
            if (c >= '0' && c <= '9') { ++p_; continue; }
            if (c == '.' || c == 'e' || c == 'E' || c == '+' || c == '-') { isFloat = true; ++p_; continue; }
            break;
        }
        std::string tok = s_.substr(start, p_ - start);
        if (tok.empty() || tok == "-" || tok == "+") error("invalid number");
        char* end = nullptr;
        if (!isFloat) {
            long long v = std::strtoll(tok.c_str(), &end, 10);
            if (end && *end == '\0') return json(v);
        }
        double d = std::strtod(tok.c_str(), &end);
        if (!end || *end != '\0') error("invalid number '" + tok + "'");
        return json(d);
    }

public:
    explicit Parser(const std::string& s) : s_(s) {}

    json parseValue()
    {
        char c = peek();
        if (c == '{') {
            ++p_;
            json obj = json::object();
            if (peek() == '}') { ++p_; return obj; }
            while (true) {
                skipWs();
                std::string key = parseString();
                expect(':');
                obj[key] = parseValue();
                char d = peek();
                ++p_;
                if (d == '}') break;
                if (d != ',') error("expected ',' or '}' in object");
                if (peek() == '}') { ++p_; break; }   // trailing comma
            }
            return obj;
        }
        if (c == '[') {
            ++p_;
            json arr = json::array();
            if (peek() == ']') { ++p_; return arr; }
            while (true) {
                arr.push_back(parseValue());
                char d = peek();
                ++p_;
                if (d == ']') break;
                if (d != ',') error("expected ',' or ']' in array");
                if (peek() == ']') { ++p_; break; }   // trailing comma
            }
            return arr;
        }
        if (c == '"') return json(parseString());
        if (s_.compare(p_, 4, "true") == 0) { p_ += 4; return json(true); }
        if (s_.compare(p_, 5, "false") == 0) { p_ += 5; return json(false); }
        if (s_.compare(p_, 4, "null") == 0) { p_ += 4; return json(nullptr); }
        if (c == '-' || c == '+' || (c >= '0' && c <= '9')) return parseNumber();
        error(std::string("unexpected character '") + c + "'");
    }

    void finish()
    {
        skipWs();
        if (p_ != s_.size()) error("trailing characters after the JSON value");
    }
};

void dumpString(std::string& out, const std::string& s)
{
    out += '"';
    for (unsigned char c : s) {
        switch (c) {
        case '"': out += "\\\""; break;
        case '\\': out += "\\\\"; break;
        case '\n': out += "\\n"; break;
        case '\r': out += "\\r"; break;
        case '\t': out += "\\t"; break;
        case '\b': out += "\\b"; break;
        case '\f': out += "\\f"; break;
        default:
            if (c < 0x20) {
                char buf[8];
                std::snprintf(buf, sizeof(buf), "\\u%04x", c);
                out += buf;
            } else {
                out += static_cast<char>(c);
            }
        }
    }
    out += '"';
}

} // namespace

json json::parse(const std::string& text)
{
    Parser p(text);
    json v = p.parseValue();
    p.finish();
    return v;
}

const char* json::type_name() const
{
    switch (type_) {
    case type_t::null: return "null";
    case type_t::boolean: return "boolean";
    case type_t::integer:
    case type_t::number: return "number";
    case type_t::string: return "string";
    case type_t::array: return "array";
    case type_t::object: return "object";
    }
    return "unknown";
}

void json::dumpImpl(std::string& out, int indent, int level) const
{
    auto newline = [&](int lvl) {
        if (indent >= 0) {
            out += '\n';
            out.append(static_cast<size_t>(indent * lvl), ' ');
        }
    };
    switch (type_) {
    case type_t::null: out += "null"; break;
    case type_t::boolean: out += bool_ ? "true" : "false"; break;
    case type_t::integer: out += std::to_string(int_); break;
    case type_t::number: {
        if (!std::isfinite(num_)) { out += "null"; break; }
        char buf[40];
        std::snprintf(buf, sizeof(buf), "%.17g", num_);
        // shortest representation that round-trips
        for (int prec = 1; prec < 17; ++prec) {
            char b2[40];
            std::snprintf(b2, sizeof(b2), "%.*g", prec, num_);
            if (std::strtod(b2, nullptr) == num_) { std::memcpy(buf, b2, sizeof(b2)); break; }
        }
        std::string t = buf;
        if (t.find_first_of(".eEn") == std::string::npos) t += ".0";
        out += t;
        break;
    }
    case type_t::string: dumpString(out, str_); break;
    case type_t::array: {
        out += '[';
        for (size_t i = 0; i < arr_.size(); ++i) {
            if (i) out += ',';
            newline(level + 1);
            arr_[i].dumpImpl(out, indent, level + 1);
        }
        if (!arr_.empty()) newline(level);
        out += ']';
        break;
    }
    case type_t::object: {
        out += '{';
        bool first = true;
        for (const auto& kv : obj_) {
            if (!first) out += ',';
            first = false;
            newline(level + 1);
            dumpString(out, kv.first);
            out += indent >= 0 ? ": " : ":";
            kv.second.dumpImpl(out, indent, level + 1);
        }
        if (!obj_.empty()) newline(level);
        out += '}';
        break;
    }
    }
}

std::string json::dump(int indent) const
{
    std::string out;
    dumpImpl(out, indent, 0);
    return out;
}

bool json::operator==(const json& o) const
{
    if (is_number() && o.is_number()) return get<double>() == o.get<double>();
    if (type_ != o.type_) return false;
    switch (type_) {
    case type_t::null: return true;
    case type_t::boolean: return bool_ == o.bool_;
    case type_t::string: return str_ == o.str_;
    case type_t::array: return arr_ == o.arr_;
    case type_t::object: return obj_ == o.obj_;
    default: return false;
    }
}

} // namespace qmlp
