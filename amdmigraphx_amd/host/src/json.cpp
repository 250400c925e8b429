#include <migraphx/json.hpp>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>

namespace migraphx {

namespace {

void write_string(std::string& out, const std::string& s)
{
    out += '"';
    for(unsigned char c : s)
    {
        switch(c)
        {
        case '"': out += "\\\""; break;
        case '\\': out += "\\\\"; break;
        case '\n': out += "\\n"; break;
        case '\r': out += "\\r"; break;
        case '\t': out += "\\t"; break;
        case '\b': out += "\\b"; break;
        case '\f': out += "\\f"; break;
        default:
            if(c < 0x20)
            {
                char buf[8];
                std::snprintf(buf, sizeof(buf), "\\u%04x", c);
                out += buf;
            }
            else
                out += static_cast<char>(c);
        }
    }
    out += '"';
}

void write(std::string& out, const value& v)
{
    switch(v.kind())
    {
    case value::null_kind: out += "null"; break;
    case value::bool_kind: out += v.get_bool() ? "true" : "false"; break;
    case value::int_kind: out += std::to_string(v.get_int64()); break;
    case value::float_kind: {
        const double d = v.get_double();
        if(not std::isfinite(d))
        {
            out += "null"; // JSON has no infinities or NaN
            break;
        }
        char buf[40];
        std::snprintf(buf, sizeof(buf), "%.17g", d);
        out += buf;
        // keep it a float on the way back
        if(std::strpbrk(buf, ".eE") == nullptr)
            out += ".0";
        break;
    }
    case value::string_kind: write_string(out, v.get_string()); break;
    case value::binary_kind: {
        out += "{\"bytes\":[";
        const auto& b = v.get_binary();
        for(std::size_t i = 0; i < b.size(); i++)
        {
            if(i > 0)
                out += ',';
            out += std::to_string(static_cast<unsigned char>(b[i]));
        }
        out += "]}";
        break;
    }
    case value::array_kind:
    case value::object_kind: {
        const auto& items = v.items();
        const bool keyed  = v.is_object() or (not items.empty() and not items.front().get_key().empty());
        out += keyed ? '{' : '[';
        for(std::size_t i = 0; i < items.size(); i++)
        {
            if(i > 0)
                out += ',';
            if(keyed)
            {
                write_string(out, items[i].get_key());
                out += ':';
            }
            write(out, items[i]);
        }
        out += keyed ? '}' : ']';
        break;
    }
    }
}

struct parser
{
    const char* p;
    const char* end;

    [[noreturn]] void fail(const std::string& what) const
    {
        MIGRAPHX_THROW("json: " + what + " at offset " + std::to_string(p - (end - size)));
    }
    std::size_t size;

    void skip()
    {
        while(p != end and (*p == ' ' or *p == '\n' or *p == '\t' or *p == '\r'))
            p++;
    }
    bool eat(char c)
    {
        skip();
        if(p != end and *p == c)
        {
            p++;
            return true;
        }
        return false;
    }
    void expect(char c)
    {
        if(not eat(c))
            fail(std::string("expected '") + c + "'");
    }
    bool word(const char* w)
    {
        const auto n = std::strlen(w);
        if(static_cast<std::size_t>(end - p) >= n and std::memcmp(p, w, n) == 0)
        {
            p += n;
            return true;
        }
        return false;
    }
    static void utf8(std::string& out, unsigned cp)
    {
        if(cp < 0x80)
            out += static_cast<char>(cp);
        else if(cp < 0x800)
        {
            out += static_cast<char>(0xc0 | (cp >> 6));
            out += static_cast<char>(0x80 | (cp & 0x3f));
        }
        else if(cp < 0x10000)
        {
            out += static_cast<char>(0xe0 | (cp >> 12));
            out += static_cast<char>(0x80 | ((cp >> 6) & 0x3f));
            out += static_cast<char>(0x80 | (cp & 0x3f));
        }
        else
        {
            out += static_cast<char>(0xf0 | (cp >> 18));
            out += static_cast<char>(0x80 | ((cp >> 12) & 0x3f));
            out += static_cast<char>(0x80 | ((cp >> 6) & 0x3f));
            out += static_cast<char>(0x80 | (cp & 0x3f));
        }
    }
    unsigned hex4()
    {
        if(end - p < 4)
            fail("short \\u escape");
        unsigned x = 0;
        for(int i = 0; i < 4; i++)
        {
            const char c = *p++;
            x <<= 4;
            if(c >= '0' and c <= '9')
                x |= c - '0';
            else if(c >= 'a' and c <= 'f')
                x |= c - 'a' + 10;
            else if(c >= 'A' and c <= 'F')
                x |= c - 'A' + 10;
            else
                fail("bad \\u escape");
        }
        return x;
    }
    std::string string()
    {
        expect('"');
        std::string s;
        while(true)
        {
            if(p == end)
                fail("unterminated string");
            const char c = *p++;
            if(c == '"')
                return s;
            if(c != '\\')
            {
                s += c;
                continue;
            }
            if(p == end)
                fail("unterminated escape");
            const char e = *p++;
            switch(e)
            {
            case 'n': s += '\n'; break;
            case 'r': s += '\r'; break;
            case 't': s += '\t'; break;
            case 'b': s += '\b'; break;
            case 'f': s += '\f'; break;
            case 'u': {
                unsigned cp = hex4();
                if(cp >= 0xd800 and cp < 0xdc00 and end - p >= 6 and p[0] == '\\' and p[1] == 'u')
                {
                    p += 2;
                    cp = 0x10000 + ((cp - 0xd800) << 10) + (hex4() - 0xdc00);
                }
                utf8(s, cp);
                break;
            }
            default: s += e; // \" \\ \/
            }
        }
    }
    value number()
    {
        const char* first = p;
        bool is_float     = false;
        if(p != end and (*p == '-' or *p == '+'))
            p++;
        while(p != end and ((*p >= '0' and *p <= '9') or *p == '.' or *p == 'e' or *p == 'E' or
                            *p == '-' or *p == '+'))
        {
            is_float = is_float or *p == '.' or *p == 'e' or *p == 'E';
            p++;
        }
        const std::string text(first, p);
        if(text.empty() or text == "-")
            fail("expected a value");
        if(is_float)
            return value(std::strtod(text.c_str(), nullptr));
        return value(static_cast<int64_t>(std::strtoll(text.c_str(), nullptr, 10)));
    }
    value get(int depth = 0)
    {
        if(depth > 256)
            fail("nesting too deep");
        skip();
        if(p == end)
            fail("unexpected end");
        if(*p == '{')
        {
            p++;
            value r = value::object();
            if(eat('}'))
                return r;
            do
            {
                skip();
                auto key = string();
                expect(':');
                r[key] = value(key, get(depth + 1));
            } while(eat(','));
            expect('}');
            if(r.size() == 1 and r.contains("bytes") and r.at("bytes").is_array())
            {
                std::string b;
                for(const auto& x : r.at("bytes").items())
                    b += static_cast<char>(x.get_int64());
                return value::binary(b.data(), b.size());
            }
            return r;
        }
        if(*p == '[')
        {
            p++;
            value r = value::array();
            if(eat(']'))
                return r;
            do
            {
                r.push_back(get(depth + 1));
            } while(eat(','));
            expect(']');
            return r;
        }
        if(*p == '"')
            return value(string());
        if(word("null"))
            return value{};
        if(word("true"))
            return value(true);
        if(word("false"))
            return value(false);
        return number();
    }
};

} // namespace

std::string to_json_string(const value& v)
{
    std::string out;
    write(out, v);
    return out;
}

value from_json_string(const char* text, std::size_t size)
{
    parser ps{text, text + size, size};
    auto v = ps.get();
    ps.skip();
    if(ps.p != ps.end)
        ps.fail("trailing characters");
    return v;
}

value from_json_string(const std::string& text) { return from_json_string(text.data(), text.size()); }

} // namespace migraphx
