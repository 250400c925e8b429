#include <migraphx/msgpack.hpp>
#include <cstdint>
#include <cstring>
#include <limits>

namespace migraphx {

namespace {

// one bin object holds at most this many bytes (src/msgpack.cpp:31)
constexpr std::size_t bin_chunk_limit = std::numeric_limits<uint32_t>::max() - 1;

struct writer
{
    std::vector<char> out;

    void byte(unsigned b) { out.push_back(static_cast<char>(b)); }
    // big endian, `n` low bytes of x
    void be(uint64_t x, int n)
    {
        for(int i = n - 1; i >= 0; i--)
            byte((x >> (8 * i)) & 0xff);
    }
    void raw(const char* p, std::size_t n) { out.insert(out.end(), p, p + n); }

    void unsigned_int(uint64_t x)
    {
        if(x < 0x80)
            byte(x);
        else if(x <= 0xff)
            byte(0xcc), be(x, 1);
        else if(x <= 0xffff)
            byte(0xcd), be(x, 2);
        else if(x <= 0xffffffffull)
            byte(0xce), be(x, 4);
        else
            byte(0xcf), be(x, 8);
    }
    void signed_int(int64_t x)
    {
        if(x >= 0)
            return unsigned_int(static_cast<uint64_t>(x));
        const auto u = static_cast<uint64_t>(x);
        if(x >= -32)
            byte(u & 0xff);
        else if(x >= std::numeric_limits<int8_t>::min())
            byte(0xd0), be(u, 1);
        else if(x >= std::numeric_limits<int16_t>::min())
            byte(0xd1), be(u, 2);
        else if(x >= std::numeric_limits<int32_t>::min())
            byte(0xd2), be(u, 4);
        else
            byte(0xd3), be(u, 8);
    }
    void float64(double d)
    {
        uint64_t bits = 0;
        std::memcpy(&bits, &d, sizeof(bits));
        byte(0xcb), be(bits, 8);
    }
    void string(const std::string& s)
    {
        const auto n = s.size();
        if(n < 32)
            byte(0xa0 | n);
        else if(n <= 0xff)
            byte(0xd9), be(n, 1);
        else if(n <= 0xffff)
            byte(0xda), be(n, 2);
        else if(n <= 0xffffffffull)
            byte(0xdb), be(n, 4);
        else
            MIGRAPHX_THROW("Size is too large for msgpack");
        raw(s.data(), n);
    }
    void bin(const char* p, std::size_t n)
    {
        if(n <= 0xff)
            byte(0xc4), be(n, 1);
        else if(n <= 0xffff)
            byte(0xc5), be(n, 2);
        else
            byte(0xc6), be(n, 4);
        raw(p, n);
    }
    void list_header(std::size_t n, unsigned fix, unsigned h16)
    {
        if(n < 16)
            byte(fix | n);
        else if(n <= 0xffff)
            byte(h16), be(n, 2);
        else if(n <= bin_chunk_limit)
            byte(h16 + 1), be(n, 4);
        else
            MIGRAPHX_THROW("Size is too large for msgpack");
    }

    void put(const value& v)
    {
        switch(v.kind())
        {
        case value::null_kind: byte(0xc0); break;
        case value::bool_kind: byte(v.get_bool() ? 0xc3 : 0xc2); break;
        case value::int_kind: signed_int(v.get_int64()); break;
        case value::float_kind: float64(v.get_double()); break;
        case value::string_kind: string(v.get_string()); break;
        case value::binary_kind: {
            const auto& b      = v.get_binary();
            const auto nchunks = 1 + (std::max<std::size_t>(1, b.size()) - 1) / bin_chunk_limit;
            list_header(nchunks, 0x90, 0xdc);
            for(std::size_t c = 0; c < nchunks; c++)
            {
                const auto first = c * bin_chunk_limit;
                bin(b.data() + first, std::min(bin_chunk_limit, b.size() - first));
            }
            break;
        }
        case value::array_kind:
        case value::object_kind: {
            const auto& items = v.items();
            // keyed items make a map, as the reference decides by the first item
            if(not items.empty() and not items.front().get_key().empty())
            {
                list_header(items.size(), 0x80, 0xde);
                for(const auto& x : items)
                {
                    string(x.get_key());
                    put(x);
                }
            }
            else
            {
                list_header(items.size(), 0x90, 0xdc);
                for(const auto& x : items)
                    put(x);
            }
            break;
        }
        }
    }
};

struct reader
{
    const unsigned char* p;
    const unsigned char* end;

    void need(std::size_t n) const
    {
        if(static_cast<std::size_t>(end - p) < n)
            MIGRAPHX_THROW("msgpack: truncated input");
    }
    uint64_t be(int n)
    {
        need(n);
        uint64_t x = 0;
        for(int i = 0; i < n; i++)
            x = (x << 8) | *p++;
        return x;
    }
    std::string bytes(std::size_t n)
    {
        need(n);
        std::string s(reinterpret_cast<const char*>(p), n);
        p += n;
        return s;
    }
    template <class T>
    static int64_t sign_extend(uint64_t x)
    {
        return static_cast<int64_t>(static_cast<T>(x));
    }

    value array(std::size_t n, int depth)
    {
        // an array that starts with a bin object is chunked binary data
        if(n != 0 and p != end and (*p == 0xc4 or *p == 0xc5 or *p == 0xc6))
        {
            std::string all;
            for(std::size_t i = 0; i < n; i++)
            {
                auto chunk = get(depth + 1);
                if(not chunk.is_binary())
                    MIGRAPHX_THROW("msgpack: mixed binary chunks");
                all += chunk.get_binary();
            }
            return value::binary(all.data(), all.size());
        }
        value r = value::array();
        for(std::size_t i = 0; i < n; i++)
            r.push_back(get(depth + 1));
        return r;
    }
    value map(std::size_t n, int depth)
    {
        value r = value::object();
        for(std::size_t i = 0; i < n; i++)
        {
            auto key = get(depth + 1);
            if(not key.is_string())
                MIGRAPHX_THROW("msgpack: map keys must be strings");
            r[key.get_string()] = value(key.get_string(), get(depth + 1));
        }
        return r;
    }

    value get(int depth = 0)
    {
        if(depth > 256)
            MIGRAPHX_THROW("msgpack: nesting too deep");
        need(1);
        const unsigned t = *p++;
        if(t < 0x80)
            return value(static_cast<int64_t>(t));
        if(t >= 0xe0)
            return value(sign_extend<int8_t>(t));
        if((t & 0xf0) == 0x80)
            return map(t & 0x0f, depth);
        if((t & 0xf0) == 0x90)
            return array(t & 0x0f, depth);
        if((t & 0xe0) == 0xa0)
            return value(bytes(t & 0x1f));
        switch(t)
        {
        case 0xc0: return value{};
        case 0xc2: return value(false);
        case 0xc3: return value(true);
        case 0xc4:
        case 0xc5:
        case 0xc6: {
            auto b = bytes(be(1 << (t - 0xc4)));
            return value::binary(b.data(), b.size());
        }
        case 0xca: {
            const auto bits = static_cast<uint32_t>(be(4));
            float f         = 0;
            std::memcpy(&f, &bits, sizeof(f));
            return value(static_cast<double>(f));
        }
        case 0xcb: {
            const uint64_t bits = be(8);
            double d            = 0;
            std::memcpy(&d, &bits, sizeof(d));
            return value(d);
        }
        case 0xcc: return value(static_cast<int64_t>(be(1)));
        case 0xcd: return value(static_cast<int64_t>(be(2)));
        case 0xce: return value(static_cast<int64_t>(be(4)));
        case 0xcf: {
            // `value` holds signed 64-bit integers only: a larger unsigned number would read back negative
            const uint64_t u = be(8);
            if(u > static_cast<uint64_t>(INT64_MAX))
                MIGRAPHX_THROW("msgpack: unsigned integer above the signed 64-bit range");
            return value(static_cast<int64_t>(u));
        }
        case 0xd0: return value(sign_extend<int8_t>(be(1)));
        case 0xd1: return value(sign_extend<int16_t>(be(2)));
        case 0xd2: return value(sign_extend<int32_t>(be(4)));
        case 0xd3: return value(sign_extend<int64_t>(be(8)));
        case 0xd9: return value(bytes(be(1)));
        case 0xda: return value(bytes(be(2)));
        case 0xdb: return value(bytes(be(4)));
        case 0xdc: return array(be(2), depth);
        case 0xdd: return array(be(4), depth);
        case 0xde: return map(be(2), depth);
        case 0xdf: return map(be(4), depth);
        default: MIGRAPHX_THROW("msgpack EXT type not supported.");
        }
    }
};

} // namespace

std::vector<char> to_msgpack(const value& v)
{
    writer w;
    w.put(v);
    return std::move(w.out);
}

value from_msgpack(const char* buffer, std::size_t size)
{
    const auto* b = reinterpret_cast<const unsigned char*>(buffer);
    reader r{b, b + size};
    return r.get();
}

value from_msgpack(const std::vector<char>& buffer)
{
    return from_msgpack(buffer.data(), buffer.size());
}

} // namespace migraphx
