// JSON reader / writer for Functions of the int8 inference path (see ngraph/serializer.hpp).
//
// Layout follows nGraph's JSONSerializer / JSONDeserializer, src/ngraph/serializer.cpp:
//   file      = [ function, ... ]                                   (:461-476, :518-521)
//   function  = {"name", "parameters": [node names], "result": [node names], "ops": [node, ...]}
//               ops in topological order                             (:556-581, :812-851)
//   node      = {"name", "op", "op_version", "friendly_name"?, "inputs": [ref, ...],
//                "control_deps"?, "outputs": [tensor names], <op attributes>}      (:2661-2724)
//   ref       = "node name"  |  {"node": "node name", "index": n}     (:2635-2649, :604-631)
//   type      = "float" | "int8_t" | ...   (c_type_string; older files: an object holding it, :404-424)
// The JSON text itself is parsed by the small recursive-descent parser below (RFC 8259).
#include "ngraph/serializer.hpp"

#include <cerrno>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <map>
#include <sstream>
#include <sys/stat.h>

#include "ngraph/ops.hpp"

using namespace ngraph;

namespace
{
    // ------------------------------------------------------------------------------ JSON value
    class Json
    {
    public:
        enum class Kind
        {
            null,
            boolean,
            integer, // fits int64_t
            uinteger, // above INT64_MAX
            real,
            string,
            array,
            object
        };
        Json() = default;
        Json(bool b) : m_kind(Kind::boolean), m_bool(b) {}
        Json(int64_t v) : m_kind(Kind::integer), m_int(v) {}
        Json(uint64_t v) : m_kind(v > static_cast<uint64_t>(INT64_MAX) ? Kind::uinteger : Kind::integer), m_int(static_cast<int64_t>(v)), m_uint(v) {}
        Json(int v) : Json(static_cast<int64_t>(v)) {}
        Json(double v) : m_kind(Kind::real), m_real(v) {}
        Json(const std::string& s) : m_kind(Kind::string), m_string(s) {}
        Json(const char* s) : m_kind(Kind::string), m_string(s) {}
        static Json array()
        {
            Json j;
            j.m_kind = Kind::array;
            return j;
        }
        static Json object()
        {
            Json j;
            j.m_kind = Kind::object;
            return j;
        }
        template <typename T>
        static Json array_of(const T& values)
        {
            Json j = array();
            for (const auto& v : values)
                j.push_back(Json(static_cast<int64_t>(v)));
            return j;
        }

        Kind kind() const { return m_kind; }
        bool is_null() const { return m_kind == Kind::null; }
        bool is_string() const { return m_kind == Kind::string; }
        bool is_object() const { return m_kind == Kind::object; }
        bool is_array() const { return m_kind == Kind::array; }
        bool is_number() const { return m_kind == Kind::integer || m_kind == Kind::uinteger || m_kind == Kind::real; }

        bool has(const std::string& key) const { return m_kind == Kind::object && m_members.count(key) != 0; }
        const Json& at(const std::string& key) const
        {
            if (m_kind != Kind::object)
                throw std::runtime_error("json value is not an object (looking up '" + key + "')");
            auto it = m_members.find(key);
            if (it == m_members.end())
                throw std::runtime_error("key '" + key + "' not found");
            return it->second;
        }
        Json& operator[](const std::string& key)
        {
            if (m_kind == Kind::null)
                m_kind = Kind::object;
            if (m_kind != Kind::object)
                throw std::runtime_error("json value is not an object (setting '" + key + "')");
            return m_members[key];
        }
        void push_back(const Json& v)
        {
            if (m_kind == Kind::null)
                m_kind = Kind::array;
            if (m_kind != Kind::array)
                throw std::runtime_error("json value is not an array");
            m_elements.push_back(v);
        }
        const std::vector<Json>& elements() const
        {
            if (m_kind != Kind::array)
                throw std::runtime_error("json value is not an array");
            return m_elements;
        }
        const std::map<std::string, Json>& members() const { return m_members; }

        const std::string& get_string() const
        {
            if (m_kind != Kind::string)
                throw std::runtime_error("json value is not a string");
            return m_string;
        }
        bool get_bool() const
        {
            if (m_kind != Kind::boolean)
                throw std::runtime_error("json value is not a boolean");
            return m_bool;
        }
        int64_t get_int() const
        {
            if (m_kind == Kind::integer)
                return m_int;
            if (m_kind == Kind::boolean)
                return m_bool;
            if (m_kind == Kind::real && std::floor(m_real) == m_real && std::fabs(m_real) < 9.2e18)
                return static_cast<int64_t>(m_real);
            throw std::runtime_error("json value is not an integer");
        }
        size_t get_size() const
        {
            if (m_kind == Kind::uinteger)
                return static_cast<size_t>(m_uint);
            int64_t v = get_int();
            if (v < 0)
                throw std::runtime_error("json value is negative where an unsigned number is expected");
            return static_cast<size_t>(v);
        }
        double get_double() const
        {
            if (m_kind == Kind::real)
                return m_real;
            if (m_kind == Kind::integer)
                return static_cast<double>(m_int);
            if (m_kind == Kind::uinteger)
                return static_cast<double>(m_uint);
            throw std::runtime_error("json value is not a number");
        }
        template <typename V>
        V get_size_vector() const
        {
            V out;
            for (const Json& e : elements())
                out.push_back(e.get_size());
            return out;
        }
        template <typename V>
        V get_int_vector() const
        {
            V out;
            for (const Json& e : elements())
                out.push_back(static_cast<typename V::value_type>(e.get_int()));
            return out;
        }
        AxisSet get_axis_set() const
        {
            AxisSet out;
            if (m_kind == Kind::array) // nGraph's deserialize_axis_set: anything else is the empty set
                for (const Json& e : m_elements)
                    out.insert(e.get_size());
            return out;
        }

        // nlohmann::json::dump(): indent < 0 compact, otherwise pretty-printed with that many blanks
        void dump(std::string& out, int indent, int depth = 0) const;

    private:
        static void dump_string(std::string& out, const std::string& s);
        Kind m_kind = Kind::null;
        bool m_bool = false;
        int64_t m_int = 0;
        uint64_t m_uint = 0;
        double m_real = 0;
        std::string m_string;
        std::vector<Json> m_elements;
        std::map<std::string, Json> m_members;
    };

    void Json::dump_string(std::string& out, const std::string& s)
    {
        out += '"';
        for (unsigned char c : s)
        {
            switch (c)
            {
            case '"': out += "\\\""; break;
            case '\\': out += "\\\\"; break;
            case '\b': out += "\\b"; break;
            case '\f': out += "\\f"; break;
            case '\n': out += "\\n"; break;
            case '\r': out += "\\r"; break;
            case '\t': out += "\\t"; break;
            default:
                if (c < 0x20)
                {
                    char buf[8];
                    std::snprintf(buf, sizeof buf, "\\u%04x", c);
                    out += buf;
                }
                else
                    out += static_cast<char>(c);
            }
        }
        out += '"';
    }

    void Json::dump(std::string& out, int indent, int depth) const
    {
        auto newline = [&](int d) {
            if (indent >= 0)
            {
                out += '\n';
                out.append(static_cast<size_t>(indent) * d, ' ');
            }
        };
        switch (m_kind)
        {
        case Kind::null: out += "null"; break;
        case Kind::boolean: out += m_bool ? "true" : "false"; break;
        case Kind::integer: out += std::to_string(m_int); break;
        case Kind::uinteger: out += std::to_string(m_uint); break;
        case Kind::real:
        {
            if (!std::isfinite(m_real))
            {
                out += "null"; // what nlohmann::json writes for NaN / Inf
                break;
            }
            char buf[40];
            for (int prec = 1; prec <= 17; ++prec) // shortest text that reads back to the same double
            {
                std::snprintf(buf, sizeof buf, "%.*g", prec, m_real);
                if (std::strtod(buf, nullptr) == m_real)
                    break;
            }
            std::string t = buf;
            if (t.find_first_of(".eEn") == std::string::npos)
                t += ".0";
            out += t;
            break;
        }
        case Kind::string: dump_string(out, m_string); break;
        case Kind::array:
            if (m_elements.empty())
            {
                out += "[]";
                break;
            }
            out += '[';
            for (size_t i = 0; i < m_elements.size(); ++i)
            {
                if (i)
                    out += ',';
                newline(depth + 1);
                m_elements[i].dump(out, indent, depth + 1);
            }
            newline(depth);
            out += ']';
            break;
        case Kind::object:
            if (m_members.empty())
            {
                out += "{}";
                break;
            }
            out += '{';
            {
                bool first = true;
                for (const auto& kv : m_members)
                {
                    if (!first)
                        out += ',';
                    first = false;
                    newline(depth + 1);
                    dump_string(out, kv.first);
                    out += indent >= 0 ? ": " : ":";
                    kv.second.dump(out, indent, depth + 1);
                }
            }
            newline(depth);
            out += '}';
            break;
        }
    }

    // ------------------------------------------------------------------------------ JSON parser
    class JsonParser
    {
    public:
        explicit JsonParser(const std::string& text) : m_text(text) {}
        Json parse()
        {
            Json v = value(0);
            skip_space();
            if (m_pos != m_text.size())
                error("text after the end of the json value");
            return v;
        }

    private:
        static constexpr int kMaxDepth = 512;
        [[noreturn]] void error(const std::string& what) const
        {
            size_t line = 1, col = 1;
            for (size_t i = 0; i < m_pos && i < m_text.size(); ++i)
            {
                if (m_text[i] == '\n')
                    ++line, col = 1;
                else
                    ++col;
            }
            throw std::runtime_error("json parse error at line " + std::to_string(line) + ", column " + std::to_string(col) + ": " + what);
        }
        void skip_space()
        {
            while (m_pos < m_text.size() && (m_text[m_pos] == ' ' || m_text[m_pos] == '\t' || m_text[m_pos] == '\n' || m_text[m_pos] == '\r'))
                ++m_pos;
        }
        bool eat(const char* word)
        {
            size_t n = std::strlen(word);
            if (m_text.compare(m_pos, n, word) == 0)
            {
                m_pos += n;
                return true;
            }
            return false;
        }
        Json value(int depth)
        {
            if (depth > kMaxDepth)
                error("nesting deeper than " + std::to_string(kMaxDepth));
            skip_space();
            if (m_pos >= m_text.size())
                error("unexpected end of text");
            char c = m_text[m_pos];
            if (c == '{')
                return object(depth);
            if (c == '[')
                return array(depth);
            if (c == '"')
                return Json(string());
            if (eat("true"))
                return Json(true);
            if (eat("false"))
                return Json(false);
            if (eat("null"))
                return Json();
            if (c == '-' || (c >= '0' && c <= '9'))
                return number();
            error(std::string("unexpected character '") + c + "'");
        }
        Json object(int depth)
        {
            Json j = Json::object();
            ++m_pos; // {
            skip_space();
            if (m_pos < m_text.size() && m_text[m_pos] == '}')
            {
                ++m_pos;
                return j;
            }
            while (true)
            {
                skip_space();
                if (m_pos >= m_text.size() || m_text[m_pos] != '"')
                    error("expected a member name");
                std::string key = string();
                skip_space();
                if (m_pos >= m_text.size() || m_text[m_pos] != ':')
                    error("expected ':' after a member name");
                ++m_pos;
                j[key] = value(depth + 1); // a repeated name keeps the last value, as nlohmann::json does
                skip_space();
                if (m_pos < m_text.size() && m_text[m_pos] == ',')
                {
                    ++m_pos;
                    continue;
                }
                if (m_pos < m_text.size() && m_text[m_pos] == '}')
                {
                    ++m_pos;
                    return j;
                }
                error("expected ',' or '}' in an object");
            }
        }
        Json array(int depth)
        {
            Json j = Json::array();
            ++m_pos; // [
            skip_space();
            if (m_pos < m_text.size() && m_text[m_pos] == ']')
            {
                ++m_pos;
                return j;
            }
            while (true)
            {
                j.push_back(value(depth + 1));
                skip_space();
                if (m_pos < m_text.size() && m_text[m_pos] == ',')
                {
                    ++m_pos;
                    continue;
                }
                if (m_pos < m_text.size() && m_text[m_pos] == ']')
                {
                    ++m_pos;
                    return j;
                }
                error("expected ',' or ']' in an array");
            }
        }
        unsigned hex4()
        {
            if (m_pos + 4 > m_text.size())
                error("truncated \\u escape");
            unsigned v = 0;
            for (int i = 0; i < 4; ++i)
            {
                char c = m_text[m_pos++];
                v <<= 4;
                if (c >= '0' && c <= '9')
                    v |= static_cast<unsigned>(c - '0');
                else if (c >= 'a' && c <= 'f')
                    v |= static_cast<unsigned>(c - 'a' + 10);
                else if (c >= 'A' && c <= 'F')
                    v |= static_cast<unsigned>(c - 'A' + 10);
                else
                    error("bad hex digit in \\u escape");
            }
            return v;
        }
        static void append_utf8(std::string& out, unsigned cp)
        {
            if (cp < 0x80)
                out += static_cast<char>(cp);
            else if (cp < 0x800)
            {
                out += static_cast<char>(0xC0 | (cp >> 6));
                out += static_cast<char>(0x80 | (cp & 0x3F));
            }
            else if (cp < 0x10000)
            {
                out += static_cast<char>(0xE0 | (cp >> 12));
                out += static_cast<char>(0x80 | ((cp >> 6) & 0x3F));
                out += static_cast<char>(0x80 | (cp & 0x3F));
            }
            else
            {
                out += static_cast<char>(0xF0 | (cp >> 18));
                out += static_cast<char>(0x80 | ((cp >> 12) & 0x3F));
                out += static_cast<char>(0x80 | ((cp >> 6) & 0x3F));
                out += static_cast<char>(0x80 | (cp & 0x3F));
            }
        }
        std::string string()
        {
            std::string out;
            ++m_pos; // opening quote
            while (true)
            {
                if (m_pos >= m_text.size())
                    error("unterminated string");
                unsigned char c = static_cast<unsigned char>(m_text[m_pos++]);
                if (c == '"')
                    return out;
                if (c < 0x20)
                    error("control character inside a string");
                if (c != '\\')
                {
                    out += static_cast<char>(c);
                    continue;
                }
                if (m_pos >= m_text.size())
                    error("unterminated escape");
                char e = m_text[m_pos++];
                switch (e)
                {
                case '"': out += '"'; break;
                case '\\': out += '\\'; break;
                case '/': out += '/'; break;
                case 'b': out += '\b'; break;
                case 'f': out += '\f'; break;
                case 'n': out += '\n'; break;
                case 'r': out += '\r'; break;
                case 't': out += '\t'; break;
                case 'u':
                {
                    unsigned cp = hex4();
                    if (cp >= 0xD800 && cp <= 0xDBFF) // high surrogate: a low one must follow
                    {
                        if (!eat("\\u"))
                            error("lone high surrogate");
                        unsigned lo = hex4();
                        if (lo < 0xDC00 || lo > 0xDFFF)
                            error("bad low surrogate");
                        cp = 0x10000 + ((cp - 0xD800) << 10) + (lo - 0xDC00);
                    }
                    else if (cp >= 0xDC00 && cp <= 0xDFFF)
                        error("lone low surrogate");
                    append_utf8(out, cp);
                    break;
                }
                default: error(std::string("unknown escape '\\") + e + "'");
                }
            }
        }
        Json number()
        {
            size_t start = m_pos;
            bool real = false;
            if (m_text[m_pos] == '-')
                ++m_pos;
            if (m_pos >= m_text.size() || m_text[m_pos] < '0' || m_text[m_pos] > '9')
                error("expected a digit");
            if (m_text[m_pos] == '0')
                ++m_pos; // no leading zeros
            else
                while (m_pos < m_text.size() && m_text[m_pos] >= '0' && m_text[m_pos] <= '9')
                    ++m_pos;
            if (m_pos < m_text.size() && m_text[m_pos] == '.')
            {
                real = true;
                ++m_pos;
                if (m_pos >= m_text.size() || m_text[m_pos] < '0' || m_text[m_pos] > '9')
                    error("expected a digit after the decimal point");
                while (m_pos < m_text.size() && m_text[m_pos] >= '0' && m_text[m_pos] <= '9')
                    ++m_pos;
            }
            if (m_pos < m_text.size() && (m_text[m_pos] == 'e' || m_text[m_pos] == 'E'))
            {
                real = true;
                ++m_pos;
                if (m_pos < m_text.size() && (m_text[m_pos] == '+' || m_text[m_pos] == '-'))
                    ++m_pos;
                if (m_pos >= m_text.size() || m_text[m_pos] < '0' || m_text[m_pos] > '9')
                    error("expected a digit in the exponent");
                while (m_pos < m_text.size() && m_text[m_pos] >= '0' && m_text[m_pos] <= '9')
                    ++m_pos;
            }
            std::string tok = m_text.substr(start, m_pos - start);
            if (!real)
            {
                errno = 0;
                if (tok[0] == '-')
                {
                    long long v = std::strtoll(tok.c_str(), nullptr, 10);
                    if (errno != ERANGE)
                        return Json(static_cast<int64_t>(v));
                }
                else
                {
                    unsigned long long v = std::strtoull(tok.c_str(), nullptr, 10);
                    if (errno != ERANGE)
                        return Json(static_cast<uint64_t>(v));
                }
            }
            return Json(std::strtod(tok.c_str(), nullptr));
        }

        const std::string& m_text;
        size_t m_pos = 0;
    };

    // ------------------------------------------------------------------------------ element types
    Json write_element_type(const element::Type& t) { return Json(t.c_type_string()); }

    element::Type read_element_type(const Json& j)
    {
        const std::string& c_type = j.is_object() ? j.at("c_type_string").get_string() : j.get_string();
        for (element::Type t : {element::boolean, element::f32, element::f64, element::i8, element::i32, element::i64, element::u8})
            if (t.c_type_string() == c_type)
                return t;
        throw std::runtime_error("element type '" + c_type + "' is not one this backend handles");
    }

    Shape read_shape(const Json& j)
    {
        if (j.is_null())
            throw std::runtime_error("dynamic shapes are not supported");
        Shape s;
        for (const Json& d : j.elements())
        {
            if (d.is_null())
                throw std::runtime_error("dynamic dimensions are not supported");
            s.push_back(d.get_size());
        }
        return s;
    }

    // ------------------------------------------------------------------------------ constants
    // op::v0::Constant::convert_value_to_string / get_value_strings (src/ngraph/op/constant.cpp:308-420):
    // reals with max_digits10 significant digits ("NAN", "INFINITY", "-INFINITY" for the specials),
    // integers through std::to_string.
    template <typename T>
    std::string real_to_string(T v)
    {
        if (std::isnan(v))
            return "NAN";
        if (std::isinf(v))
            return v > 0 ? "INFINITY" : "-INFINITY";
        std::stringstream ss;
        ss.precision(std::numeric_limits<T>::max_digits10);
        ss << v;
        return ss.str();
    }

    std::string element_to_string(const element::Type& et, const uint8_t* p)
    {
        switch (et.get_type_enum())
        {
        case element::Type_t::boolean: return std::to_string(static_cast<int>(*reinterpret_cast<const char*>(p)));
        case element::Type_t::f32:
        {
            float v;
            std::memcpy(&v, p, sizeof v);
            return real_to_string(v);
        }
        case element::Type_t::f64:
        {
            double v;
            std::memcpy(&v, p, sizeof v);
            return real_to_string(v);
        }
        case element::Type_t::i8: return std::to_string(static_cast<int>(*reinterpret_cast<const int8_t*>(p)));
        case element::Type_t::u8: return std::to_string(static_cast<int>(*p));
        case element::Type_t::i32:
        {
            int32_t v;
            std::memcpy(&v, p, sizeof v);
            return std::to_string(v);
        }
        case element::Type_t::i64:
        {
            int64_t v;
            std::memcpy(&v, p, sizeof v);
            return std::to_string(v);
        }
        default: throw std::runtime_error("unsupported constant type");
        }
    }

    // parse_string<T> of src/ngraph/util.cpp:382-435: the whole literal must be consumed
    void string_to_element(const element::Type& et, const std::string& s, uint8_t* p)
    {
        const char* begin = s.c_str();
        char* end = nullptr;
        auto whole = [&]() {
            if (end == begin || *end != 0)
                throw std::runtime_error("Could not parse literal '" + s + "'");
        };
        switch (et.get_type_enum())
        {
        case element::Type_t::f32:
        {
            float v = std::strtof(begin, &end);
            whole();
            std::memcpy(p, &v, sizeof v);
            break;
        }
        case element::Type_t::f64:
        {
            double v = std::strtod(begin, &end);
            whole();
            std::memcpy(p, &v, sizeof v);
            break;
        }
        case element::Type_t::boolean:
        case element::Type_t::i8:
        case element::Type_t::u8:
        {
            long v = std::strtol(begin, &end, 10);
            whole();
            *p = static_cast<uint8_t>(v); // narrowed as the reference's int8_t / uint8_t result
            break;
        }
        case element::Type_t::i32:
        {
            long long v = std::strtoll(begin, &end, 10);
            whole();
            int32_t w = static_cast<int32_t>(v);
            std::memcpy(p, &w, sizeof w);
            break;
        }
        case element::Type_t::i64:
        {
            long long v = std::strtoll(begin, &end, 10);
            whole();
            int64_t w = v;
            std::memcpy(p, &w, sizeof w);
            break;
        }
        default: throw std::runtime_error("unsupported constant type");
        }
    }

    std::shared_ptr<Node> read_constant(const Json& node_js)
    {
        const Json& type_js = node_js.has("element_type") ? node_js : node_js.at("value_type");
        element::Type et = read_element_type(type_js.at("element_type"));
        Shape shape = read_shape(type_js.at("shape"));
        const std::vector<Json>& values = node_js.at("value").elements();
        size_t n = shape_size(shape), w = et.size();
        // one literal fills the tensor, otherwise one per element (op::v0::Constant's string constructor)
        if (values.size() != n && values.size() != 1)
            throw std::runtime_error("Did not get the expected number of literals for a constant of " + std::to_string(n) + " elements (got " +
                                     std::to_string(values.size()) + ")");
        std::vector<uint8_t> bytes(n * w + 8);
        if (values.size() == 1 && n != 1)
        {
            string_to_element(et, values[0].get_string(), bytes.data());
            for (size_t i = 1; i < n; ++i)
                std::memcpy(bytes.data() + i * w, bytes.data(), w);
        }
        else
            for (size_t i = 0; i < n; ++i)
                string_to_element(et, values[i].get_string(), bytes.data() + i * w);
        return std::make_shared<op::v0::Constant>(et, shape, bytes.data());
    }

    Json write_constant_values(const op::v0::Constant& c)
    {
        const element::Type& et = c.get_output_element_type(0);
        size_t n = shape_size(c.get_output_shape(0)), w = et.size();
        const uint8_t* p = static_cast<const uint8_t*>(c.get_data_ptr());
        bool identical = n > 0;
        for (size_t i = 1; i < n && identical; ++i)
            identical = std::memcmp(p, p + i * w, w) == 0;
        Json values = Json::array();
        if (identical)
            values.push_back(Json(element_to_string(et, p)));
        else
            for (size_t i = 0; i < n; ++i)
                values.push_back(Json(element_to_string(et, p + i * w)));
        return values;
    }

    // ------------------------------------------------------------------------------ reader
    class Reader
    {
    public:
        std::shared_ptr<Function> function(const Json& func_js)
        {
            const std::string& name = func_js.at("name").get_string();
            for (const Json& node_js : func_js.at("ops").elements())
                node(node_js);
            // graphs with op::v0::Result on every output, or (older files) on none
            ResultVector results;
            size_t have = 0;
            const std::vector<Json>& result_refs = func_js.at("result").elements();
            for (const Json& ref : result_refs)
            {
                std::shared_ptr<Node> n = node_reference(ref);
                if (auto r = as_type_ptr<op::v0::Result>(n))
                {
                    results.push_back(r);
                    ++have;
                }
                else
                    results.push_back(std::make_shared<op::v0::Result>(n));
            }
            if (have != 0 && have != result_refs.size())
                throw ngraph_error("Graph serialization is inconsistent. Some op::v0::Results appear to be missing");
            ParameterVector params;
            for (const Json& ref : func_js.at("parameters").elements())
            {
                auto p = as_type_ptr<op::v0::Parameter>(node_reference(ref));
                if (!p)
                    throw ngraph_error("Function parameter '" + ref.get_string() + "' is not a Parameter node");
                params.push_back(p);
            }
            return std::make_shared<Function>(results, params, name);
        }

    private:
        std::shared_ptr<Node> node_reference(const Json& j) const
        {
            const std::string& name = j.get_string();
            auto it = m_nodes.find(name);
            if (it == m_nodes.end())
                throw std::runtime_error("reference to node '" + name + "', which has not been defined");
            return it->second;
        }
        Output<Node> output(const Json& j) const
        {
            std::string name;
            size_t index = 0;
            if (j.is_string())
                name = j.get_string();
            else if (j.is_object())
            {
                name = j.at("node").get_string();
                index = j.at("index").get_size();
            }
            else
                throw ngraph_error("Expected string or object an output while deserializing");
            auto alias = m_goe_alias.find(name);
            if (alias != m_goe_alias.end())
                return alias->second;
            auto it = m_nodes.find(name);
            if (it == m_nodes.end())
                throw std::runtime_error("input refers to node '" + name + "', which has not been defined");
            if (index >= it->second->get_output_size())
                throw std::runtime_error("input refers to output " + std::to_string(index) + " of node '" + name + "', which has " +
                                         std::to_string(it->second->get_output_size()));
            return Output<Node>(it->second, index);
        }
        // serializer.cpp:369-383 (opset-0 files: {"type": n, "axis": a}) and the attribute-visitor
        // spelling (a string); only what the elementwise ops here implement is let through
        static void check_auto_broadcast(const Json& node_js)
        {
            if (!node_js.has("auto_broadcast"))
                return;
            const Json& j = node_js.at("auto_broadcast");
            bool pdpd = j.is_string() ? (j.get_string() == "PDPD") : (j.at("type").get_int() == 2);
            if (pdpd)
                throw std::runtime_error("PDPD auto-broadcast is not supported");
        }
        template <typename OP>
        static std::shared_ptr<Node> binary(const Json& node_js, const OutputVector& args)
        {
            check_auto_broadcast(node_js);
            return std::make_shared<OP>(args.at(0), args.at(1));
        }

        std::shared_ptr<Node> make(const std::string& op_name, size_t version, const std::string& node_name, const Json& node_js, const OutputVector& args)
        {
            using namespace op;
            auto arg = [&](size_t i) -> const Output<Node>& {
                if (i >= args.size())
                    throw std::runtime_error("op " + op_name + " needs input " + std::to_string(i) + ", the node has " + std::to_string(args.size()));
                return args[i];
            };
            if (version == 0)
            {
                if (op_name == "Parameter")
                {
                    const Json& t = node_js.has("element_type") ? node_js : node_js.at("value_type");
                    return std::make_shared<v0::Parameter>(read_element_type(t.at("element_type")), read_shape(t.at("shape")));
                }
                if (op_name == "Constant")
                    return read_constant(node_js);
                if (op_name == "Result")
                    return std::make_shared<v0::Result>(arg(0));
                if (op_name == "GetOutputElement") // older files: an alias of output n of its input
                {
                    size_t n = node_js.has("n") ? node_js.at("n").get_size() : arg(0).get_index();
                    m_goe_alias.insert({node_name, Output<Node>(arg(0).get_node_shared_ptr(), n)});
                    return nullptr;
                }
                if (op_name == "Quantize")
                {
                    int64_t mode = node_js.at("round_mode").get_int();
                    if (mode < 0 || mode > static_cast<int64_t>(v0::Quantize::RoundMode::ROUND_DOWN))
                        throw std::runtime_error("round_mode " + std::to_string(mode) + " out of range");
                    return std::make_shared<v0::Quantize>(arg(0),
                                                          arg(1),
                                                          arg(2),
                                                          read_element_type(node_js.at("type")),
                                                          node_js.at("axes").get_axis_set(),
                                                          static_cast<v0::Quantize::RoundMode>(mode));
                }
                if (op_name == "Dequantize")
                    return std::make_shared<v0::Dequantize>(arg(0), arg(1), arg(2), read_element_type(node_js.at("type")), node_js.at("axes").get_axis_set());
                if (op_name == "QuantizedConvolution")
                    return std::make_shared<v0::QuantizedConvolution>(arg(0),
                                                                      arg(1),
                                                                      node_js.at("window_movement_strides").get_size_vector<Strides>(),
                                                                      node_js.at("window_dilation_strides").get_size_vector<Strides>(),
                                                                      node_js.at("padding_below").get_int_vector<CoordinateDiff>(),
                                                                      node_js.at("padding_above").get_int_vector<CoordinateDiff>(),
                                                                      node_js.at("data_dilation_strides").get_size_vector<Strides>(),
                                                                      arg(2),
                                                                      arg(3),
                                                                      arg(4),
                                                                      arg(5),
                                                                      arg(6),
                                                                      arg(7),
                                                                      read_element_type(node_js.at("output_type")),
                                                                      node_js.at("input_axes").get_axis_set(),
                                                                      node_js.at("filter_axes").get_axis_set(),
                                                                      node_js.at("output_axes").get_axis_set());
                if (op_name == "QuantizedDot")
                    return std::make_shared<v0::QuantizedDot>(arg(0),
                                                              arg(1),
                                                              node_js.at("reduction_axes_count").get_size(),
                                                              arg(2),
                                                              arg(3),
                                                              arg(4),
                                                              arg(5),
                                                              arg(6),
                                                              arg(7),
                                                              read_element_type(node_js.at("output_type")),
                                                              node_js.at("input0_axes").get_axis_set(),
                                                              node_js.at("input1_axes").get_axis_set(),
                                                              node_js.at("output_axes").get_axis_set());
                if (op_name == "Convert")
                    return std::make_shared<v0::Convert>(arg(0), read_element_type(node_js.at("target_type")));
                if (op_name == "Broadcast")
                    return std::make_shared<v0::Broadcast>(arg(0), read_shape(node_js.at("shape")), node_js.at("axes").get_axis_set());
                if (op_name == "Reshape")
                    return std::make_shared<v0::Reshape>(arg(0), node_js.at("input_order").get_size_vector<AxisVector>(), read_shape(node_js.at("output_shape")));
                if (op_name == "Abs")
                    return std::make_shared<v0::Abs>(arg(0));
                if (op_name == "Relu")
                    return std::make_shared<v0::Relu>(arg(0));
                if (op_name == "Erf")
                    return std::make_shared<v0::Erf>(arg(0));
                if (op_name == "Gelu")
                    return std::make_shared<v0::Gelu>(arg(0));
                if (op_name == "MaxPool" || op_name == "AvgPool")
                {
                    if (node_js.has("pad_type") && node_js.at("pad_type").get_int() != 0)
                        throw std::runtime_error("only explicit padding (pad_type 0) is supported");
                    if (node_js.has("ceil_mode") && node_js.at("ceil_mode").get_bool())
                        throw std::runtime_error("ceil_mode is not supported");
                    Shape window = read_shape(node_js.at("window_shape"));
                    Strides strides = node_js.at("window_movement_strides").get_size_vector<Strides>();
                    // MaxPool: both paddings may be absent (older files), but not just one
                    bool has_below = node_js.has("padding_below") && !node_js.at("padding_below").is_null();
                    bool has_above = node_js.has("padding_above") && !node_js.at("padding_above").is_null();
                    if (has_below != has_above)
                        throw std::runtime_error(op_name + ": padding_below and padding_above must come together");
                    Shape below = has_below ? read_shape(node_js.at("padding_below")) : Shape(window.size(), 0);
                    Shape above = has_above ? read_shape(node_js.at("padding_above")) : Shape(window.size(), 0);
                    if (op_name == "MaxPool")
                        return std::make_shared<v0::MaxPool>(arg(0), window, strides, below, above);
                    return std::make_shared<v0::AvgPool>(arg(0), window, strides, below, above, node_js.at("include_padding_in_avg_computation").get_bool());
                }
                if (op_name == "Concat")
                    return std::make_shared<v0::Concat>(args, static_cast<int64_t>(node_js.at("axis").get_size()));
                if (op_name == "Slice") // serializer.cpp:2387-2394
                    return std::make_shared<v0::Slice>(arg(0),
                                                       node_js.at("lower_bounds").get_size_vector<Coordinate>(),
                                                       node_js.at("upper_bounds").get_size_vector<Coordinate>(),
                                                       node_js.at("strides").get_size_vector<Strides>());
                if (op_name == "Softmax")
                {
                    if (node_js.has("softmax_axes"))
                        return std::make_shared<v0::Softmax>(arg(0), node_js.at("softmax_axes").get_axis_set());
                    // current files: the axes are a second, constant input
                    auto axes_node = as_type_ptr<v0::Constant>(arg(1).get_node_shared_ptr());
                    if (!axes_node)
                        throw std::runtime_error("Softmax axes must be a Constant");
                    AxisSet axes;
                    for (double a : axes_node->get_values_as_double())
                        axes.insert(static_cast<size_t>(a));
                    return std::make_shared<v0::Softmax>(arg(0), axes);
                }
                if (op_name == "LayerNorm")
                {
                    bool keep_stats = node_js.at("keep_stats").get_bool();
                    double epsilon = node_js.at("epsilon").get_double();
                    int64_t begin_norm_axis = node_js.at("begin_norm_axis").get_int();
                    if (node_js.at("use_affine").get_bool())
                        return std::make_shared<v0::LayerNorm>(arg(0), arg(1), arg(2), keep_stats, begin_norm_axis, epsilon);
                    return std::make_shared<v0::LayerNorm>(arg(0), keep_stats, begin_norm_axis, epsilon);
                }
                if (op_name == "BatchMatMul")
                    return std::make_shared<v0::BatchMatMul>(arg(0), arg(1));
                if (op_name == "BatchMatMulTranspose")
                    return std::make_shared<v0::BatchMatMulTranspose>(arg(0), arg(1), node_js.at("transpose_0").get_bool(), node_js.at("transpose_1").get_bool());
            }
            if (version <= 1)
            {
                // opset-0 names build the opset-1 ops, as nGraph's reader does (serializer.cpp:923-928 ...)
                if (op_name == "Add")
                    return binary<v1::Add>(node_js, args);
                if (op_name == "Subtract")
                    return binary<v1::Subtract>(node_js, args);
                if (op_name == "Multiply")
                    return binary<v1::Multiply>(node_js, args);
                if (op_name == "Maximum")
                    return binary<v1::Maximum>(node_js, args);
                if (op_name == "Minimum")
                    return binary<v1::Minimum>(node_js, args);
                if (op_name == "Divide")
                {
                    check_auto_broadcast(node_js);
                    bool pythondiv = true; // "pythondiv" in opset-0 files, the visited member "m_pythondiv" in opset 1
                    if (node_js.has("pythondiv"))
                        pythondiv = node_js.at("pythondiv").get_bool();
                    else if (node_js.has("m_pythondiv"))
                        pythondiv = node_js.at("m_pythondiv").get_bool();
                    return std::make_shared<v1::Divide>(arg(0), arg(1), pythondiv);
                }
            }
            throw std::runtime_error("unsupported op " + op_name + ":" + std::to_string(version));
        }

        void node(const Json& node_js)
        {
            std::string node_name = "UNKNOWN";
            try
            {
                const std::string& op = node_js.at("op").get_string();
                size_t version = node_js.has("op_version") ? node_js.at("op_version").get_size() : 0;
                node_name = node_js.at("name").get_string();
                OutputVector args;
                if (node_js.has("inputs") && node_js.at("inputs").is_array())
                    for (const Json& in : node_js.at("inputs").elements())
                        args.push_back(output(in));
                // "control_deps" order side effects; the ops read here have none, so they are not kept
                std::shared_ptr<Node> n = make(op, version, node_name, node_js, args);
                if (!n)
                    return;
                std::string friendly = node_js.has("friendly_name") ? node_js.at("friendly_name").get_string() : std::string();
                n->set_friendly_name(friendly.empty() ? node_name : friendly);
                m_nodes[node_name] = n;
            }
            catch (const std::exception& err)
            {
                if (node_name == "UNKNOWN" && node_js.is_object() && node_js.has("name") && node_js.at("name").is_string())
                    node_name = node_js.at("name").get_string();
                throw std::runtime_error("Error parsing json at node '" + node_name + "': " + err.what());
            }
        }

        std::map<std::string, std::shared_ptr<Node>> m_nodes;
        std::map<std::string, Output<Node>> m_goe_alias;
    };

    // ------------------------------------------------------------------------------ writer
    Json write_output(const Output<Node>& o)
    {
        if (o.get_index() == 0)
            return Json(o.get_node()->get_name());
        Json j = Json::object();
        j["node"] = Json(o.get_node()->get_name());
        j["index"] = Json(static_cast<uint64_t>(o.get_index()));
        return j;
    }

    Json write_axis_set(const AxisSet& s) { return Json::array_of(s); }

    Json write_node(const Node& n)
    {
        using namespace op;
        const NodeTypeInfo& info = n.get_type_info();
        Json node = Json::object();
        node["name"] = Json(n.get_name());
        node["op_version"] = Json(static_cast<uint64_t>(info.version));
        if (n.get_name() != n.get_friendly_name())
            node["friendly_name"] = Json(n.get_friendly_name());
        node["op"] = Json(info.name);
        if (n.get_input_size())
        {
            Json inputs = Json::array();
            for (size_t i = 0; i < n.get_input_size(); ++i)
                inputs.push_back(write_output(n.input_value(i)));
            node["inputs"] = inputs;
        }
        if (n.get_output_size())
        {
            Json outputs = Json::array();
            for (size_t i = 0; i < n.get_output_size(); ++i)
                outputs.push_back(Json(n.get_output_tensor(i).get_name()));
            node["outputs"] = outputs;
        }
        const Node* p = &n;
        if (auto c = as_type<const v0::Parameter>(p))
        {
            node["shape"] = Json::array_of(c->get_output_shape(0));
            node["cacheable"] = Json(false);
            node["element_type"] = write_element_type(c->get_output_element_type(0));
        }
        else if (auto c = as_type<const v0::Constant>(p))
        {
            node["value"] = write_constant_values(*c);
            node["shape"] = Json::array_of(c->get_output_shape(0));
            node["element_type"] = write_element_type(c->get_output_element_type(0));
        }
        else if (is_type<v0::Result>(p))
            node["needs_default_layout"] = Json(false);
        else if (auto c = as_type<const v0::Quantize>(p))
        {
            node["type"] = write_element_type(c->get_output_element_type(0));
            node["axes"] = write_axis_set(c->get_axes());
            node["round_mode"] = Json(static_cast<int64_t>(c->get_round_mode()));
        }
        else if (auto c = as_type<const v0::Dequantize>(p))
        {
            node["type"] = write_element_type(c->get_output_element_type(0));
            node["axes"] = write_axis_set(c->get_axes());
        }
        else if (auto c = as_type<const v0::QuantizedConvolution>(p))
        {
            node["window_movement_strides"] = Json::array_of(c->get_window_movement_strides());
            node["window_dilation_strides"] = Json::array_of(c->get_window_dilation_strides());
            node["padding_below"] = Json::array_of(c->get_padding_below());
            node["padding_above"] = Json::array_of(c->get_padding_above());
            node["data_dilation_strides"] = Json::array_of(c->get_data_dilation_strides());
            node["output_type"] = write_element_type(c->get_output_element_type(0));
            node["input_axes"] = write_axis_set(c->get_input_axes());
            node["filter_axes"] = write_axis_set(c->get_filter_axes());
            node["output_axes"] = write_axis_set(c->get_output_axes());
        }
        else if (auto c = as_type<const v0::QuantizedDot>(p))
        {
            node["reduction_axes_count"] = Json(static_cast<uint64_t>(c->get_reduction_axes_count()));
            node["output_type"] = write_element_type(c->get_output_element_type(0));
            node["input0_axes"] = write_axis_set(c->get_input0_axes());
            node["input1_axes"] = write_axis_set(c->get_input1_axes());
            node["output_axes"] = write_axis_set(c->get_output_axes());
        }
        else if (auto c = as_type<const v0::Convert>(p))
            node["target_type"] = write_element_type(c->get_destination_type());
        else if (auto c = as_type<const v0::Broadcast>(p))
        {
            node["axes"] = write_axis_set(c->get_broadcast_axes());
            node["shape"] = Json::array_of(c->get_broadcast_shape());
        }
        else if (auto c = as_type<const v0::Reshape>(p))
        {
            node["input_order"] = Json::array_of(c->get_input_order());
            node["output_shape"] = Json::array_of(c->get_output_shape(0));
        }
        else if (auto c = as_type<const v0::MaxPool>(p))
        {
            node["window_shape"] = Json::array_of(c->get_window_shape());
            node["window_movement_strides"] = Json::array_of(c->get_window_movement_strides());
            node["padding_below"] = Json::array_of(c->get_padding_below());
            node["padding_above"] = Json::array_of(c->get_padding_above());
            node["pad_type"] = Json(0);
        }
        else if (auto c = as_type<const v0::AvgPool>(p))
        {
            node["window_shape"] = Json::array_of(c->get_window_shape());
            node["window_movement_strides"] = Json::array_of(c->get_window_movement_strides());
            node["padding_below"] = Json::array_of(c->get_padding_below());
            node["padding_above"] = Json::array_of(c->get_padding_above());
            node["include_padding_in_avg_computation"] = Json(c->get_include_padding_in_avg_computation());
            node["pad_type"] = Json(0);
            node["ceil_mode"] = Json(false);
        }
        else if (auto c = as_type<const v0::Concat>(p))
            node["axis"] = Json(c->get_concatenation_axis());
        else if (auto c = as_type<const v0::Slice>(p))
        {
            node["lower_bounds"] = Json::array_of(c->get_lower_bounds());
            node["upper_bounds"] = Json::array_of(c->get_upper_bounds());
            node["strides"] = Json::array_of(c->get_strides());
        }
        else if (auto c = as_type<const v0::Softmax>(p))
            node["softmax_axes"] = write_axis_set(c->get_axes()); // the form with the axes as an attribute (serializer.cpp:2397-2401)
        else if (auto c = as_type<const v0::LayerNorm>(p))
        {
            node["keep_stats"] = Json(c->get_keep_stats());
            node["use_affine"] = Json(c->get_use_affine());
            node["epsilon"] = Json(c->get_epsilon());
            node["begin_norm_axis"] = Json(c->get_begin_norm_axis());
        }
        else if (auto c = as_type<const v0::BatchMatMulTranspose>(p))
        {
            node["transpose_0"] = Json(c->get_transpose_arg0());
            node["transpose_1"] = Json(c->get_transpose_arg1());
        }
        else if (is_type<v0::Abs>(p) || is_type<v0::Relu>(p) || is_type<v0::Erf>(p) || is_type<v0::Gelu>(p) || is_type<v0::BatchMatMul>(p))
        {
        }
        else if (is_type<v1::Add>(p) || is_type<v1::Subtract>(p) || is_type<v1::Multiply>(p) || is_type<v1::Maximum>(p) || is_type<v1::Minimum>(p) ||
                 is_type<v1::Divide>(p))
        {
            // opset-1 ops go through the attribute visitor in nGraph (serializer.cpp:3681-3694);
            // Maximum / Minimum have cases of their own there that write the same member
            if (!is_type<v1::Maximum>(p) && !is_type<v1::Minimum>(p))
            {
                node["attribute_visitor"] = Json(true);
                node["auto_broadcast"] = Json("NUMPY");
            }
            else
            {
                Json spec = Json::object();
                spec["type"] = Json(1); // AutoBroadcastType::NUMPY
                spec["axis"] = Json(0);
                node["auto_broadcast"] = spec;
            }
            if (auto d = as_type<const v1::Divide>(p))
                node["m_pythondiv"] = Json(d->is_pythondiv());
        }
        else
            throw ngraph_error(std::string("Cannot serialize: v") + std::to_string(info.version) + "::" + info.name);
        return node;
    }

    Json write_function(const Function& f)
    {
        Json function = Json::object();
        function["name"] = Json(f.get_name());
        Json params = Json::array();
        for (const auto& p : f.get_parameters())
            params.push_back(Json(p->get_name()));
        function["parameters"] = params;
        Json results = Json::array();
        for (const auto& r : f.get_results())
            results.push_back(Json(r->get_name()));
        function["result"] = results;
        Json ops = Json::array();
        for (const auto& n : f.get_ordered_ops())
            ops.push_back(write_node(*n));
        function["ops"] = ops;
        return function;
    }

    bool file_exists(const std::string& path)
    {
        struct stat st;
        return !path.empty() && path.size() < 4096 && path.find('\n') == std::string::npos && ::stat(path.c_str(), &st) == 0 && S_ISREG(st.st_mode);
    }

    std::shared_ptr<Function> read_text(const std::string& text)
    {
        // cpio containers (src/ngraph/cpio.cpp:297-325: magic 0x71C7 in either byte order, or the
        // ASCII forms) hold the json plus binary constants; they are not read here
        if (text.size() >= 2)
        {
            unsigned char a = static_cast<unsigned char>(text[0]), b = static_cast<unsigned char>(text[1]);
            if ((a == 0x71 && b == 0xC7) || (a == 0xC7 && b == 0x71) || text.compare(0, 5, "07070") == 0)
                throw ngraph_error("cpio containers are not supported: serialize the function as plain json");
        }
        Json js = JsonParser(text).parse();
        std::shared_ptr<Function> rc;
        for (const Json& func : js.elements())
        {
            Reader reader;
            rc = reader.function(func);
        }
        if (!rc)
            throw ngraph_error("the json holds no function");
        return rc;
    }
}

std::string ngraph::serialize(std::shared_ptr<Function> func, size_t indent)
{
    Json j = Json::array();
    j.push_back(write_function(*func));
    std::string out;
    j.dump(out, indent == 0 ? -1 : static_cast<int>(indent));
    return out;
}

void ngraph::serialize(const std::string& path, std::shared_ptr<Function> func, size_t indent)
{
    std::ofstream out(path);
    if (!out)
        throw ngraph_error("cannot open '" + path + "' for writing");
    serialize(out, func, indent);
}

void ngraph::serialize(std::ostream& out, std::shared_ptr<Function> func, size_t indent)
{
    out << serialize(func, indent);
}

std::shared_ptr<Function> ngraph::deserialize(std::istream& in)
{
    std::stringstream ss;
    ss << in.rdbuf();
    return read_text(ss.str());
}

std::shared_ptr<Function> ngraph::deserialize(const std::string& s)
{
    if (file_exists(s)) // a file name rather than json text (serializer.cpp:535-542)
    {
        std::ifstream in(s, std::ios_base::binary | std::ios_base::in);
        return deserialize(in);
    }
    return read_text(s);
}
