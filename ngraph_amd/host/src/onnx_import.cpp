// ONNX ingress for the quantized path (include/ngraph/frontend/onnx_import/onnx.hpp).
// Three layers: (1) a protobuf reader for binary and text files that yields one generic message
// tree (the ONNX messages involved are described by a small field table: no libprotobuf, no
// generated code); (2) the ONNX graph walk of src/ngraph/frontend/onnx_import/core/graph.cpp:
// initializers become Constants, the other graph inputs Parameters, nodes are converted in file
// order; (3) the operator functions, each following the reference's importer file named at it.
#include "ngraph/frontend/onnx_import/onnx.hpp"

#include <algorithm>
#include <cmath>
#include <cstring>
#include <fstream>
#include <functional>
#include <map>
#include <sstream>

#include "ngraph/builder.hpp"
#include "ngraph/ops.hpp"

using namespace std;

namespace ngraph
{
    namespace onnx_import
    {
        namespace
        {
            struct parse_error : ngraph_error
            {
                explicit parse_error(const string& what) : ngraph_error("ONNX model: " + what) {}
            };

            // ---------------------------------------------------------------- generic message tree
            struct Message;
            struct Value
            {
                enum Kind
                {
                    INT,
                    REAL,
                    STR,
                    MSG
                } kind = INT;
                int64_t i = 0;
                double d = 0.0;
                string s; // strings, bytes, and enum identifiers of text files
                shared_ptr<Message> m;
                int64_t as_int() const { return kind == REAL ? static_cast<int64_t>(d) : i; }
                double as_real() const { return kind == REAL ? d : static_cast<double>(i); }
            };
            struct Message
            {
                vector<pair<string, Value>> fields;
                vector<const Value*> all(const string& name) const
                {
                    vector<const Value*> out;
                    for (const auto& f : fields)
                        if (f.first == name)
                            out.push_back(&f.second);
                    return out;
                }
                const Value* one(const string& name) const
                {
                    const Value* last = nullptr; // protobuf: the last occurrence of a singular field wins
                    for (const auto& f : fields)
                        if (f.first == name)
                            last = &f.second;
                    return last;
                }
                bool has(const string& name) const { return one(name) != nullptr; }
                int64_t get_int(const string& name, int64_t dflt = 0) const
                {
                    const Value* v = one(name);
                    return v ? v->as_int() : dflt;
                }
                string get_str(const string& name, const string& dflt = "") const
                {
                    const Value* v = one(name);
                    return v ? v->s : dflt;
                }
                const Message* get_msg(const string& name) const
                {
                    const Value* v = one(name);
                    return v && v->kind == Value::MSG ? v->m.get() : nullptr;
                }
            };

            // ---------------------------------------------------------------- the ONNX schema, as far as needed
            // (onnx.proto of ONNX 1.x: field numbers and wire kinds of the messages a model of this kind uses)
            enum Wire
            {
                W_INT,   // varint (int32 / int64 / enum); repeated ones may come packed
                W_F32,   // fixed32 float; repeated ones may come packed
                W_F64,   // fixed64 double; repeated ones may come packed
                W_BYTES, // string / bytes
                W_MSG
            };
            struct FieldDesc
            {
                const char* name;
                Wire wire;
                const char* message; // W_MSG: type of the nested message
            };
            const map<string, map<int, FieldDesc>>& schema()
            {
                static const map<string, map<int, FieldDesc>> s = {
                    {"Model",
                     {{1, {"ir_version", W_INT, nullptr}},
                      {2, {"producer_name", W_BYTES, nullptr}},
                      {3, {"producer_version", W_BYTES, nullptr}},
                      {4, {"domain", W_BYTES, nullptr}},
                      {5, {"model_version", W_INT, nullptr}},
                      {6, {"doc_string", W_BYTES, nullptr}},
                      {7, {"graph", W_MSG, "Graph"}},
                      {8, {"opset_import", W_MSG, "OperatorSetId"}}}},
                    {"OperatorSetId", {{1, {"domain", W_BYTES, nullptr}}, {2, {"version", W_INT, nullptr}}}},
                    {"Graph",
                     {{1, {"node", W_MSG, "Node"}},
                      {2, {"name", W_BYTES, nullptr}},
                      {5, {"initializer", W_MSG, "Tensor"}},
                      {10, {"doc_string", W_BYTES, nullptr}},
                      {11, {"input", W_MSG, "ValueInfo"}},
                      {12, {"output", W_MSG, "ValueInfo"}},
                      {13, {"value_info", W_MSG, "ValueInfo"}}}},
                    {"Node",
                     {{1, {"input", W_BYTES, nullptr}},
                      {2, {"output", W_BYTES, nullptr}},
                      {3, {"name", W_BYTES, nullptr}},
                      {4, {"op_type", W_BYTES, nullptr}},
                      {5, {"attribute", W_MSG, "Attribute"}},
                      {6, {"doc_string", W_BYTES, nullptr}},
                      {7, {"domain", W_BYTES, nullptr}}}},
                    {"Attribute",
                     {{1, {"name", W_BYTES, nullptr}},
                      {2, {"f", W_F32, nullptr}},
                      {3, {"i", W_INT, nullptr}},
                      {4, {"s", W_BYTES, nullptr}},
                      {5, {"t", W_MSG, "Tensor"}},
                      {7, {"floats", W_F32, nullptr}},
                      {8, {"ints", W_INT, nullptr}},
                      {9, {"strings", W_BYTES, nullptr}},
                      {13, {"doc_string", W_BYTES, nullptr}},
                      {20, {"type", W_INT, nullptr}}}},
                    {"Tensor",
                     {{1, {"dims", W_INT, nullptr}},
                      {2, {"data_type", W_INT, nullptr}},
                      {4, {"float_data", W_F32, nullptr}},
                      {5, {"int32_data", W_INT, nullptr}},
                      {6, {"string_data", W_BYTES, nullptr}},
                      {7, {"int64_data", W_INT, nullptr}},
                      {8, {"name", W_BYTES, nullptr}},
                      {9, {"raw_data", W_BYTES, nullptr}},
                      {10, {"double_data", W_F64, nullptr}},
                      {11, {"uint64_data", W_INT, nullptr}},
                      {12, {"doc_string", W_BYTES, nullptr}}}},
                    {"ValueInfo", {{1, {"name", W_BYTES, nullptr}}, {2, {"type", W_MSG, "Type"}}, {3, {"doc_string", W_BYTES, nullptr}}}},
                    {"Type", {{1, {"tensor_type", W_MSG, "TypeTensor"}}}},
                    {"TypeTensor", {{1, {"elem_type", W_INT, nullptr}}, {2, {"shape", W_MSG, "Shape"}}}},
                    {"Shape", {{1, {"dim", W_MSG, "Dimension"}}}},
                    {"Dimension", {{1, {"dim_value", W_INT, nullptr}}, {2, {"dim_param", W_BYTES, nullptr}}, {3, {"denotation", W_BYTES, nullptr}}}},
                };
                return s;
            }

            // ---------------------------------------------------------------- binary wire format
            struct WireReader
            {
                const uint8_t* p;
                const uint8_t* end;
                bool more() const { return p < end; }
                uint64_t varint()
                {
                    uint64_t v = 0;
                    for (int shift = 0; shift < 70; shift += 7)
                    {
                        if (p >= end)
                            throw parse_error("truncated varint");
                        const uint8_t b = *p++;
                        v |= static_cast<uint64_t>(b & 0x7F) << (shift & 63);
                        if (!(b & 0x80))
                            return v;
                    }
                    throw parse_error("varint too long");
                }
                const uint8_t* take(size_t n)
                {
                    if (static_cast<size_t>(end - p) < n)
                        throw parse_error("truncated field");
                    const uint8_t* q = p;
                    p += n;
                    return q;
                }
            };

            Value real_value(double d)
            {
                Value v;
                v.kind = Value::REAL;
                v.d = d;
                return v;
            }
            Value int_value(int64_t i)
            {
                Value v;
                v.kind = Value::INT;
                v.i = i;
                return v;
            }

            shared_ptr<Message> read_binary(const uint8_t* begin, const uint8_t* end, const string& type, int depth = 0)
            {
                if (depth > 32)
                    throw parse_error("messages nested too deep");
                const auto& fields = schema().at(type);
                auto msg = make_shared<Message>();
                WireReader r{begin, end};
                while (r.more())
                {
                    const uint64_t key = r.varint();
                    const int number = static_cast<int>(key >> 3), wt = static_cast<int>(key & 7);
                    if (number == 0)
                        throw parse_error("field number 0");
                    const auto it = fields.find(number);
                    const FieldDesc* fd = it == fields.end() ? nullptr : &it->second;
                    switch (wt)
                    {
                    case 0:
                    {
                        const uint64_t v = r.varint();
                        if (fd && fd->wire == W_INT)
                            msg->fields.emplace_back(fd->name, int_value(static_cast<int64_t>(v)));
                        else if (fd)
                            throw parse_error(string("field ") + fd->name + " has the wrong wire type");
                        break;
                    }
                    case 1:
                    {
                        const uint8_t* q = r.take(8);
                        if (fd && fd->wire == W_F64)
                        {
                            double d;
                            memcpy(&d, q, 8);
                            msg->fields.emplace_back(fd->name, real_value(d));
                        }
                        else if (fd)
                            throw parse_error(string("field ") + fd->name + " has the wrong wire type");
                        break;
                    }
                    case 5:
                    {
                        const uint8_t* q = r.take(4);
                        if (fd && fd->wire == W_F32)
                        {
                            float f;
                            memcpy(&f, q, 4);
                            msg->fields.emplace_back(fd->name, real_value(f));
                        }
                        else if (fd)
                            throw parse_error(string("field ") + fd->name + " has the wrong wire type");
                        break;
                    }
                    case 2:
                    {
                        const uint64_t n = r.varint();
                        if (n > static_cast<uint64_t>(r.end - r.p))
                            throw parse_error("length-delimited field runs past the end");
                        const uint8_t* q = r.take(static_cast<size_t>(n));
                        if (!fd)
                            break;
                        if (fd->wire == W_BYTES)
                        {
                            Value v;
                            v.kind = Value::STR;
                            v.s.assign(reinterpret_cast<const char*>(q), static_cast<size_t>(n));
                            msg->fields.emplace_back(fd->name, move(v));
                        }
                        else if (fd->wire == W_MSG)
                        {
                            Value v;
                            v.kind = Value::MSG;
                            v.m = read_binary(q, q + n, fd->message, depth + 1);
                            msg->fields.emplace_back(fd->name, move(v));
                        }
                        else if (fd->wire == W_INT) // packed
                        {
                            WireReader pr{q, q + n};
                            while (pr.more())
                                msg->fields.emplace_back(fd->name, int_value(static_cast<int64_t>(pr.varint())));
                        }
                        else if (fd->wire == W_F32)
                        {
                            if (n % 4)
                                throw parse_error("packed floats of odd length");
                            for (uint64_t k = 0; k < n; k += 4)
                            {
                                float f;
                                memcpy(&f, q + k, 4);
                                msg->fields.emplace_back(fd->name, real_value(f));
                            }
                        }
                        else
                        {
                            if (n % 8)
                                throw parse_error("packed doubles of odd length");
                            for (uint64_t k = 0; k < n; k += 8)
                            {
                                double d;
                                memcpy(&d, q + k, 8);
                                msg->fields.emplace_back(fd->name, real_value(d));
                            }
                        }
                        break;
                    }
                    default: throw parse_error("unsupported wire type " + to_string(wt));
                    }
                }
                return msg;
            }

            // ---------------------------------------------------------------- text format
            class TextReader
            {
            public:
                explicit TextReader(const string& text) : m_text(text) {}
                shared_ptr<Message> parse()
                {
                    auto m = message(false, '}', 0);
                    skip();
                    if (m_pos != m_text.size())
                        fail("text after the end of the message");
                    return m;
                }

            private:
                const string& m_text;
                size_t m_pos = 0;

                [[noreturn]] void fail(const string& what) const
                {
                    size_t line = 1 + static_cast<size_t>(count(m_text.begin(), m_text.begin() + static_cast<ptrdiff_t>(min(m_pos, m_text.size())), '\n'));
                    throw parse_error("text format, line " + to_string(line) + ": " + what);
                }
                void skip()
                {
                    while (m_pos < m_text.size())
                    {
                        const char c = m_text[m_pos];
                        if (c == '#')
                            while (m_pos < m_text.size() && m_text[m_pos] != '\n')
                                ++m_pos;
                        else if (isspace(static_cast<unsigned char>(c)) || c == ',' || c == ';')
                            ++m_pos;
                        else
                            break;
                    }
                }
                bool at(char c)
                {
                    skip();
                    return m_pos < m_text.size() && m_text[m_pos] == c;
                }
                string identifier()
                {
                    skip();
                    const size_t start = m_pos;
                    while (m_pos < m_text.size() && (isalnum(static_cast<unsigned char>(m_text[m_pos])) || m_text[m_pos] == '_' || m_text[m_pos] == '.'))
                        ++m_pos;
                    if (m_pos == start)
                        fail("a field name was expected");
                    return m_text.substr(start, m_pos - start);
                }
                string quoted()
                {
                    // adjacent literals concatenate; C escapes, octal and hex included
                    string out;
                    while (at('"') || at('\''))
                    {
                        const char quote = m_text[m_pos++];
                        for (;;)
                        {
                            if (m_pos >= m_text.size())
                                fail("unterminated string");
                            char c = m_text[m_pos++];
                            if (c == quote)
                                break;
                            if (c != '\\')
                            {
                                out.push_back(c);
                                continue;
                            }
                            if (m_pos >= m_text.size())
                                fail("unterminated escape");
                            c = m_text[m_pos++];
                            if (c >= '0' && c <= '7')
                            {
                                int v = c - '0';
                                for (int k = 0; k < 2 && m_pos < m_text.size() && m_text[m_pos] >= '0' && m_text[m_pos] <= '7'; ++k)
                                    v = v * 8 + (m_text[m_pos++] - '0');
                                out.push_back(static_cast<char>(v));
                            }
                            else if (c == 'x' || c == 'X')
                            {
                                int v = 0, k = 0;
                                for (; k < 2 && m_pos < m_text.size() && isxdigit(static_cast<unsigned char>(m_text[m_pos])); ++k)
                                {
                                    const char h = m_text[m_pos++];
                                    v = v * 16 + (isdigit(static_cast<unsigned char>(h)) ? h - '0' : (tolower(h) - 'a' + 10));
                                }
                                if (k == 0)
                                    fail("\\x without digits");
                                out.push_back(static_cast<char>(v));
                            }
                            else
                            {
                                switch (c)
                                {
                                case 'n': out.push_back('\n'); break;
                                case 't': out.push_back('\t'); break;
                                case 'r': out.push_back('\r'); break;
                                case 'a': out.push_back('\a'); break;
                                case 'b': out.push_back('\b'); break;
                                case 'f': out.push_back('\f'); break;
                                case 'v': out.push_back('\v'); break;
                                default: out.push_back(c); // \\ \" \' \?
                                }
                            }
                        }
                    }
                    return out;
                }
                Value scalar()
                {
                    skip();
                    if (m_pos >= m_text.size())
                        fail("a value was expected");
                    const char c = m_text[m_pos];
                    Value v;
                    if (c == '"' || c == '\'')
                    {
                        v.kind = Value::STR;
                        v.s = quoted();
                        return v;
                    }
                    const size_t start = m_pos;
                    while (m_pos < m_text.size() && (isalnum(static_cast<unsigned char>(m_text[m_pos])) || strchr("+-._", m_text[m_pos])))
                        ++m_pos;
                    const string tok = m_text.substr(start, m_pos - start);
                    if (tok.empty())
                        fail("a value was expected");
                    string low = tok;
                    transform(low.begin(), low.end(), low.begin(), [](unsigned char ch) { return static_cast<char>(tolower(ch)); });
                    if (low == "inf" || low == "infinity" || low == "+inf")
                        return real_value(INFINITY);
                    if (low == "-inf" || low == "-infinity")
                        return real_value(-INFINITY);
                    if (low == "nan" || low == "-nan")
                        return real_value(NAN);
                    if (low == "true" || low == "false")
                        return int_value(low == "true");
                    if (isdigit(static_cast<unsigned char>(tok[0])) || ((tok[0] == '-' || tok[0] == '+' || tok[0] == '.') && tok.size() > 1))
                    {
                        string num = tok;
                        if (!num.empty() && (num.back() == 'f' || num.back() == 'F') && num.find_first_of("xX") == string::npos)
                            num.pop_back();
                        char* endp = nullptr;
                        if (num.find_first_of(".eE") == string::npos || num.find_first_of("xX") != string::npos)
                        {
                            errno = 0;
                            const long long i = strtoll(num.c_str(), &endp, 0);
                            if (*endp == '\0' && errno == 0)
                                return int_value(i);
                            errno = 0;
                            const unsigned long long u = strtoull(num.c_str(), &endp, 0);
                            if (*endp == '\0' && errno == 0)
                                return int_value(static_cast<int64_t>(u));
                        }
                        const double d = strtod(num.c_str(), &endp);
                        if (*endp != '\0')
                            fail("malformed number '" + tok + "'");
                        return real_value(d);
                    }
                    v.kind = Value::STR; // an enum identifier
                    v.s = tok;
                    return v;
                }
                shared_ptr<Message> message(bool nested, char close, int depth)
                {
                    if (depth > 32)
                        fail("messages nested too deep");
                    auto msg = make_shared<Message>();
                    for (;;)
                    {
                        skip();
                        if (m_pos >= m_text.size())
                        {
                            if (nested)
                                fail("unterminated message");
                            return msg;
                        }
                        if (nested && m_text[m_pos] == close)
                        {
                            ++m_pos;
                            return msg;
                        }
                        const string name = identifier();
                        const bool colon = at(':');
                        if (colon)
                            ++m_pos;
                        if (at('{') || at('<'))
                        {
                            const char closing = m_text[m_pos] == '{' ? '}' : '>';
                            ++m_pos;
                            Value v;
                            v.kind = Value::MSG;
                            v.m = message(true, closing, depth + 1);
                            msg->fields.emplace_back(name, move(v));
                            continue;
                        }
                        if (!colon)
                            fail("':' or '{' expected after '" + name + "'");
                        if (at('['))
                        {
                            ++m_pos;
                            while (!at(']'))
                            {
                                if (at('{') || at('<'))
                                {
                                    const char closing = m_text[m_pos] == '{' ? '}' : '>';
                                    ++m_pos;
                                    Value v;
                                    v.kind = Value::MSG;
                                    v.m = message(true, closing, depth + 1);
                                    msg->fields.emplace_back(name, move(v));
                                }
                                else
                                    msg->fields.emplace_back(name, scalar());
                            }
                            ++m_pos;
                            continue;
                        }
                        msg->fields.emplace_back(name, scalar());
                    }
                }
            };

            shared_ptr<Message> read_model(const string& bytes)
            {
                // binary first, text second (onnx.cpp:54-71)
                try
                {
                    auto m = read_binary(reinterpret_cast<const uint8_t*>(bytes.data()), reinterpret_cast<const uint8_t*>(bytes.data()) + bytes.size(), "Model");
                    if (m->get_msg("graph"))
                        return m;
                }
                catch (const parse_error&)
                {
                }
                shared_ptr<Message> m;
                try
                {
                    m = TextReader(bytes).parse();
                }
                catch (const parse_error& e)
                {
                    throw ngraph_error(string("Failure parsing data from the provided input stream (") + e.what() + ")");
                }
                if (!m->get_msg("graph"))
                    throw ngraph_error("Failure parsing data from the provided input stream (the model has no graph)");
                return m;
            }

            // ---------------------------------------------------------------- tensors and types
            // TensorProto.DataType
            enum
            {
                ONNX_FLOAT = 1,
                ONNX_UINT8 = 2,
                ONNX_INT8 = 3,
                ONNX_INT32 = 6,
                ONNX_INT64 = 7,
                ONNX_BOOL = 9,
                ONNX_DOUBLE = 11
            };
            element::Type element_type_of(int64_t onnx_type, const string& where)
            {
                switch (onnx_type)
                {
                case ONNX_FLOAT: return element::f32;
                case ONNX_UINT8: return element::u8;
                case ONNX_INT8: return element::i8;
                case ONNX_INT32: return element::i32;
                case ONNX_INT64: return element::i64;
                case ONNX_BOOL: return element::boolean;
                case ONNX_DOUBLE: return element::f64;
                default: throw ngraph_error("ONNX model: " + where + " has element type " + to_string(onnx_type) + ", which this importer does not map");
                }
            }
            // an enum field: a number in binary files, a number or the enumerator's name in text files
            int64_t data_type_of(const Message& m, const string& field)
            {
                const Value* v = m.one(field);
                if (!v)
                    return 0;
                if (v->kind != Value::STR)
                    return v->as_int();
                static const map<string, int64_t> names = {{"FLOAT", ONNX_FLOAT}, {"UINT8", ONNX_UINT8}, {"INT8", ONNX_INT8}, {"INT32", ONNX_INT32},
                                                           {"INT64", ONNX_INT64}, {"BOOL", ONNX_BOOL},   {"DOUBLE", ONNX_DOUBLE}};
                const auto it = names.find(v->s);
                return it == names.end() ? -1 : it->second;
            }

            shared_ptr<op::v0::Constant> constant_of(const Message& t, const string& where)
            {
                Shape shape;
                for (const Value* d : t.all("dims"))
                {
                    NGRAPH_CHECK(d->as_int() >= 0, "ONNX model: ", where, " has a negative dimension");
                    shape.push_back(static_cast<size_t>(d->as_int()));
                }
                const int64_t dt = data_type_of(t, "data_type");
                const element::Type et = element_type_of(dt, where);
                const size_t count = shape_size(shape);
                if (const Value* raw = t.one("raw_data"))
                {
                    NGRAPH_CHECK(raw->s.size() == count * et.size(), "ONNX model: ", where, " holds ", raw->s.size(), " raw bytes for ", count, " elements of ", et.size(), " bytes");
                    return make_shared<op::v0::Constant>(et, shape, raw->s.data());
                }
                const char* field = dt == ONNX_FLOAT ? "float_data" : dt == ONNX_DOUBLE ? "double_data" : dt == ONNX_INT64 ? "int64_data" : "int32_data";
                vector<double> values;
                for (const Value* v : t.all(field))
                    values.push_back(v->as_real());
                NGRAPH_CHECK(values.size() == count, "ONNX model: ", where, " holds ", values.size(), " values in ", field, " for ", count, " elements");
                if (count == 0)
                    return make_shared<op::v0::Constant>(et, shape, static_cast<const void*>(""));
                if (dt == ONNX_INT64)
                {
                    vector<int64_t> exact; // doubles would round above 2^53
                    for (const Value* v : t.all(field))
                        exact.push_back(v->as_int());
                    return make_shared<op::v0::Constant>(et, shape, exact.data());
                }
                return make_shared<op::v0::Constant>(et, shape, values);
            }

            // ---------------------------------------------------------------- a node of the ONNX graph
            class OnnxNode
            {
            public:
                OnnxNode(const Message& m, OutputVector inputs, int64_t opset) : m_msg(m), m_inputs(move(inputs)), m_opset(opset) {}
                const OutputVector& inputs() const { return m_inputs; }
                // an optional input that was left out ("" in the file, or past the end of the list)
                bool has_input(size_t i) const { return i < m_inputs.size() && m_inputs[i].get_node() != nullptr; }
                const Output<Node>& input(size_t i) const
                {
                    if (!has_input(i))
                        throw ngraph_error(description() + ": input " + to_string(i) + " is missing");
                    return m_inputs[i];
                }
                int64_t opset() const { return m_opset; }
                string op_type() const { return m_msg.get_str("op_type"); }
                string description() const
                {
                    const string name = m_msg.get_str("name");
                    return "ONNX node " + (name.empty() ? string("<") + m_msg.get_str("op_type") + ">" : name + " (" + m_msg.get_str("op_type") + ")");
                }
                const Message* attribute(const string& name) const
                {
                    for (const Value* a : m_msg.all("attribute"))
                        if (a->kind == Value::MSG && a->m->get_str("name") == name)
                            return a->m.get();
                    return nullptr;
                }
                bool has_attribute(const string& name) const { return attribute(name) != nullptr; }
                int64_t get_int(const string& name, int64_t dflt) const
                {
                    const Message* a = attribute(name);
                    return a && a->has("i") ? a->get_int("i") : dflt;
                }
                string get_string(const string& name, const string& dflt) const
                {
                    const Message* a = attribute(name);
                    return a && a->has("s") ? a->get_str("s") : dflt;
                }
                vector<int64_t> get_ints(const string& name) const
                {
                    vector<int64_t> out;
                    if (const Message* a = attribute(name))
                        for (const Value* v : a->all("ints"))
                            out.push_back(v->as_int());
                    return out;
                }

            private:
                const Message& m_msg;
                OutputVector m_inputs;
                int64_t m_opset;
            };

            // ---------------------------------------------------------------- convolution attributes
            // src/ngraph/frontend/onnx_import/utils/convpool.cpp:31-200
            struct ConvGeometry
            {
                Strides strides, dilations, data_dilations;
                CoordinateDiff pads_below, pads_above;
            };
            ConvGeometry conv_geometry(const OnnxNode& node, const Output<Node>& data, const Output<Node>& filters)
            {
                const Shape& ds = data.get_shape();
                const Shape& fs = filters.get_shape();
                NGRAPH_CHECK(ds.size() >= 3 && fs.size() == ds.size(), node.description(), ": data and filters must have the same rank, at least 3");
                const size_t spatial = ds.size() - 2;
                auto sizes = [&](const string& attr) {
                    vector<size_t> out(spatial, 1);
                    if (node.has_attribute(attr))
                    {
                        const auto v = node.get_ints(attr);
                        NGRAPH_CHECK(v.size() == spatial, node.description(), ": '", attr, "' must have one value a spatial axis");
                        for (size_t i = 0; i < spatial; ++i)
                        {
                            NGRAPH_CHECK(v[i] >= 1, node.description(), ": '", attr, "' must be positive");
                            out[i] = static_cast<size_t>(v[i]);
                        }
                    }
                    return out;
                };
                ConvGeometry g;
                g.strides = Strides(sizes("strides"));
                g.dilations = Strides(sizes("dilations"));
                g.data_dilations = Strides(spatial, 1);
                CoordinateDiff pads(spatial, 0);
                if (node.has_attribute("pads"))
                {
                    const auto v = node.get_ints("pads");
                    pads = CoordinateDiff(v.begin(), v.end());
                }
                if (pads.size() == spatial * 2)
                {
                    g.pads_below = CoordinateDiff(pads.begin(), pads.begin() + static_cast<ptrdiff_t>(spatial));
                    g.pads_above = CoordinateDiff(pads.begin() + static_cast<ptrdiff_t>(spatial), pads.end());
                }
                else // none, or one side only: the same at both ends
                {
                    NGRAPH_CHECK(pads.size() == spatial, node.description(), ": 'pads' must have one or two values a spatial axis");
                    g.pads_below = g.pads_above = pads;
                }
                const string auto_pad = node.get_string("auto_pad", "NOTSET");
                NGRAPH_CHECK(auto_pad == "NOTSET" || auto_pad == "" || auto_pad == "VALID" || auto_pad == "SAME_UPPER" || auto_pad == "SAME_LOWER",
                             node.description(),
                             ": Provided `auto_pad` attribute value: '",
                             auto_pad,
                             "' is invalid.");
                if (auto_pad == "SAME_UPPER" || auto_pad == "SAME_LOWER")
                {
                    // src/ngraph/validation_util.cpp:604-627 (infer_auto_padding)
                    g.pads_below.clear();
                    g.pads_above.clear();
                    for (size_t i = 0; i < spatial; ++i)
                    {
                        const int64_t image = static_cast<int64_t>(ds[i + 2]);
                        const int64_t window = (static_cast<int64_t>(fs[i + 2]) - 1) * static_cast<int64_t>(g.dilations[i]) + 1;
                        const int64_t stride = static_cast<int64_t>(g.strides[i]);
                        const int64_t out = (image + stride - 1) / stride;
                        const int64_t needed = max<int64_t>(0, (out - 1) * stride + window - image);
                        const int64_t lhs = needed / 2, rhs = needed - lhs;
                        g.pads_below.push_back(auto_pad == "SAME_UPPER" ? lhs : rhs);
                        g.pads_above.push_back(auto_pad == "SAME_UPPER" ? rhs : lhs);
                    }
                }
                return g;
            }

            element::Type quantized_result_type(const OnnxNode& node, const Output<Node>& a, const Output<Node>& b)
            {
                // quant_conv.cpp:69-79, matmul_factory.cpp:167-178: u8 x i8 -> i8, u8 x u8 -> u8
                if (a.get_element_type() == element::u8 && b.get_element_type() == element::i8)
                    return element::i8;
                if (a.get_element_type() == element::u8 && b.get_element_type() == element::u8)
                    return element::u8;
                throw ngraph_error(node.description() + ": operands must be u8 x i8 or u8 x u8");
            }

            // ---------------------------------------------------------------- operators
            using OperatorFn = function<OutputVector(const OnnxNode&)>;

            // op/quantize_linear.cpp:33-72
            OutputVector quantize_linear(const OnnxNode& node)
            {
                const Output<Node>& x = node.input(0);
                const Output<Node>& y_scale = node.input(1);
                const Output<Node>& y_zero_point = node.input(2);
                AxisSet axes;
                if (node.has_attribute("axis"))
                {
                    const int64_t axis = node.get_int("axis", 1);
                    const int64_t rank = static_cast<int64_t>(x.get_shape().size());
                    NGRAPH_CHECK(axis >= -rank && axis < rank, node.description(), ": axis ", axis, " is out of range for rank ", rank);
                    axes.insert(static_cast<size_t>(axis >= 0 ? axis : axis + rank));
                }
                return {make_shared<op::v0::Quantize>(x, y_scale, y_zero_point, y_zero_point.get_element_type(), axes, op::v0::Quantize::RoundMode::ROUND_NEAREST_TOWARD_EVEN)};
            }

            // op/dequantize_linear.cpp:37-80
            OutputVector dequantize_linear(const OnnxNode& node)
            {
                const Output<Node>& x = node.input(0);
                const Output<Node>& x_scale = node.input(1);
                Output<Node> zero_point = node.has_input(2) ? node.input(2) : Output<Node>(builder::make_constant(x.get_element_type(), Shape{}, 0));
                AxisSet axes;
                if (node.has_attribute("axis"))
                {
                    const int64_t axis = node.get_int("axis", 1);
                    const int64_t rank = static_cast<int64_t>(x.get_shape().size());
                    NGRAPH_CHECK(axis >= -rank && axis < rank, node.description(), ": axis ", axis, " is out of range for rank ", rank);
                    axes.insert(static_cast<size_t>(axis >= 0 ? axis : axis + rank));
                }
                if (x.get_element_type() != zero_point.get_element_type())
                    zero_point = make_shared<op::v0::Convert>(zero_point, x.get_element_type());
                return {make_shared<op::v0::Dequantize>(x, x_scale, zero_point, x_scale.get_element_type(), axes)};
            }

            // op/quant_conv.cpp:57-270
            OutputVector qlinear_conv(const OnnxNode& node)
            {
                const Output<Node>& data = node.input(0);
                const Output<Node>& filters = node.input(3);
                const int64_t groups = node.get_int("group", 1);
                NGRAPH_CHECK(data.get_shape().size() >= 3 && filters.get_shape().size() >= 3, node.description(), ": data and filters must have rank 3 or more");
                NGRAPH_CHECK(groups >= 0 && groups <= static_cast<int64_t>(data.get_shape().at(1)) && groups <= static_cast<int64_t>(filters.get_shape().at(0)),
                             node.description(),
                             ": incorrect value of 'group' attribute: ",
                             groups);
                NGRAPH_CHECK(groups >= 1 && data.get_shape().at(1) % static_cast<size_t>(groups) == 0 && filters.get_shape().at(0) % static_cast<size_t>(groups) == 0,
                             node.description(),
                             ": the channels of data and filters must be multiples of 'group' (",
                             groups,
                             ")");
                const ConvGeometry g = conv_geometry(node, data, filters);
                if (groups > 1)
                {
                    // quant_conv.cpp:80-138: one convolution a group over slices of the data's channels and of
                    // the filters, concatenated along the channel axis
                    if (node.has_input(8))
                        throw ngraph_error(node.description() + ": Groups != 1 not supported for Quantized Convolution with bias.");
                    const size_t data_group = data.get_shape().at(1) / static_cast<size_t>(groups), filters_group = filters.get_shape().at(0) / static_cast<size_t>(groups);
                    OutputVector pieces;
                    for (size_t group = 0; group < static_cast<size_t>(groups); ++group)
                    {
                        Coordinate data_lower(data.get_shape().size(), 0), data_upper(data.get_shape().begin(), data.get_shape().end());
                        data_lower[1] = group * data_group;
                        data_upper[1] = (group + 1) * data_group;
                        Coordinate filters_lower(filters.get_shape().size(), 0), filters_upper(filters.get_shape().begin(), filters.get_shape().end());
                        filters_lower[0] = group * filters_group;
                        filters_upper[0] = (group + 1) * filters_group;
                        const Output<Node> sliced_data = make_shared<op::v0::Slice>(data, data_lower, data_upper);
                        const Output<Node> sliced_filters = make_shared<op::v0::Slice>(filters, filters_lower, filters_upper);
                        pieces.push_back(make_shared<op::v0::QuantizedConvolution>(sliced_data,
                                                                                   sliced_filters,
                                                                                   g.strides,
                                                                                   g.dilations,
                                                                                   g.pads_below,
                                                                                   g.pads_above,
                                                                                   g.data_dilations,
                                                                                   node.input(1),
                                                                                   node.input(2),
                                                                                   node.input(4),
                                                                                   node.input(5),
                                                                                   node.input(6),
                                                                                   node.input(7),
                                                                                   quantized_result_type(node, data, filters),
                                                                                   AxisSet{},
                                                                                   AxisSet{},
                                                                                   AxisSet{}));
                    }
                    return {make_shared<op::v0::Concat>(pieces, 1)};
                }
                if (node.has_input(8))
                {
                    // builder/quantization/quantized_linear_convolution.cpp:38-77
                    const Output<Node>& bias = node.input(8);
                    const Output<Node> in_times_filter = make_shared<op::v1::Multiply>(node.input(1), node.input(4));
                    const Output<Node> requantization_scale = make_shared<op::v1::Divide>(in_times_filter, node.input(6));
                    Output<Node> my_bias = bias;
                    if (bias.get_element_type() != element::i32)
                    {
                        const auto zero = builder::make_constant(element::i32, node.input(1).get_shape(), 0);
                        const Output<Node> bias_scale = make_shared<op::v1::Multiply>(node.input(1), node.input(4));
                        my_bias = make_shared<op::v0::Quantize>(bias, bias_scale, zero, element::i32, AxisSet{}, op::v0::Quantize::RoundMode::ROUND_NEAREST_TOWARD_EVEN);
                    }
                    return {make_shared<op::v0::QuantizedConvolutionBias>(data, filters, my_bias, g.strides, g.dilations, g.pads_below, g.pads_above, g.data_dilations, requantization_scale, false)};
                }
                return {make_shared<op::v0::QuantizedConvolution>(data,
                                                                  filters,
                                                                  g.strides,
                                                                  g.dilations,
                                                                  g.pads_below,
                                                                  g.pads_above,
                                                                  g.data_dilations,
                                                                  node.input(1),
                                                                  node.input(2),
                                                                  node.input(4),
                                                                  node.input(5),
                                                                  node.input(6),
                                                                  node.input(7),
                                                                  quantized_result_type(node, data, filters),
                                                                  AxisSet{},
                                                                  AxisSet{},
                                                                  AxisSet{})};
            }

            // op/conv_integer.cpp:34-113
            OutputVector conv_integer(const OnnxNode& node)
            {
                const Output<Node>& input = node.input(0);
                const Output<Node>& filters = node.input(1);
                const int64_t groups = node.get_int("group", 1);
                NGRAPH_CHECK(groups == 1, node.description(), ": Only value of 1 for 'group' supported for ConvInteger. Given: ", groups);
                const ConvGeometry g = conv_geometry(node, input, filters);
                const Output<Node> scale_one = builder::make_constant(element::f32, Shape{}, 1);
                const Output<Node> input_zero_point = node.has_input(2) ? node.input(2) : Output<Node>(builder::make_constant(input.get_element_type(), Shape{}, 0));
                const Output<Node> filters_zero_point = node.has_input(3) ? node.input(3) : Output<Node>(builder::make_constant(filters.get_element_type(), Shape{}, 0));
                const Output<Node> output_zero_point = builder::make_constant(element::i32, Shape{}, 0);
                return {make_shared<op::v0::QuantizedConvolution>(input,
                                                                  filters,
                                                                  g.strides,
                                                                  g.dilations,
                                                                  g.pads_below,
                                                                  g.pads_above,
                                                                  g.data_dilations,
                                                                  scale_one,
                                                                  input_zero_point,
                                                                  scale_one,
                                                                  filters_zero_point,
                                                                  scale_one,
                                                                  output_zero_point,
                                                                  element::i32,
                                                                  AxisSet{},
                                                                  AxisSet{},
                                                                  AxisSet{})};
            }

            // builder/matmul_factory.cpp:71-150: operands of rank <= 2 are one dot; stacks of matrices get
            // their stack axes broadcast numpy-style against each other (builder/autobroadcast.cpp:95-110,
            // 138-184, 285-318: a Reshape that drops the axes of length 1 to be repeated, then a
            // Broadcast over them), are collapsed to rank 3, multiplied matrix by matrix (Slice, squeeze,
            // dot, expand) and concatenated, then given their stack axes back.
            OutputVector matmul_of(const OnnxNode& node, Output<Node> left, Output<Node> right, const function<Output<Node>(const Output<Node>&, const Output<Node>&)>& make_dot)
            {
                if (left.get_shape().size() <= 2 && right.get_shape().size() <= 2)
                    return {make_dot(left, right)};
                // (the reference slices nothing out of a vector and multiplies it with every matrix of
                // the other operand's stack; the quantized dot of this library takes matrices)
                if (left.get_shape().size() < 2 || right.get_shape().size() < 2)
                    throw ngraph_error(node.description() + ": a vector against a stack of matrices is not supported here");
                auto identity_order = [](size_t rank) {
                    AxisVector order(rank);
                    for (size_t i = 0; i < rank; ++i)
                        order[i] = i;
                    return order;
                };
                {
                    const Shape ls = left.get_shape(), rs = right.get_shape();
                    const Shape lstack(ls.begin(), ls.end() - 2), rstack(rs.begin(), rs.end() - 2);
                    // the stack both operands are repeated to: axes aligned at the right, lengths equal or 1
                    const size_t rank = max(lstack.size(), rstack.size());
                    Shape lfull(rank - lstack.size(), 1), rfull(rank - rstack.size(), 1), target(rank);
                    lfull.insert(lfull.end(), lstack.begin(), lstack.end());
                    rfull.insert(rfull.end(), rstack.begin(), rstack.end());
                    for (size_t i = 0; i < rank; ++i)
                    {
                        if (lfull[i] != rfull[i] && lfull[i] != 1 && rfull[i] != 1)
                            throw ngraph_error(node.description() + ": the stack shapes of the operands cannot be broadcast against each other (axis " + to_string(i) + ": " +
                                               to_string(lfull[i]) + " and " + to_string(rfull[i]) + ")");
                        target[i] = lfull[i] == 1 ? rfull[i] : lfull[i];
                    }
                    auto repeat = [&](const Output<Node>& x, Shape full) -> Output<Node> {
                        const Shape& xs = x.get_shape();
                        Shape out = target;
                        out.insert(out.end(), xs.end() - 2, xs.end());
                        full.insert(full.end(), xs.end() - 2, xs.end());
                        if (out == xs)
                            return x;
                        AxisSet repeated;
                        Shape squeezed;
                        for (size_t i = 0; i < out.size(); ++i)
                        {
                            if (full[i] == 1 && out[i] != 1)
                                repeated.insert(i);
                            else
                                squeezed.push_back(full[i]);
                        }
                        Output<Node> y = x;
                        if (squeezed != xs)
                            y = make_shared<op::v0::Reshape>(y, identity_order(xs.size()), squeezed);
                        if (!repeated.empty())
                            y = make_shared<op::v0::Broadcast>(y, out, repeated);
                        return y;
                    };
                    left = repeat(left, lfull);
                    right = repeat(right, rfull);
                }
                const Shape left_shape = left.get_shape(), right_shape = right.get_shape();
                auto reshape = [](const Output<Node>& x, const Shape& to) {
                    AxisVector order(x.get_shape().size());
                    for (size_t i = 0; i < order.size(); ++i)
                        order[i] = i;
                    return Output<Node>(make_shared<op::v0::Reshape>(x, order, to));
                };
                auto collapse = [&](const Output<Node>& x) {
                    const Shape& s = x.get_shape();
                    if (s.size() <= 3)
                        return x;
                    size_t stack = 1;
                    for (size_t i = 0; i + 2 < s.size(); ++i)
                        stack *= s[i];
                    return reshape(x, Shape{stack, s[s.size() - 2], s[s.size() - 1]});
                };
                left = collapse(left);
                right = collapse(right);
                const size_t groups = left.get_shape().at(0);
                auto sub_matrix = [&](const Output<Node>& x, size_t idx) {
                    const Shape& s = x.get_shape();
                    Coordinate lower(s.size(), 0), upper(s.begin(), s.end());
                    lower[0] = idx;
                    upper[0] = idx + 1;
                    return reshape(make_shared<op::v0::Slice>(x, lower, upper), Shape{s[1], s[2]});
                };
                OutputVector small_dots;
                for (size_t g = 0; g < groups; ++g)
                {
                    const Output<Node> sub_dot = make_dot(sub_matrix(left, g), sub_matrix(right, g));
                    const Shape& ds = sub_dot.get_shape();
                    small_dots.push_back(reshape(sub_dot, Shape{1, ds.at(0), ds.at(1)}));
                }
                const Output<Node> result = make_shared<op::v0::Concat>(small_dots, 0);
                if (left_shape.size() <= 3)
                    return {result};
                Shape result_shape(left_shape.begin(), left_shape.end() - 2);
                result_shape.push_back(result.get_shape().at(1));
                result_shape.push_back(result.get_shape().at(2));
                return {reshape(result, result_shape)};
            }

            // op/qlinear_matmul.cpp:30-47 with builder/matmul_factory.cpp:159-193
            OutputVector qlinear_matmul(const OnnxNode& node)
            {
                return matmul_of(node, node.input(0), node.input(3), [&](const Output<Node>& left, const Output<Node>& right) {
                    return Output<Node>(make_shared<op::v0::QuantizedDot>(left,
                                                                         right,
                                                                         1,
                                                                         node.input(1),
                                                                         node.input(2),
                                                                         node.input(4),
                                                                         node.input(5),
                                                                         node.input(6),
                                                                         node.input(7),
                                                                         quantized_result_type(node, left, right),
                                                                         AxisSet{},
                                                                         AxisSet{},
                                                                         AxisSet{}));
                });
            }

            // op/matmul_integer.cpp with builder/matmul_factory.cpp:195-243
            OutputVector matmul_integer(const OnnxNode& node)
            {
                const Output<Node> scale_one = builder::make_constant(element::f32, Shape{}, 1);
                const Output<Node> output_zero_point = builder::make_constant(element::i32, Shape{}, 0);
                const Output<Node> left_zero_point = node.has_input(2) ? node.input(2) : Output<Node>(builder::make_constant(node.input(0).get_element_type(), Shape{}, 0));
                const Output<Node> right_zero_point = node.has_input(3) ? node.input(3) : Output<Node>(builder::make_constant(node.input(1).get_element_type(), Shape{}, 0));
                return matmul_of(node, node.input(0), node.input(1), [&](const Output<Node>& left, const Output<Node>& right) {
                    return Output<Node>(make_shared<op::v0::QuantizedDot>(
                        left, right, 1, scale_one, left_zero_point, scale_one, right_zero_point, scale_one, output_zero_point, element::i32, AxisSet{}, AxisSet{}, AxisSet{}));
                });
            }

            // op/constant.cpp: the `value` tensor
            OutputVector constant(const OnnxNode& node)
            {
                const Message* a = node.attribute("value");
                const Message* t = a ? a->get_msg("t") : nullptr;
                if (!t)
                    throw ngraph_error(node.description() + ": a 'value' tensor attribute is required");
                return {constant_of(*t, node.description())};
            }

            OutputVector identity(const OnnxNode& node) { return {node.input(0)}; }
            OutputVector relu(const OnnxNode& node) { return {make_shared<op::v0::Relu>(node.input(0))}; }
            OutputVector add(const OnnxNode& node)
            {
                // (opset 7 and later broadcast numpy-style; the models of this path add equal shapes)
                NGRAPH_CHECK(node.input(0).get_shape() == node.input(1).get_shape(), node.description(), ": operands of different shapes are not supported here");
                return {make_shared<op::v1::Add>(node.input(0), node.input(1))};
            }

            // name -> first opset version that has it -> function (ops_bridge.cpp keeps the same map)
            const map<string, map<int64_t, OperatorFn>>& operators()
            {
                static const map<string, map<int64_t, OperatorFn>> ops = {
                    {"Add", {{1, add}}},
                    {"Constant", {{1, constant}}},
                    {"ConvInteger", {{1, conv_integer}}},
                    {"DequantizeLinear", {{1, dequantize_linear}}},
                    {"Identity", {{1, identity}}},
                    {"MatMulInteger", {{1, matmul_integer}}},
                    {"QLinearConv", {{1, qlinear_conv}}},
                    {"QLinearMatMul", {{1, qlinear_matmul}}},
                    {"QuantizeLinear", {{1, quantize_linear}}},
                    {"Relu", {{1, relu}}},
                };
                return ops;
            }

            const OperatorFn* find_operator(const string& name, int64_t version, const string& domain)
            {
                if (!domain.empty() && domain != "ai.onnx")
                    return nullptr;
                const auto it = operators().find(name);
                if (it == operators().end())
                    return nullptr;
                // the newest definition not newer than the model's opset (ops_bridge.cpp:57-75)
                const OperatorFn* best = nullptr;
                for (const auto& v : it->second)
                    if (v.first <= version)
                        best = &v.second;
                return best;
            }

            // ---------------------------------------------------------------- the graph (core/graph.cpp:63-150)
            shared_ptr<Function> build_function(const Message& model)
            {
                const Message& graph = *model.get_msg("graph");
                int64_t opset = 1; // models without opset_import are version 1 (core/model.cpp)
                for (const Value* o : model.all("opset_import"))
                    if (o->kind == Value::MSG && (o->m->get_str("domain").empty() || o->m->get_str("domain") == "ai.onnx"))
                        opset = o->m->get_int("version", 1);

                map<string, Output<Node>> values;
                for (const Value* init : graph.all("initializer"))
                {
                    if (init->kind != Value::MSG)
                        continue;
                    const string name = init->m->get_str("name");
                    auto c = constant_of(*init->m, "initializer '" + name + "'");
                    c->set_friendly_name(name);
                    values[name] = c;
                }
                ParameterVector parameters;
                for (const Value* in : graph.all("input"))
                {
                    if (in->kind != Value::MSG)
                        continue;
                    const string name = in->m->get_str("name");
                    if (values.count(name))
                        continue; // an initializer supplies it
                    const Message* type = in->m->get_msg("type");
                    const Message* tensor = type ? type->get_msg("tensor_type") : nullptr;
                    if (!tensor)
                        throw ngraph_error("ONNX model: graph input '" + name + "' has no tensor type");
                    Shape shape;
                    if (const Message* sh = tensor->get_msg("shape"))
                        for (const Value* d : sh->all("dim"))
                        {
                            if (d->kind != Value::MSG || !d->m->has("dim_value"))
                                throw ngraph_error("ONNX model: graph input '" + name + "' has a symbolic dimension; this importer needs static shapes");
                            NGRAPH_CHECK(d->m->get_int("dim_value") >= 0, "ONNX model: graph input '", name, "' has a negative dimension");
                            shape.push_back(static_cast<size_t>(d->m->get_int("dim_value")));
                        }
                    auto p = make_shared<op::v0::Parameter>(element_type_of(data_type_of(*tensor, "elem_type"), "graph input '" + name + "'"), shape);
                    p->set_friendly_name(name);
                    parameters.push_back(p);
                    values[name] = p;
                }
                for (const Value* nv : graph.all("node"))
                {
                    if (nv->kind != Value::MSG)
                        continue;
                    const Message& nm = *nv->m;
                    OutputVector inputs;
                    for (const Value* in : nm.all("input"))
                    {
                        if (in->s.empty())
                        {
                            inputs.emplace_back(); // an optional input left out
                            continue;
                        }
                        const auto it = values.find(in->s);
                        if (it == values.end())
                            throw ngraph_error("ONNX model: node '" + nm.get_str("name") + "' (" + nm.get_str("op_type") + ") reads '" + in->s + "', which nothing before it produces");
                        inputs.push_back(it->second);
                    }
                    const OnnxNode node(nm, inputs, opset);
                    const OperatorFn* fn = find_operator(nm.get_str("op_type"), opset, nm.get_str("domain"));
                    if (!fn)
                        throw ngraph_error("ONNX model: unsupported operator " + (nm.get_str("domain").empty() ? string() : nm.get_str("domain") + ".") + nm.get_str("op_type") + " (opset " +
                                           to_string(opset) + ")");
                    const OutputVector outs = (*fn)(node);
                    const auto names = nm.all("output");
                    NGRAPH_CHECK(names.size() <= outs.size(), node.description(), ": the node names ", names.size(), " outputs, the operator has ", outs.size());
                    for (size_t i = 0; i < names.size(); ++i)
                    {
                        if (names[i]->s.empty())
                            continue;
                        values[names[i]->s] = outs[i];
                        if (outs[i].get_node() && !outs[i].get_node()->is_parameter() && !outs[i].get_node()->is_constant())
                            outs[i].get_node()->set_friendly_name(names[i]->s);
                    }
                }
                OutputVector results;
                vector<string> result_names;
                for (const Value* out : graph.all("output"))
                {
                    if (out->kind != Value::MSG)
                        continue;
                    const string name = out->m->get_str("name");
                    const auto it = values.find(name);
                    if (it == values.end())
                        throw ngraph_error("ONNX model: graph output '" + name + "' is produced by no node");
                    results.push_back(it->second);
                    result_names.push_back(name);
                }
                NGRAPH_CHECK(!results.empty(), "ONNX model: the graph has no outputs");
                auto f = make_shared<Function>(results, parameters, graph.get_str("name"));
                for (size_t i = 0; i < f->get_output_size(); ++i)
                    f->get_output_op(i)->set_friendly_name(result_names[i]);
                return f;
            }
        }

        set<string> get_supported_operators(int64_t version, const string& domain)
        {
            set<string> out;
            for (const auto& op : operators())
                if (find_operator(op.first, version, domain))
                    out.insert(op.first);
            return out;
        }

        bool is_operator_supported(const string& op_name, int64_t version, const string& domain) { return find_operator(op_name, version, domain) != nullptr; }

        shared_ptr<Function> import_onnx_model(istream& stream)
        {
            stringstream ss;
            ss << stream.rdbuf();
            const string bytes = ss.str();
            return build_function(*read_model(bytes));
        }

        shared_ptr<Function> import_onnx_model(const string& file_path)
        {
            ifstream ifs{file_path, ios::in | ios::binary};
            if (!ifs.is_open())
                throw ngraph_error("Failure opening file: " + file_path);
            return import_onnx_model(ifs);
        }
    }
}
