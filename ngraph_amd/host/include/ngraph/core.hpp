// Host-side graph vocabulary for the int8 path: a small, source-compatible subset of the nGraph
// core API (same namespaces, class names and signatures for what the quantized-inference graphs and
// their tests touch).  Written from scratch; static shapes only.
//
// Mirrors (nGraph tree): src/ngraph/{shape,strides,coordinate_diff,axis_set,axis_vector}.hpp,
// src/ngraph/type/element_type.hpp:40-160, src/ngraph/node.hpp, src/ngraph/function.hpp:34-144,
// src/ngraph/except.hpp, src/ngraph/check.hpp.
#pragma once

#include <cstddef>
#include <cstdint>
#include <functional>
#include <memory>
#include <set>
#include <sstream>
#include <stdexcept>
#include <string>
#include <type_traits>
#include <vector>

#define NGRAPH_API __attribute__((visibility("default")))

namespace ngraph
{
    // ------------------------------------------------------------------ errors
    class NGRAPH_API ngraph_error : public std::runtime_error
    {
    public:
        explicit ngraph_error(const std::string& what) : std::runtime_error(what) {}
    };

    class NGRAPH_API unsupported_op : public std::runtime_error
    {
    public:
        explicit unsupported_op(const std::string& what) : std::runtime_error(what) {}
    };

    class NGRAPH_API CheckFailure : public ngraph_error
    {
    public:
        explicit CheckFailure(const std::string& what) : ngraph_error(what) {}
    };

    class NGRAPH_API NodeValidationFailure : public CheckFailure
    {
    public:
        explicit NodeValidationFailure(const std::string& what) : CheckFailure(what) {}
    };

    namespace detail
    {
        inline void stream_all(std::ostream&) {}
        template <typename T, typename... R>
        void stream_all(std::ostream& os, const T& v, const R&... rest)
        {
            os << v;
            stream_all(os, rest...);
        }
    }

#define NGRAPH_CHECK(cond, ...)                                                                    \
    do                                                                                             \
    {                                                                                              \
        if (!(cond))                                                                               \
        {                                                                                          \
            std::ostringstream ss_;                                                                \
            ss_ << "Check '" #cond "' failed: ";                                                   \
            ::ngraph::detail::stream_all(ss_, ##__VA_ARGS__);                                      \
            throw ::ngraph::CheckFailure(ss_.str());                                               \
        }                                                                                          \
    } while (0)

#define NODE_VALIDATION_CHECK(node, cond, ...)                                                     \
    do                                                                                             \
    {                                                                                              \
        if (!(cond))                                                                               \
        {                                                                                          \
            std::ostringstream ss_;                                                                \
            ss_ << "While validating node '" << (node)->get_name() << "': ";                       \
            ::ngraph::detail::stream_all(ss_, ##__VA_ARGS__);                                      \
            throw ::ngraph::NodeValidationFailure(ss_.str());                                      \
        }                                                                                          \
    } while (0)

    // ------------------------------------------------------------------ value types
    class NGRAPH_API Shape : public std::vector<size_t>
    {
    public:
        using std::vector<size_t>::vector;
        Shape() = default;
        Shape(const std::vector<size_t>& v) : std::vector<size_t>(v) {}
    };
    class NGRAPH_API Strides : public std::vector<size_t>
    {
    public:
        using std::vector<size_t>::vector;
        Strides() = default;
        Strides(const std::vector<size_t>& v) : std::vector<size_t>(v) {}
    };
    class NGRAPH_API Coordinate : public std::vector<size_t>
    {
    public:
        using std::vector<size_t>::vector;
    };
    class NGRAPH_API CoordinateDiff : public std::vector<std::ptrdiff_t>
    {
    public:
        using std::vector<std::ptrdiff_t>::vector;
        CoordinateDiff() = default;
    };
    class NGRAPH_API AxisVector : public std::vector<size_t>
    {
    public:
        using std::vector<size_t>::vector;
    };
    class NGRAPH_API AxisSet : public std::set<size_t>
    {
    public:
        using std::set<size_t>::set;
        AxisSet() = default;
    };
    using PartialShape = Shape; // static shapes only

    inline size_t shape_size(const Shape& s)
    {
        size_t n = 1;
        for (size_t d : s)
            n *= d;
        return n;
    }
    NGRAPH_API std::ostream& operator<<(std::ostream& os, const Shape& s);
    NGRAPH_API std::ostream& operator<<(std::ostream& os, const AxisSet& s);

    // ------------------------------------------------------------------ element types
    namespace element
    {
        enum class Type_t
        {
            undefined,
            dynamic,
            boolean,
            f32,
            f64,
            i8,
            i32,
            i64,
            u8
        };

        class NGRAPH_API Type
        {
        public:
            Type() : m_type(Type_t::undefined) {}
            constexpr Type(Type_t t) : m_type(t) {}
            size_t size() const;
            size_t bitwidth() const { return size() * 8; }
            bool is_static() const { return m_type != Type_t::dynamic && m_type != Type_t::undefined; }
            bool is_dynamic() const { return m_type == Type_t::dynamic; }
            bool is_real() const { return m_type == Type_t::f32 || m_type == Type_t::f64; }
            bool is_integral() const { return is_static() && !is_real(); }
            bool is_signed() const { return m_type != Type_t::u8 && m_type != Type_t::boolean; }
            // src/ngraph/type/element_type.cpp:83-88
            bool is_quantized() const { return m_type == Type_t::i8 || m_type == Type_t::u8 || m_type == Type_t::i32; }
            bool compatible(const Type& o) const { return is_dynamic() || o.is_dynamic() || m_type == o.m_type; }
            const std::string& c_type_string() const;
            const std::string& get_type_name() const;
            Type_t get_type_enum() const { return m_type; }
            bool operator==(const Type& o) const { return m_type == o.m_type; }
            bool operator!=(const Type& o) const { return m_type != o.m_type; }
            bool operator<(const Type& o) const { return m_type < o.m_type; }
            operator Type_t() const { return m_type; }

        private:
            Type_t m_type;
        };

        constexpr Type dynamic(Type_t::dynamic);
        constexpr Type boolean(Type_t::boolean);
        constexpr Type f32(Type_t::f32);
        constexpr Type f64(Type_t::f64);
        constexpr Type i8(Type_t::i8);
        constexpr Type i32(Type_t::i32);
        constexpr Type i64(Type_t::i64);
        constexpr Type u8(Type_t::u8);

        template <typename T>
        Type from();
        template <>
        inline Type from<char>()
        {
            return boolean;
        }
        template <>
        inline Type from<bool>()
        {
            return boolean;
        }
        template <>
        inline Type from<float>()
        {
            return f32;
        }
        template <>
        inline Type from<double>()
        {
            return f64;
        }
        template <>
        inline Type from<int8_t>()
        {
            return i8;
        }
        template <>
        inline Type from<int32_t>()
        {
            return i32;
        }
        template <>
        inline Type from<int64_t>()
        {
            return i64;
        }
        template <>
        inline Type from<uint8_t>()
        {
            return u8;
        }

        NGRAPH_API std::ostream& operator<<(std::ostream& os, const Type& t);
    }

    // ------------------------------------------------------------------ graph
    class Node;
    class Function;

    struct NGRAPH_API NodeTypeInfo
    {
        const char* name;
        uint64_t version;
        bool operator==(const NodeTypeInfo& o) const { return version == o.version && std::string(name) == o.name; }
        bool operator!=(const NodeTypeInfo& o) const { return !(*this == o); }
    };

    namespace descriptor
    {
        // type + shape of one node output
        class NGRAPH_API Tensor
        {
        public:
            Tensor() = default;
            Tensor(const element::Type& t, const Shape& s, const std::string& name = "")
                : m_type(t), m_shape(s), m_name(name)
            {
            }
            const element::Type& get_element_type() const { return m_type; }
            const Shape& get_shape() const { return m_shape; }
            const PartialShape& get_partial_shape() const { return m_shape; }
            const std::string& get_name() const { return m_name; }
            size_t size() const { return shape_size(m_shape) * m_type.size(); }

        private:
            element::Type m_type;
            Shape m_shape;
            std::string m_name;
        };
    }

    template <typename T>
    class Output;

    template <>
    class NGRAPH_API Output<Node>
    {
    public:
        Output() = default;
        Output(const std::shared_ptr<Node>& node, size_t index) : m_node(node), m_index(index) {}
        template <typename T, typename = typename std::enable_if<std::is_base_of<Node, T>::value>::type>
        Output(const std::shared_ptr<T>& node) : m_node(node), m_index(0)
        {
        }
        Node* get_node() const { return m_node.get(); }
        std::shared_ptr<Node> get_node_shared_ptr() const { return m_node; }
        size_t get_index() const { return m_index; }
        const element::Type& get_element_type() const;
        const Shape& get_shape() const;
        const PartialShape& get_partial_shape() const { return get_shape(); }
        bool operator==(const Output& o) const { return m_node == o.m_node && m_index == o.m_index; }
        bool operator!=(const Output& o) const { return !(*this == o); }
        bool operator<(const Output& o) const { return m_node < o.m_node || (m_node == o.m_node && m_index < o.m_index); }

    private:
        std::shared_ptr<Node> m_node;
        size_t m_index = 0;
    };

    using OutputVector = std::vector<Output<Node>>;
    using NodeVector = std::vector<std::shared_ptr<Node>>;

    class NGRAPH_API Node : public std::enable_shared_from_this<Node>
    {
    public:
        virtual ~Node();
        virtual const NodeTypeInfo& get_type_info() const = 0;
        const char* get_type_name() const { return get_type_info().name; }
        virtual std::string description() const { return get_type_name(); }
        const std::string& get_name() const;
        void set_friendly_name(const std::string& n) { m_friendly_name = n; }
        const std::string& get_friendly_name() const { return m_friendly_name.empty() ? get_name() : m_friendly_name; }

        size_t get_input_size() const { return m_inputs.size(); }
        const Output<Node>& input_value(size_t i) const { return m_inputs.at(i); }
        OutputVector input_values() const { return m_inputs; }
        const element::Type& get_input_element_type(size_t i) const { return m_inputs.at(i).get_element_type(); }
        const Shape& get_input_shape(size_t i) const { return m_inputs.at(i).get_shape(); }
        const PartialShape& get_input_partial_shape(size_t i) const { return get_input_shape(i); }
        std::shared_ptr<Node> get_argument(size_t i) const { return m_inputs.at(i).get_node_shared_ptr(); }

        size_t get_output_size() const { return m_outputs.size(); }
        const element::Type& get_output_element_type(size_t i) const { return m_outputs.at(i).get_element_type(); }
        const Shape& get_output_shape(size_t i) const { return m_outputs.at(i).get_shape(); }
        const PartialShape& get_output_partial_shape(size_t i) const { return get_output_shape(i); }
        const element::Type& get_element_type() const;
        const Shape& get_shape() const;
        const descriptor::Tensor& get_output_tensor(size_t i) const { return m_outputs.at(i); }
        Output<Node> output(size_t i) { return Output<Node>(shared_from_this(), i); }

        virtual void validate_and_infer_types() {}
        virtual std::shared_ptr<Node> clone_with_new_inputs(const OutputVector& new_args) const = 0;
        std::shared_ptr<Node> copy_with_new_inputs(const OutputVector& new_args) const { return clone_with_new_inputs(new_args); }

        virtual bool is_parameter() const { return false; }
        virtual bool is_constant() const { return false; }
        virtual bool is_output() const { return false; }

        // provenance is bookkeeping the hot path does not use
        std::shared_ptr<Node> add_provenance_group_members_above(const OutputVector&) { return shared_from_this(); }

        // replaces input i (used by the rewriting passes)
        void set_argument(size_t i, const Output<Node>& v) { m_inputs.at(i) = v; }

    protected:
        Node() = default;
        explicit Node(const OutputVector& args) : m_inputs(args) {}
        void set_arguments(const OutputVector& args) { m_inputs = args; }
        void set_output_size(size_t n) { m_outputs.resize(n); }
        void set_output_type(size_t i, const element::Type& t, const Shape& s);
        void constructor_validate_and_infer_types() { validate_and_infer_types(); }

    private:
        OutputVector m_inputs;
        std::vector<descriptor::Tensor> m_outputs;
        mutable std::string m_name;
        std::string m_friendly_name;
    };

    NGRAPH_API void check_new_args_count(const Node* node, const OutputVector& new_args);

    template <typename T>
    bool is_type(const Node* n)
    {
        return n && n->get_type_info() == T::type_info;
    }
    template <typename T>
    bool is_type(const std::shared_ptr<Node>& n)
    {
        return is_type<T>(n.get());
    }
    template <typename T>
    std::shared_ptr<T> as_type_ptr(const std::shared_ptr<Node>& n)
    {
        return is_type<T>(n) ? std::static_pointer_cast<T>(n) : std::shared_ptr<T>();
    }
    // src/ngraph/type.hpp:80-90: casts a Value* to a Type* if it is of that type, nullptr otherwise
    // (Type carries the constness: as_type<const op::v0::Quantize>(const Node*))
    template <typename Type, typename Value>
    Type* as_type(Value value)
    {
        return is_type<typename std::remove_const<Type>::type>(value) ? static_cast<Type*>(value) : nullptr;
    }

    namespace op
    {
        class NGRAPH_API Op : public Node
        {
        protected:
            Op() = default;
            explicit Op(const OutputVector& args) : Node(args) {}
        };
        namespace v0
        {
            class Parameter;
            class Result;
        }
    }

    using ParameterVector = std::vector<std::shared_ptr<op::v0::Parameter>>;
    using ResultVector = std::vector<std::shared_ptr<op::v0::Result>>;

    class NGRAPH_API Function
    {
    public:
        Function(const OutputVector& results, const ParameterVector& parameters, const std::string& name = "");
        Function(const std::shared_ptr<Node>& result, const ParameterVector& parameters, const std::string& name = "");
        Function(const NodeVector& results, const ParameterVector& parameters, const std::string& name = "");
        Function(const ResultVector& results, const ParameterVector& parameters, const std::string& name = "");

        const ParameterVector& get_parameters() const { return m_parameters; }
        const ResultVector& get_results() const { return m_results; }
        size_t get_output_size() const { return m_results.size(); }
        const element::Type& get_output_element_type(size_t i) const;
        const Shape& get_output_shape(size_t i) const;
        std::shared_ptr<Node> get_output_op(size_t i) const;
        std::shared_ptr<Node> get_result() const;
        const std::string& get_name() const { return m_name; }
        // topological order, every node a Result depends on (src/ngraph/function.cpp get_ordered_ops)
        std::vector<std::shared_ptr<Node>> get_ordered_ops() const;
        std::vector<std::shared_ptr<Node>> get_ops() const { return get_ordered_ops(); }
        // replaces `target` by `replacement` (output 0) everywhere it feeds a node of this function
        void replace_node(const std::shared_ptr<Node>& target, const std::shared_ptr<Node>& replacement);

    private:
        void init(const OutputVector& results);
        ResultVector m_results;
        ParameterVector m_parameters;
        std::string m_name;
    };

    // deep copy of the graph (src/ngraph/graph_util.hpp clone_function)
    NGRAPH_API std::shared_ptr<Function> clone_function(const Function& f);
}
