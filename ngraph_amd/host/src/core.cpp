// Graph vocabulary: element types, nodes, functions, cloning.
#include <atomic>
#include <map>
#include <unordered_map>
#include <unordered_set>

#include "ngraph/ops.hpp"

namespace ngraph
{
    std::ostream& operator<<(std::ostream& os, const Shape& s)
    {
        // the reference prints shapes in validation messages as "{64,3}"
        os << "{";
        for (size_t i = 0; i < s.size(); ++i)
            os << (i ? "," : "") << s[i];
        return os << "}";
    }

    std::ostream& operator<<(std::ostream& os, const AxisSet& s)
    {
        os << "AxisSet{";
        bool first = true;
        for (size_t a : s)
        {
            os << (first ? "" : ", ") << a;
            first = false;
        }
        return os << "}";
    }

    namespace element
    {
        size_t Type::size() const
        {
            switch (m_type)
            {
            case Type_t::boolean:
            case Type_t::i8:
            case Type_t::u8: return 1;
            case Type_t::f32:
            case Type_t::i32: return 4;
            case Type_t::f64:
            case Type_t::i64: return 8;
            default: return 0;
            }
        }

        const std::string& Type::c_type_string() const
        {
            static const std::map<Type_t, std::string> names = {{Type_t::undefined, "undefined"},
                                                                {Type_t::dynamic, "dynamic"},
                                                                {Type_t::boolean, "char"},
                                                                {Type_t::f32, "float"},
                                                                {Type_t::f64, "double"},
                                                                {Type_t::i8, "int8_t"},
                                                                {Type_t::i32, "int32_t"},
                                                                {Type_t::i64, "int64_t"},
                                                                {Type_t::u8, "uint8_t"}};
            return names.at(m_type);
        }

        const std::string& Type::get_type_name() const
        {
            static const std::map<Type_t, std::string> names = {{Type_t::undefined, "undefined"},
                                                                {Type_t::dynamic, "dynamic"},
                                                                {Type_t::boolean, "boolean"},
                                                                {Type_t::f32, "f32"},
                                                                {Type_t::f64, "f64"},
                                                                {Type_t::i8, "i8"},
                                                                {Type_t::i32, "i32"},
                                                                {Type_t::i64, "i64"},
                                                                {Type_t::u8, "u8"}};
            return names.at(m_type);
        }

        std::ostream& operator<<(std::ostream& os, const Type& t) { return os << t.get_type_name(); }
    }

    const element::Type& Output<Node>::get_element_type() const { return m_node->get_output_element_type(m_index); }
    const Shape& Output<Node>::get_shape() const { return m_node->get_output_shape(m_index); }

    Node::~Node() {}

    const std::string& Node::get_name() const
    {
        static std::atomic<size_t> counter{0};
        if (m_name.empty())
            m_name = std::string(get_type_name()) + "_" + std::to_string(counter++);
        return m_name;
    }

    const element::Type& Node::get_element_type() const
    {
        NGRAPH_CHECK(m_outputs.size() == 1, "get_element_type() must be called on a node with exactly one output.");
        return m_outputs[0].get_element_type();
    }

    const Shape& Node::get_shape() const
    {
        NGRAPH_CHECK(m_outputs.size() == 1, "get_shape() must be called on a node with exactly one output (", description(), ")");
        return m_outputs[0].get_shape();
    }

    void Node::set_output_type(size_t i, const element::Type& t, const Shape& s)
    {
        if (m_outputs.size() <= i)
            m_outputs.resize(i + 1);
        m_outputs[i] = descriptor::Tensor(t, s, get_name() + "_" + std::to_string(i));
    }

    void check_new_args_count(const Node* node, const OutputVector& new_args)
    {
        NODE_VALIDATION_CHECK(node,
                              new_args.size() == node->get_input_size(),
                              "copy_with_new_args() expected ",
                              node->get_input_size(),
                              " argument",
                              (node->get_input_size() == 1 ? "" : "s"),
                              " but got ",
                              new_args.size());
    }

    // ------------------------------------------------------------------ Function
    void Function::init(const OutputVector& results)
    {
        for (const auto& r : results)
        {
            auto existing = as_type_ptr<op::v0::Result>(r.get_node_shared_ptr());
            m_results.push_back(existing ? existing : std::make_shared<op::v0::Result>(r));
        }
        // every Parameter reachable from the results must have been declared
        std::unordered_set<Node*> declared;
        for (const auto& p : m_parameters)
            declared.insert(p.get());
        for (const auto& n : get_ordered_ops())
            if (n->is_parameter() && !declared.count(n.get()))
                throw ngraph_error("Function references undeclared parameter '" + n->get_name() + "'");
    }

    Function::Function(const OutputVector& results, const ParameterVector& parameters, const std::string& name)
        : m_parameters(parameters), m_name(name)
    {
        init(results);
    }

    Function::Function(const std::shared_ptr<Node>& result, const ParameterVector& parameters, const std::string& name)
        : m_parameters(parameters), m_name(name)
    {
        init(OutputVector{Output<Node>(result, 0)});
    }

    Function::Function(const NodeVector& results, const ParameterVector& parameters, const std::string& name)
        : m_parameters(parameters), m_name(name)
    {
        OutputVector o;
        for (const auto& n : results)
            o.emplace_back(n, 0);
        init(o);
    }

    Function::Function(const ResultVector& results, const ParameterVector& parameters, const std::string& name)
        : m_parameters(parameters), m_name(name)
    {
        OutputVector o;
        for (const auto& n : results)
            o.emplace_back(std::static_pointer_cast<Node>(n), 0);
        init(o);
    }

    const element::Type& Function::get_output_element_type(size_t i) const { return m_results.at(i)->get_output_element_type(0); }
    const Shape& Function::get_output_shape(size_t i) const { return m_results.at(i)->get_output_shape(0); }
    std::shared_ptr<Node> Function::get_output_op(size_t i) const { return m_results.at(i); }
    std::shared_ptr<Node> Function::get_result() const
    {
        NGRAPH_CHECK(m_results.size() == 1, "get_result() must be called on a function with exactly one result.");
        return m_results[0];
    }

    std::vector<std::shared_ptr<Node>> Function::get_ordered_ops() const
    {
        std::vector<std::shared_ptr<Node>> order;
        std::unordered_set<Node*> done;
        // iterative post-order DFS from the results, then any parameter nothing depends on
        std::vector<std::pair<std::shared_ptr<Node>, size_t>> stack;
        auto visit = [&](const std::shared_ptr<Node>& root) {
            if (done.count(root.get()))
                return;
            stack.emplace_back(root, 0);
            while (!stack.empty())
            {
                auto& top = stack.back();
                if (top.second < top.first->get_input_size())
                {
                    auto arg = top.first->get_argument(top.second++);
                    if (!done.count(arg.get()))
                    {
                        bool on_stack = false;
                        for (const auto& e : stack)
                            on_stack |= (e.first == arg);
                        if (on_stack)
                            throw ngraph_error("cycle in graph");
                        stack.emplace_back(arg, 0);
                    }
                }
                else
                {
                    if (!done.count(top.first.get()))
                    {
                        done.insert(top.first.get());
                        order.push_back(top.first);
                    }
                    stack.pop_back();
                }
            }
        };
        for (const auto& p : m_parameters)
            visit(p);
        for (const auto& r : m_results)
            visit(r);
        return order;
    }

    void Function::replace_node(const std::shared_ptr<Node>& target, const std::shared_ptr<Node>& replacement)
    {
        for (const auto& n : get_ordered_ops())
            for (size_t i = 0; i < n->get_input_size(); ++i)
                if (n->input_value(i).get_node() == target.get())
                    n->set_argument(i, Output<Node>(replacement, n->input_value(i).get_index()));
    }

    std::shared_ptr<Function> clone_function(const Function& f)
    {
        std::unordered_map<Node*, std::shared_ptr<Node>> map;
        for (const auto& n : f.get_ordered_ops())
        {
            OutputVector args;
            for (size_t i = 0; i < n->get_input_size(); ++i)
            {
                const auto& in = n->input_value(i);
                args.emplace_back(map.at(in.get_node()), in.get_index());
            }
            auto c = n->clone_with_new_inputs(args);
            c->set_friendly_name(n->get_friendly_name());
            map[n.get()] = c;
        }
        ParameterVector params;
        for (const auto& p : f.get_parameters())
            params.push_back(std::static_pointer_cast<op::v0::Parameter>(map.at(p.get())));
        ResultVector results;
        for (const auto& r : f.get_results())
            results.push_back(std::static_pointer_cast<op::v0::Result>(map.at(r.get())));
        return std::make_shared<Function>(results, params, f.get_name());
    }
}
