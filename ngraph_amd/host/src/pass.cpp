// Pass manager, NGRAPH_PASS_ENABLES parsing, host-side constant folding of the scale sub-graphs.
#include <cmath>
#include <cstdlib>

#include "ngraph/pass.hpp"

using namespace std;

namespace ngraph
{
    namespace pass
    {
        static void parse_flags(const char* env, char sep, map<string, bool>& out)
        {
            if (!env)
                return;
            string s(env);
            size_t pos = 0;
            while (pos <= s.size())
            {
                size_t end = s.find(';', pos);
                if (end == string::npos)
                    end = s.size();
                string item = s.substr(pos, end - pos);
                size_t c = item.find(sep);
                if (!item.empty())
                {
                    if (c == string::npos)
                        out[item] = true;
                    else
                        out[item.substr(0, c)] = atoi(item.substr(c + 1).c_str()) != 0;
                }
                pos = end + 1;
            }
        }

        PassConfig::PassConfig()
        {
            parse_flags(getenv("NGRAPH_PASS_ENABLES"), ':', m_pass_enables);
            parse_flags(getenv("NGRAPH_PASS_ATTRIBUTES"), '=', m_pass_attributes);
        }

        bool PassConfig::get_pass_enable(const string& name) const
        {
            auto it = m_pass_enables.find(name);
            return it != m_pass_enables.end() && it->second;
        }

        bool PassConfig::get_pass_attribute(const string& name) const
        {
            auto it = m_pass_attributes.find(name);
            return it != m_pass_attributes.end() && it->second;
        }

        void Manager::run_passes(shared_ptr<Function> f)
        {
            for (auto& p : m_passes)
                p->run_on_function(f);
        }

        // ---- constant folding ----------------------------------------------------------------
        template <typename T>
        static T fold_binary(const NodeTypeInfo& ti, T a, T b)
        {
            if (ti == op::v1::Add::type_info)
                return a + b;
            if (ti == op::v1::Subtract::type_info)
                return a - b;
            if (ti == op::v1::Multiply::type_info)
                return a * b;
            if (ti == op::v1::Divide::type_info)
                return a / b;
            if (ti == op::v1::Maximum::type_info)
                return a > b ? a : b;
            return a < b ? a : b;
        }

        template <typename T>
        static shared_ptr<Node> fold_binary_node(const Node& n, const op::v0::Constant& a, const op::v0::Constant& b)
        {
            const size_t count = shape_size(n.get_output_shape(0));
            const size_t an = shape_size(a.get_output_shape(0)), bn = shape_size(b.get_output_shape(0));
            vector<T> out(count);
            const T* pa = a.get_data_ptr<T>();
            const T* pb = b.get_data_ptr<T>();
            for (size_t i = 0; i < count; ++i)
                out[i] = fold_binary<T>(n.get_type_info(), pa[an == 1 ? 0 : i], pb[bn == 1 ? 0 : i]);
            return make_shared<op::v0::Constant>(n.get_output_element_type(0), n.get_output_shape(0), out.data());
        }

        static bool is_binary(const Node& n)
        {
            const auto& ti = n.get_type_info();
            return ti == op::v1::Add::type_info || ti == op::v1::Subtract::type_info || ti == op::v1::Multiply::type_info ||
                   ti == op::v1::Divide::type_info || ti == op::v1::Maximum::type_info || ti == op::v1::Minimum::type_info;
        }

        static shared_ptr<Node> fold(const shared_ptr<Node>& n)
        {
            vector<shared_ptr<op::v0::Constant>> args;
            for (size_t i = 0; i < n->get_input_size(); ++i)
            {
                auto c = as_type_ptr<op::v0::Constant>(n->get_argument(i));
                if (!c)
                    return nullptr;
                args.push_back(c);
            }
            if (args.empty())
                return nullptr;
            const auto et = n->get_output_element_type(0);
            const Shape& shape = n->get_output_shape(0);
            if (is_binary(*n))
            {
                // f32 in f32 arithmetic, exactly as the device kernels (and the reference) do it
                if (et == element::f32)
                    return fold_binary_node<float>(*n, *args[0], *args[1]);
                if (et == element::f64)
                    return fold_binary_node<double>(*n, *args[0], *args[1]);
                return nullptr;
            }
            if (is_type<op::v0::Abs>(n) || is_type<op::v0::Relu>(n))
            {
                if (et != element::f32)
                    return nullptr;
                vector<float> v = args[0]->get_vector<float>();
                for (auto& x : v)
                    x = is_type<op::v0::Abs>(n) ? (x < 0 ? -x : x) : (x > 0 ? x : 0);
                return make_shared<op::v0::Constant>(et, shape, v.data());
            }
            if (is_type<op::v0::Broadcast>(n))
            {
                if (shape_size(args[0]->get_output_shape(0)) != 1)
                    return nullptr;
                const size_t eb = et.size();
                vector<uint8_t> bytes(shape_size(shape) * eb);
                for (size_t i = 0; i < shape_size(shape); ++i)
                    memcpy(bytes.data() + i * eb, args[0]->get_data_ptr(), eb);
                return make_shared<op::v0::Constant>(et, shape, bytes.data());
            }
            if (is_type<op::v0::Convert>(n))
            {
                // static_cast between the value as stored and the target type
                return make_shared<op::v0::Constant>(et, shape, args[0]->get_values_as_double());
            }
            return nullptr;
        }

        bool ConstantFolding::run_on_function(shared_ptr<Function> f)
        {
            bool changed = false;
            for (const auto& n : f->get_ordered_ops())
            {
                if (n->is_constant() || n->is_parameter() || n->is_output())
                    continue;
                auto c = fold(n);
                if (c)
                {
                    f->replace_node(n, c);
                    changed = true;
                }
            }
            return changed;
        }
    }
}
