// HIPQuantFusion: see ngraph/runtime/hip/pass/hip_quant_fusion.hpp.  The reference expresses these
// rewrites as pattern-matcher graphs; here each is a direct walk from the root node it would match.
#include <cstring>
#include <map>
#include <vector>

#include "ngraph/builder/make_constant.hpp"
#include "ngraph/ngraph.hpp"
#include "ngraph/runtime/hip/pass/hip_quant_fusion.hpp"

using namespace std;
using namespace ngraph;

namespace
{
    using Users = map<const Node*, vector<Node*>>;

    Users users_of(const Function& f)
    {
        Users u;
        for (const auto& n : f.get_ordered_ops())
            for (size_t i = 0; i < n->get_input_size(); ++i)
                u[n->input_value(i).get_node()].push_back(n.get());
        return u;
    }

    size_t user_count(const Users& u, const Node* n)
    {
        auto it = u.find(n);
        return it == u.end() ? 0 : it->second.size();
    }

    // src/ngraph/graph_util.cpp is_zero: a Constant whose every element is zero
    bool is_zero(const shared_ptr<Node>& n)
    {
        auto c = as_type_ptr<op::v0::Constant>(n);
        if (!c)
            return false;
        const size_t bytes = shape_size(c->get_output_shape(0)) * c->get_output_element_type(0).size();
        const unsigned char* p = static_cast<const unsigned char*>(c->get_data_ptr());
        for (size_t i = 0; i < bytes; ++i)
            if (p[i] != 0)
                return false;
        return true;
    }

    // src/ngraph/graph_util.cpp compare_constants: both Constants, same shape and the same values
    bool same_constants(const shared_ptr<Node>& a, const shared_ptr<Node>& b)
    {
        if (a == b && a->is_constant())
            return true;
        auto ca = as_type_ptr<op::v0::Constant>(a), cb = as_type_ptr<op::v0::Constant>(b);
        if (!ca || !cb || ca->get_output_shape(0) != cb->get_output_shape(0) || ca->get_output_element_type(0) != cb->get_output_element_type(0))
            return false;
        const size_t bytes = shape_size(ca->get_output_shape(0)) * ca->get_output_element_type(0).size();
        return memcmp(ca->get_data_ptr(), cb->get_data_ptr(), bytes) == 0;
    }

    // through any Broadcast, then any Reshape, above `n` (the pattern's Skip nodes)
    shared_ptr<Node> skip_reshape_broadcast(shared_ptr<Node> n)
    {
        while (is_type<op::v0::Broadcast>(n))
            n = n->get_argument(0);
        while (is_type<op::v0::Reshape>(n))
            n = n->get_argument(0);
        return n;
    }

    // every path from `n` to a Result passes through `through` (the in-place summand of a fused
    // add must have no other live reader): here, conservatively, `n`'s users are inside the matched
    // sub-graph, i.e. its only user chain leads to `through`
    bool only_feeds(const Users& u, const Node* n, const Node* through)
    {
        const Node* cur = n;
        while (cur != through)
        {
            auto it = u.find(cur);
            if (it == u.end() || it->second.size() != 1)
                return false;
            cur = it->second[0];
        }
        return true;
    }

    shared_ptr<Node> dequantize_like(const shared_ptr<op::v0::Dequantize>& dq, const shared_ptr<Node>& arg, const shared_ptr<Node>& zp)
    {
        return make_shared<op::v0::Dequantize>(arg, dq->input_value(1), zp, dq->get_output_element_type(0), dq->get_axes());
    }

    // ---- Relu roots ----------------------------------------------------------------------------
    bool fuse_qconv_relu(Function& f, const Users& users, const shared_ptr<Node>& relu)
    {
        auto dq = as_type_ptr<op::v0::Dequantize>(relu->get_argument(0));
        if (!dq || !is_zero(dq->get_argument(2)) || user_count(users, dq->get_argument(0).get()) > 1)
            return false;
        shared_ptr<Node> fused;
        if (auto qcb = as_type_ptr<op::v0::QuantizedConvolutionBias>(dq->get_argument(0)))
        {
            if (qcb->with_relu())
                return false;
            fused = make_shared<op::v0::QuantizedConvolutionBias>(qcb->input_value(0), qcb->input_value(1), qcb->input_value(2), qcb->get_window_movement_strides(),
                                                                  qcb->get_window_dilation_strides(), qcb->get_padding_below(), qcb->get_padding_above(),
                                                                  qcb->get_data_dilation_strides(), qcb->input_value(3), true);
        }
        else if (auto qc = as_type_ptr<op::v0::QuantizedConvolution>(dq->get_argument(0)))
        {
            // the fused op has no zero points and one scale: u8 data, i8 filter and output, all zero points 0
            if (qc->get_input_element_type(0) != element::u8 || qc->get_input_element_type(1) != element::i8 || qc->get_output_element_type(0) != element::i8 ||
                !is_zero(qc->get_argument(3)) || !is_zero(qc->get_argument(5)) || !is_zero(qc->get_argument(7)) || shape_size(qc->get_input_shape(2)) != 1 ||
                shape_size(qc->get_input_shape(4)) != 1 || shape_size(qc->get_input_shape(6)) != 1)
                return false;
            auto requant = (qc->input_value(2) * qc->input_value(4)) / qc->input_value(6);
            fused = make_shared<op::v0::QuantizedConvolutionRelu>(qc->input_value(0), qc->input_value(1), qc->get_window_movement_strides(),
                                                                  qc->get_window_dilation_strides(), qc->get_padding_below(), qc->get_padding_above(),
                                                                  qc->get_data_dilation_strides(), requant);
        }
        else
            return false;
        auto zp = builder::make_constant<uint8_t>(element::u8, dq->get_input_shape(1), 0);
        f.replace_node(relu, dequantize_like(dq, fused, zp));
        return true;
    }

    bool fuse_qconvb_add(Function& f, const Users& users, const shared_ptr<Node>& relu)
    {
        auto add = as_type_ptr<op::v1::Add>(relu->get_argument(0));
        if (!add)
            return false;
        auto dq_l = as_type_ptr<op::v0::Dequantize>(skip_reshape_broadcast(add->get_argument(0)));
        auto dq_r = as_type_ptr<op::v0::Dequantize>(skip_reshape_broadcast(add->get_argument(1)));
        if (!dq_l || !dq_r)
            return false;
        const bool l_conv = is_type<op::v0::QuantizedConvolutionBias>(dq_l->get_argument(0));
        const bool r_conv = is_type<op::v0::QuantizedConvolutionBias>(dq_r->get_argument(0));
        if (!l_conv && !r_conv)
            return false;
        if (!l_conv)
            swap(dq_l, dq_r);
        else if (r_conv)
        {
            // both sides are convolutions: the one whose scale a following Quantize repeats stays the convolution
            auto it = users.find(relu.get());
            if (it != users.end())
                for (Node* user : it->second)
                    if (is_type<op::v0::Quantize>(user))
                    {
                        auto q_scale = user->get_argument(1);
                        if (!same_constants(q_scale, dq_l->get_argument(1)) && same_constants(q_scale, dq_r->get_argument(1)))
                            swap(dq_l, dq_r);
                        break;
                    }
        }
        auto qconv = as_type_ptr<op::v0::QuantizedConvolutionBias>(dq_l->get_argument(0));
        auto summand = dq_r->get_argument(0);
        if (qconv->with_relu() || !is_zero(dq_l->get_argument(2)) || !is_zero(dq_r->get_argument(2)))
            return false;
        if (dq_r->get_input_element_type(0) != element::i8 && dq_r->get_input_element_type(0) != element::u8)
            return false;
        if (user_count(users, qconv.get()) > 1)
            return false;
        if (!only_feeds(users, summand.get(), add.get()) || summand->is_parameter())
            return false;
        if (summand->get_output_shape(0) != qconv->get_output_shape(0))
            return false;
        if (shape_size(dq_l->get_input_shape(1)) != 1 || shape_size(dq_r->get_input_shape(1)) != 1)
            return false;
        auto sum_scale = dq_r->input_value(1) / dq_l->input_value(1);
        shared_ptr<Node> fused;
        if (dq_r->get_input_element_type(0) == element::i8)
            fused = make_shared<op::v0::Convert>(
                make_shared<op::v0::QuantizedConvolutionBiasSignedAdd>(qconv->input_value(0), qconv->input_value(1), qconv->input_value(2), summand,
                                                                       qconv->get_window_movement_strides(), qconv->get_window_dilation_strides(),
                                                                       qconv->get_padding_below(), qconv->get_padding_above(), qconv->get_data_dilation_strides(),
                                                                       qconv->input_value(3), sum_scale, true),
                element::u8);
        else
            fused = make_shared<op::v0::QuantizedConvolutionBiasAdd>(qconv->input_value(0), qconv->input_value(1), qconv->input_value(2), summand,
                                                                     qconv->get_window_movement_strides(), qconv->get_window_dilation_strides(),
                                                                     qconv->get_padding_below(), qconv->get_padding_above(), qconv->get_data_dilation_strides(),
                                                                     qconv->input_value(3), sum_scale, true);
        // the sum was taken after any Reshape / Broadcast of the two sides: only shape-preserving ones
        // can be dropped
        if (relu->get_output_shape(0) != fused->get_output_shape(0))
            return false;
        auto zp = op::v0::Constant::create(element::u8, Shape{}, {0});
        f.replace_node(relu, make_shared<op::v0::Dequantize>(fused, dq_l->input_value(1), zp, element::f32, AxisSet{}));
        return true;
    }

    // ---- pools, concat, Quantize roots -----------------------------------------------------------
    bool hoist_pool(Function& f, const shared_ptr<Node>& pool)
    {
        auto dq = as_type_ptr<op::v0::Dequantize>(pool->get_argument(0));
        // a per-tensor scale commutes with pooling; 8-bit data is what the integer pools take
        if (!dq || !dq->get_axes().empty() || dq->get_input_element_type(0).size() != 1)
            return false;
        shared_ptr<Node> q_pool;
        if (auto mp = as_type_ptr<op::v0::MaxPool>(pool))
            q_pool = make_shared<op::v0::MaxPool>(dq->input_value(0), mp->get_window_shape(), mp->get_window_movement_strides(), mp->get_padding_below(), mp->get_padding_above());
        else
        {
            auto ap = as_type_ptr<op::v0::AvgPool>(pool);
            q_pool = make_shared<op::v0::AvgPool>(dq->input_value(0), ap->get_window_shape(), ap->get_window_movement_strides(), ap->get_padding_below(), ap->get_padding_above(),
                                                  ap->get_include_padding_in_avg_computation());
        }
        f.replace_node(pool, dequantize_like(dq, q_pool, dq->get_argument(2)));
        return true;
    }

    bool hoist_concat(Function& f, const shared_ptr<Node>& concat)
    {
        auto cc = as_type_ptr<op::v0::Concat>(concat);
        if (cc->get_input_size() < 2)
            return false;
        auto dq0 = as_type_ptr<op::v0::Dequantize>(cc->get_argument(0));
        if (!dq0 || !dq0->get_axes().empty())
            return false;
        OutputVector args;
        for (size_t i = 0; i < cc->get_input_size(); ++i)
        {
            auto dq = as_type_ptr<op::v0::Dequantize>(cc->get_argument(i));
            if (!dq || !dq->get_axes().empty() || dq->get_input_element_type(0) != dq0->get_input_element_type(0))
                return false;
            if (!same_constants(dq->get_argument(1), dq0->get_argument(1)) || !same_constants(dq->get_argument(2), dq0->get_argument(2)))
                return false;
            args.push_back(dq->input_value(0));
        }
        auto q_concat = make_shared<op::v0::Concat>(args, cc->get_concatenation_axis());
        f.replace_node(concat, dequantize_like(dq0, q_concat, dq0->get_argument(2)));
        return true;
    }

    bool drop_dq_q(Function& f, const shared_ptr<Node>& q)
    {
        auto dq = as_type_ptr<op::v0::Dequantize>(q->get_argument(0));
        if (!dq || !is_zero(q->get_argument(2)) || !is_zero(dq->get_argument(2)))
            return false;
        if (q->get_output_element_type(0) != dq->get_input_element_type(0))
            return false;
        if (!same_constants(q->get_argument(1), dq->get_argument(1)))
            return false;
        f.replace_node(q, dq->get_argument(0));
        return true;
    }
}

bool runtime::hip::pass::HIPQuantFusion::run_on_function(shared_ptr<Function> f)
{
    bool changed = false;
    for (bool again = true; again;)
    {
        again = false;
        const Users users = users_of(*f);
        for (const auto& n : f->get_ordered_ops())
        {
            bool hit = false;
            if (is_type<op::v0::Relu>(n))
                hit = fuse_qconvb_add(*f, users, n) || fuse_qconv_relu(*f, users, n);
            else if (is_type<op::v0::MaxPool>(n) || is_type<op::v0::AvgPool>(n))
                hit = hoist_pool(*f, n);
            else if (is_type<op::v0::Concat>(n))
                hit = hoist_concat(*f, n);
            else if (is_type<op::v0::Quantize>(n))
                hit = drop_dq_q(*f, n);
            if (hit)
            {
                changed = again = true;
                break; // the node list and the user map are stale
            }
        }
    }
    return changed;
}
