// The "HIP" nGraph backend: runtime::Backend / Executable / Tensor over the C ABI of libhipq.so.
//
// This file never includes a HIP header; the GPU is reached only through include/hipq.h.
// Structure follows the reference's minimal plugins (src/runtime/nop/nop_backend.cpp:36-81 for the
// registration seam, src/ngraph/runtime/interpreter/int_executable.cpp:63-278 for compile / call):
// compile() clones the function, folds the constant scale sub-graphs, and lowers the ordered ops to
// a flat list of launches over device buffers; call() binds parameter / result tensors and replays
// the list on one stream.
#include <cstring>
#include <functional>
#include <map>
#include <mutex>
#include <unordered_map>
#include <unordered_set>

#include "hipq.h"
#include "ngraph/ngraph.hpp"
#include "ngraph/pass/constant_folding.hpp"
#include "ngraph/pass/manager.hpp"
#include "ngraph/pass/pass_config.hpp"
#include "ngraph/runtime/backend_manager.hpp"
#include "ngraph/runtime/executable.hpp"
#include "ngraph/runtime/hip/pass/hip_quant_fusion.hpp"
#include "ngraph/runtime/performance_counter.hpp"
#include "ngraph/runtime/tensor.hpp"

using namespace std;
using namespace ngraph;

#define HIP_BACKEND_API __attribute__((visibility("default")))

namespace
{
    void check(int rc, const char* what)
    {
        if (rc != HIPQ_OK)
        {
            string msg = string(what) + ": " + hipq_last_error();
            if (rc == HIPQ_ERR_UNSUPPORTED)
                throw unsupported_op(msg);
            throw ngraph_error(msg);
        }
    }

    int dtype_of(const element::Type& t)
    {
        switch (t.get_type_enum())
        {
        case element::Type_t::u8:
        case element::Type_t::boolean: return HIPQ_U8;
        case element::Type_t::i8: return HIPQ_I8;
        case element::Type_t::i32: return HIPQ_I32;
        case element::Type_t::f32: return HIPQ_F32;
        case element::Type_t::f64: return HIPQ_F64;
        default: throw unsupported_op("HIP backend: unsupported element type " + t.get_type_name());
        }
    }

    // ------------------------------------------------------------------ tensor
    class HIPTensor : public runtime::Tensor
    {
    public:
        HIPTensor(const element::Type& et, const Shape& shape, void* device_memory = nullptr)
            : runtime::Tensor(make_shared<descriptor::Tensor>(et, shape, "external")), m_ptr(device_memory), m_owned(device_memory == nullptr)
        {
            if (m_owned)
                check(hipq_malloc(&m_ptr, get_size_in_bytes()), "HIPTensor allocation");
        }
        ~HIPTensor() override
        {
            if (m_owned)
                hipq_free(m_ptr);
        }
        void write(const void* p, size_t n) override
        {
            if (n != get_size_in_bytes())
                throw out_of_range("partial tensor write not supported");
            if (n && !p)
                throw runtime_error("HIPTensor::write: null source");
            check(hipq_memcpy_h2d(m_ptr, p, n, nullptr), "HIPTensor::write");
        }
        void read(void* p, size_t n) const override
        {
            if (n != get_size_in_bytes())
                throw out_of_range("partial tensor read access not supported");
            if (n && !p)
                throw runtime_error("HIPTensor::read: null destination");
            check(hipq_memcpy_d2h(p, m_ptr, n, nullptr), "HIPTensor::read");
        }
        void copy_from(const runtime::Tensor& source) override
        {
            auto src = dynamic_cast<const HIPTensor*>(&source);
            if (!src)
                return runtime::Tensor::copy_from(source);
            if (get_element_count() != source.get_element_count())
                throw invalid_argument("runtime::Tensor::copy_from: element count does not match");
            if (get_element_type() != source.get_element_type())
                throw invalid_argument("runtime::Tensor::copy_from: element types do not match");
            check(hipq_memcpy_d2d(m_ptr, src->m_ptr, get_size_in_bytes(), nullptr), "HIPTensor::copy_from");
            check(hipq_stream_sync(nullptr), "HIPTensor::copy_from");
        }
        void* device_ptr() const { return m_ptr; }

    private:
        void* m_ptr;
        bool m_owned;
    };

    // device allocation released with the executable
    struct DeviceBlock
    {
        void* ptr = nullptr;
        explicit DeviceBlock(size_t bytes) { check(hipq_malloc(&ptr, bytes), "device allocation"); }
        ~DeviceBlock() { hipq_free(ptr); }
        DeviceBlock(const DeviceBlock&) = delete;
        DeviceBlock& operator=(const DeviceBlock&) = delete;
    };

    // ------------------------------------------------------------------ executable
    struct Step
    {
        shared_ptr<Node> node;
        vector<int> inputs; // value ids
        int output = -1;    // value id
        // launch(input pointers, output pointer, stream)
        function<void(const vector<void*>&, void*, void*)> launch;
    };

    class HIPExecutable : public runtime::Executable
    {
    public:
        HIPExecutable(const shared_ptr<Function>& func, int device, bool enable_performance_data);
        ~HIPExecutable() override;
        bool call(const vector<shared_ptr<runtime::Tensor>>& outputs, const vector<shared_ptr<runtime::Tensor>>& inputs) override;
        vector<runtime::PerformanceCounter> get_performance_data() const override;
        shared_ptr<runtime::Tensor> create_input_tensor(size_t i) override
        {
            return make_shared<HIPTensor>(m_parameters.at(i)->get_output_element_type(0), m_parameters.at(i)->get_output_shape(0));
        }
        shared_ptr<runtime::Tensor> create_output_tensor(size_t i) override
        {
            return make_shared<HIPTensor>(m_results.at(i)->get_output_element_type(0), m_results.at(i)->get_output_shape(0));
        }
        shared_ptr<runtime::Tensor> create_input_tensor(size_t i, void* p) override
        {
            return make_shared<HIPTensor>(m_parameters.at(i)->get_output_element_type(0), m_parameters.at(i)->get_output_shape(0), p);
        }
        shared_ptr<runtime::Tensor> create_output_tensor(size_t i, void* p) override
        {
            return make_shared<HIPTensor>(m_results.at(i)->get_output_element_type(0), m_results.at(i)->get_output_shape(0), p);
        }

    private:
        // the outputs of a node have consecutive value ids
        int value_of(const Output<Node>& o) const { return m_value_of.at(o.get_node()) + static_cast<int>(o.get_index()); }
        void* constant_ptr(const Output<Node>& o) const;
        void lower(const shared_ptr<Node>& n);
        void lower_conv(const shared_ptr<Node>& n, Step& st);
        void lower_dot(const shared_ptr<Node>& n, Step& st, const hipq_quant_out_t* gelu_quantize = nullptr, int gelu_quantize_at = -1);
        void lower_pool(const shared_ptr<Node>& n, Step& st);
        // the library call a convolution node stands for: descriptors and the positions of its inputs
        struct ConvCall
        {
            hipq_conv_desc_t d;
            hipq_fused_desc_t f;
            int bias_i = -1, sum_i = -1, scale_i = -1, sum_scale_i = -1;
            bool plain = false;
        };
        ConvCall conv_call(const shared_ptr<Node>& n) const;
        hipq_pool_desc_t pool_desc(const shared_ptr<Node>& n) const;
        shared_ptr<DeviceBlock> packed_filter(const shared_ptr<Node>& n, const ConvCall& c);
        void assign_layouts();
        void plan_glue_fusion();
        bool nxc(const Node* n) const { return m_nxc.count(n) != 0; }
        shared_ptr<DeviceBlock> alloc(size_t bytes)
        {
            auto b = make_shared<DeviceBlock>(bytes ? bytes : 1);
            m_blocks.push_back(b);
            return b;
        }

        int m_device;
        bool m_perf;
        shared_ptr<Function> m_function;
        unordered_map<const Node*, int> m_value_of; // node -> value id of its output 0
        unordered_map<const Node*, bool> m_nxc;     // nodes whose output tensor is kept channels-last
        // f32 glue folded into its neighbours (plan_glue_fusion): nodes that get no launch of their own ...
        unordered_set<const Node*> m_folded;
        // ... a Softmax that multiplies its input by a constant first, a LayerNorm that adds two tensors
        // first, and a LayerNorm / Gelu that also writes the Quantize of its result
        struct ScaledInput
        {
            Output<Node> x;
            float factor;
        };
        unordered_map<const Node*, ScaledInput> m_softmax_of_product;
        // ... a BatchMatMul that stands for the attention of a batch of heads:
        // BatchMatMul(Softmax(Multiply(BatchMatMulTranspose(q, k), factor)), v), one launch
        struct Attention
        {
            Output<Node> q, k, v;
            bool scaled;
            float factor;
        };
        unordered_map<const Node*, Attention> m_attention;
        unordered_map<const Node*, pair<Output<Node>, Output<Node>>> m_layer_norm_of_sum;
        // ... a MaxPool that also runs the convolution in front of it (a network's first two layers):
        // one launch, the convolution's own output is never written
        unordered_map<const Node*, shared_ptr<Node>> m_pool_of_conv;
        struct QuantizedCopy
        {
            shared_ptr<Node> quantize;
            float scale;
            int32_t zero_point;
            bool only_user; // the f32 result has no other reader
            bool through_gelu = false; // keyed by a QuantizedDotBias: a folded Gelu stands between it and the Quantize
        };
        unordered_map<const Node*, QuantizedCopy> m_quantized_copy;
        vector<void*> m_value_ptr;                  // persistent device pointer, or null when bound per call
        vector<size_t> m_value_bytes;
        vector<int> m_value_uses;
        vector<bool> m_value_external; // a Parameter's or Constant's memory: never redirected into a caller's output tensor
        vector<int> m_param_value, m_result_value;
        vector<Step> m_steps;
        vector<shared_ptr<DeviceBlock>> m_blocks;
        void* m_stream = nullptr;
        mutex m_mutex;
        // HIP graph of the call's launch sequence: captured on the second call with a given set of
        // tensor addresses, replayed while the addresses (and the library's workspace) stay the same
        bool m_use_graph = true;
        void* m_graph = nullptr;
        vector<void*> m_graph_key, m_last_key;
        uint64_t m_graph_epoch = 0;
        // performance data
        vector<void*> m_events;
        vector<double> m_step_us;
        size_t m_calls = 0;
    };

    void* HIPExecutable::constant_ptr(const Output<Node>& o) const { return m_value_ptr.at(value_of(o)); }

    bool constant_is_zero(const Output<Node>& o)
    {
        auto c = as_type_ptr<op::v0::Constant>(o.get_node_shared_ptr());
        if (!c)
            return false;
        // zero in every element type of a zero point (u8, i8, i32) is all bytes zero
        const auto* bytes = static_cast<const unsigned char*>(c->get_data_ptr());
        const size_t count = shape_size(c->get_output_shape(0)) * c->get_output_element_type(0).size();
        for (size_t i = 0; i < count; ++i)
            if (bytes[i] != 0)
                return false;
        return true;
    }

    // the five attributes every quantized convolution op carries, read through the getters each op
    // class has of its own (src/ngraph/op/quantized_convolution.hpp:72-80,
    // src/ngraph/op/experimental/quantized_conv_bias.hpp, quantized_conv_relu.hpp)
    struct ConvAttrs
    {
        Strides window_movement_strides, window_dilation_strides, data_dilation_strides;
        CoordinateDiff padding_below, padding_above;
        const Strides& get_window_movement_strides() const { return window_movement_strides; }
        const Strides& get_window_dilation_strides() const { return window_dilation_strides; }
        const Strides& get_data_dilation_strides() const { return data_dilation_strides; }
        const CoordinateDiff& get_padding_below() const { return padding_below; }
        const CoordinateDiff& get_padding_above() const { return padding_above; }
    };
    template <typename OP>
    ConvAttrs conv_attrs(const OP& op)
    {
        return ConvAttrs{op.get_window_movement_strides(), op.get_window_dilation_strides(), op.get_data_dilation_strides(), op.get_padding_below(), op.get_padding_above()};
    }

    void fill_conv_desc(hipq_conv_desc_t& d, const Node& n, const ConvAttrs& a)
    {
        memset(&d, 0, sizeof(d));
        const Shape& ds = n.get_input_shape(0);
        const Shape& fs = n.get_input_shape(1);
        const Shape& os = n.get_output_shape(0);
        const size_t ns = ds.size() - 2;
        if (ns < 1 || ns > HIPQ_MAX_SPATIAL)
            throw unsupported_op("HIP backend: convolution with " + to_string(ns) + " spatial dimensions");
        d.n_spatial = static_cast<int32_t>(ns);
        d.data_t = dtype_of(n.get_input_element_type(0));
        d.filter_t = dtype_of(n.get_input_element_type(1));
        d.out_t = dtype_of(n.get_output_element_type(0));
        d.data_layout = HIPQ_LAYOUT_NCX;
        d.out_layout = HIPQ_LAYOUT_NCX;
        d.N = static_cast<int64_t>(ds[0]);
        d.C = static_cast<int64_t>(ds[1]);
        d.K = static_cast<int64_t>(fs[0]);
        for (size_t i = 0; i < HIPQ_MAX_SPATIAL; ++i)
        {
            d.in_sp[i] = d.f_sp[i] = d.out_sp[i] = d.stride[i] = d.dilation[i] = d.data_dilation[i] = 1;
            d.pad_below[i] = d.pad_above[i] = 0;
        }
        for (size_t i = 0; i < ns; ++i)
        {
            d.in_sp[i] = static_cast<int64_t>(ds[2 + i]);
            d.f_sp[i] = static_cast<int64_t>(fs[2 + i]);
            d.out_sp[i] = static_cast<int64_t>(os[2 + i]);
            d.stride[i] = static_cast<int64_t>(a.get_window_movement_strides()[i]);
            d.dilation[i] = static_cast<int64_t>(a.get_window_dilation_strides()[i]);
            d.data_dilation[i] = static_cast<int64_t>(a.get_data_dilation_strides()[i]);
            d.pad_below[i] = a.get_padding_below()[i];
            d.pad_above[i] = a.get_padding_above()[i];
        }
    }


    // ------------------------------------------------------------------ HIPLayout
    // Keeps the interior of a quantized network channels-last, the layout the convolution kernels
    // read and write without a transposition -- the job CPULayout does for the reference's CPU
    // backend with its blocked formats (src/ngraph/runtime/cpu/pass/cpu_layout.cpp:80-160), minus
    // the inserted ConvertLayout nodes: a convolution converts on the way in or out for free, so
    // tensors only ever change layout inside one.  Tensors joined by layout-agnostic ops (Relu,
    // Convert, elementwise binaries, per-tensor Quantize / Dequantize, pools, Concat) form a class
    // that shares a layout; a class becomes channels-last unless some member is produced or read by
    // an op that only knows nGraph's [N, C, spatial...] (Parameters, Results, Reshape, Dot, ...).
    // NGRAPH_PASS_ENABLES "HIPLayout:0" keeps every tensor in nGraph's layout.
    int binary_code(const Node& n);
    static bool is_conv(const Node* n)
    {
        return is_type<op::v0::QuantizedConvolution>(n) || is_type<op::v0::QuantizedConvolutionBias>(n) || is_type<op::v0::QuantizedConvolutionRelu>(n) ||
               is_type<op::v0::QuantizedConvolutionBiasAdd>(n) || is_type<op::v0::QuantizedConvolutionBiasSignedAdd>(n);
    }
    static int conv_sum_input(const Node* n)
    {
        return (is_type<op::v0::QuantizedConvolutionBiasAdd>(n) || is_type<op::v0::QuantizedConvolutionBiasSignedAdd>(n)) ? 3 : -1;
    }
    // A pool that leaves no spatial extent (a global average): its output has the same bytes in
    // either layout, so it reads whatever layout its input has and ties nothing -- a Reshape or a
    // GEMM behind it must not pull the network in front of it back into nGraph's layout.
    static bool pool_to_points(const Node* n)
    {
        if (!(is_type<op::v0::MaxPool>(n) || is_type<op::v0::AvgPool>(n)) || n->get_output_size() != 1)
            return false;
        const Shape& s = n->get_output_shape(0);
        size_t spatial = 1;
        for (size_t i = 2; i < s.size(); ++i)
            spatial *= s[i];
        return s.size() >= 3 && spatial == 1;
    }
    // inputs of a layout-agnostic op that must share its output's layout (empty: not such an op)
    static vector<size_t> tied_inputs(const Node* n)
    {
        vector<size_t> r;
        const size_t rank = n->get_output_size() == 1 ? n->get_output_shape(0).size() : 0;
        if (rank < 3 || pool_to_points(n))
            return r;
        if (is_type<op::v0::Relu>(n) || is_type<op::v0::Abs>(n) || is_type<op::v0::Convert>(n) || is_type<op::v0::MaxPool>(n) || is_type<op::v0::AvgPool>(n))
            r.push_back(0);
        else if (auto q = as_type<const op::v0::Quantize>(n))
        {
            if (q->get_axes().empty())
                r.push_back(0);
        }
        else if (auto dq = as_type<const op::v0::Dequantize>(n))
        {
            if (dq->get_axes().empty())
                r.push_back(0);
        }
        else if (is_type<op::v0::Concat>(n))
            for (size_t i = 0; i < n->get_input_size(); ++i)
                r.push_back(i);
        else if (binary_code(*n) >= 0)
            for (size_t i = 0; i < 2; ++i)
                if (n->get_input_shape(i) == n->get_output_shape(0))
                    r.push_back(i);
        return r;
    }

    // One f32 value shared by every element of a Constant (also behind Broadcasts): what a graph's
    // "x * c" looks like before and after constant folding.
    bool uniform_f32_constant(const Output<Node>& o, float* value)
    {
        shared_ptr<Node> n = o.get_node_shared_ptr();
        while (is_type<op::v0::Broadcast>(n))
            n = n->get_argument(0);
        auto c = as_type_ptr<op::v0::Constant>(n);
        if (!c || c->get_output_element_type(0) != element::f32)
            return false;
        const size_t count = shape_size(c->get_output_shape(0));
        if (count == 0)
            return false;
        const float* p = static_cast<const float*>(c->get_data_ptr());
        for (size_t i = 1; i < count; ++i)
            if (memcmp(p + i, p, sizeof(float)) != 0)
                return false;
        *value = p[0];
        return true;
    }

    // Launches that only re-read and re-write a tensor are folded into a neighbour (every fused form
    // of the library equals the op sequence bit for bit): Multiply by a constant into the Softmax it
    // feeds, Add into the LayerNorm it feeds, Quantize (one scale and zero point) into the LayerNorm
    // or Gelu that produces its input.  Switch: NGRAPH_PASS_ENABLES "HIPGlueFusion:0".
    void HIPExecutable::plan_glue_fusion()
    {
        pass::PassConfig config;
        auto en = config.get_enables().find("HIPGlueFusion");
        if (en != config.get_enables().end() && !en->second)
            return;
        unordered_map<const Node*, vector<const Node*>> users;
        for (const auto& n : m_function->get_ordered_ops())
            for (size_t i = 0; i < n->get_input_size(); ++i)
                users[n->input_value(i).get_node()].push_back(n.get());
        auto single_user = [&](const Node* n) { return users[n].size() == 1; };
        for (const auto& n : m_function->get_ordered_ops())
        {
            if (is_type<op::v0::MaxPool>(n))
            {
                // MaxPool(QuantizedConvolutionBias / Relu) with a constant filter, for the pairs the
                // library has a fused kernel for (a network's first two layers)
                const auto conv = n->input_value(0).get_node_shared_ptr();
                if ((is_type<op::v0::QuantizedConvolutionBias>(conv) || is_type<op::v0::QuantizedConvolutionRelu>(conv)) && single_user(conv.get()) &&
                    !conv->is_output() && conv->get_argument(1)->is_constant())
                {
                    const ConvCall c = conv_call(conv);
                    hipq_pool_desc_t pd;
                    try
                    {
                        pd = pool_desc(n);
                    }
                    catch (const exception&)
                    {
                        continue; // (lowering the pool by itself reports what is wrong with it)
                    }
                    if (hipq_conv_max_pool_fusable(&c.d, &c.f, &pd))
                    {
                        m_pool_of_conv[n.get()] = conv;
                        m_folded.insert(conv.get());
                    }
                }
                continue;
            }
            if (auto sm = as_type_ptr<op::v0::Softmax>(n))
            {
                auto mul = as_type_ptr<op::v1::Multiply>(n->input_value(0).get_node_shared_ptr());
                if (!mul || !single_user(mul.get()) || n->get_output_element_type(0) != element::f32 || mul->get_output_shape(0) != n->get_output_shape(0))
                    continue;
                for (size_t side = 0; side < 2; ++side)
                {
                    float c = 0.0f;
                    if (mul->get_input_shape(1 - side) == n->get_output_shape(0) && uniform_f32_constant(mul->input_value(side), &c))
                    {
                        m_softmax_of_product[n.get()] = ScaledInput{mul->input_value(1 - side), c};
                        m_folded.insert(mul.get());
                        break;
                    }
                }
            }
            else if (auto ln = as_type_ptr<op::v0::LayerNorm>(n))
            {
                auto add = as_type_ptr<op::v1::Add>(n->input_value(0).get_node_shared_ptr());
                if (add && single_user(add.get()) && !ln->get_keep_stats() && n->get_output_element_type(0) == element::f32 &&
                    add->get_input_shape(0) == add->get_output_shape(0) && add->get_input_shape(1) == add->get_output_shape(0))
                {
                    m_layer_norm_of_sum[n.get()] = {add->input_value(0), add->input_value(1)};
                    m_folded.insert(add.get());
                }
            }
        }
        // attention: context = BatchMatMul(Softmax over the keys of [Multiply(] BatchMatMulTranspose(q, k) [, c)], v)
        // with 128 keys of depth 64 and query rows in multiples of 32 (what hipq_attention_f32 takes);
        // scores, product and probabilities must have no other reader
        for (const auto& n : m_function->get_ordered_ops())
        {
            const bool plain = is_type<op::v0::BatchMatMul>(n);
            auto bt = as_type_ptr<op::v0::BatchMatMulTranspose>(n);
            if (!plain && !(bt && !bt->get_transpose_arg0() && !bt->get_transpose_arg1()))
                continue;
            auto sm = as_type_ptr<op::v0::Softmax>(n->input_value(0).get_node_shared_ptr());
            if (!sm || !single_user(sm.get()) || n->get_output_element_type(0) != element::f32 || sm->get_output_shape(0).size() != 3 || sm->get_axes() != AxisSet{2})
                continue;
            const auto product = m_softmax_of_product.find(sm.get());
            const Output<Node> scores_out = product != m_softmax_of_product.end() ? product->second.x : sm->input_value(0);
            auto scores = as_type_ptr<op::v0::BatchMatMulTranspose>(scores_out.get_node_shared_ptr());
            if (!scores || scores->get_transpose_arg0() || !scores->get_transpose_arg1() || !single_user(scores.get()))
                continue;
            const Shape& qs = scores->get_input_shape(0);
            const Shape& ks = scores->get_input_shape(1);
            const Shape& vs = n->get_input_shape(1);
            if (ks[1] != 128 || ks[2] != 64 || qs[1] % 32 != 0 || vs != ks)
                continue;
            m_attention[n.get()] = Attention{scores->input_value(0), scores->input_value(1), n->input_value(1), product != m_softmax_of_product.end(),
                                             product != m_softmax_of_product.end() ? product->second.factor : 1.0f};
            m_folded.insert(scores.get());
            m_folded.insert(sm.get()); // (a Multiply in between is folded already)
        }
        for (const auto& n : m_function->get_ordered_ops())
        {
            auto q = as_type_ptr<op::v0::Quantize>(n);
            if (!q || !q->get_axes().empty() || n->get_input_element_type(0) != element::f32)
                continue;
            const auto qt = n->get_output_element_type(0);
            if (qt != element::i8 && qt != element::u8)
                continue;
            const Node* producer = n->input_value(0).get_node();
            const bool from_ln = is_type<op::v0::LayerNorm>(producer) && !static_cast<const op::v0::LayerNorm*>(producer)->get_keep_stats();
            if (!(from_ln || is_type<op::v0::Gelu>(producer)) || m_quantized_copy.count(producer))
                continue;
            auto cs = as_type_ptr<op::v0::Constant>(n->input_value(1).get_node_shared_ptr());
            auto cz = as_type_ptr<op::v0::Constant>(n->input_value(2).get_node_shared_ptr());
            if (!cs || !cz || shape_size(cs->get_output_shape(0)) != 1 || shape_size(cz->get_output_shape(0)) != 1)
                continue;
            const float scale = *static_cast<const float*>(cs->get_data_ptr());
            const int32_t zp = qt == element::i8 ? static_cast<int32_t>(*static_cast<const int8_t*>(cz->get_data_ptr())) : static_cast<int32_t>(*static_cast<const uint8_t*>(cz->get_data_ptr()));
            m_quantized_copy[producer] = QuantizedCopy{n, scale, zp, single_user(producer)};
            m_folded.insert(n.get());
        }
        // Quantize(Gelu(QuantizedDotBias -> f32)) with nothing else reading the product or the Gelu, and
        // constant (prepacked) weights: Gelu and Quantize ride in the product's epilogue
        for (const auto& n : m_function->get_ordered_ops())
        {
            if (!is_type<op::v0::Gelu>(n))
                continue;
            const auto qc = m_quantized_copy.find(n.get());
            if (qc == m_quantized_copy.end() || !qc->second.only_user)
                continue;
            const Node* dot = n->input_value(0).get_node();
            if (!is_type<op::v0::QuantizedDotBias>(dot) || !single_user(dot) || dot->get_output_element_type(0) != element::f32 || !dot->get_argument(1)->is_constant())
                continue;
            {
                // the fused entry point needs the weights lower_dot prepacks: shapes the library does not
                // pack (a reduction that is not a multiple of 16, ...) keep Gelu and Quantize as they are
                hipq_dot_desc_t d;
                memset(&d, 0, sizeof(d));
                d.a_t = dtype_of(dot->get_input_element_type(0));
                d.b_t = dtype_of(dot->get_input_element_type(1));
                d.out_t = dtype_of(dot->get_output_element_type(0));
                d.b_layout = HIPQ_B_NK;
                d.M = static_cast<int64_t>(dot->get_input_shape(0).at(0));
                d.K = static_cast<int64_t>(dot->get_input_shape(0).at(1));
                d.N = static_cast<int64_t>(dot->get_input_shape(1).at(0));
                if (hipq_dot_packed_bytes(&d) == 0)
                    continue;
            }
            QuantizedCopy copy = qc->second;
            copy.through_gelu = true;
            m_quantized_copy.erase(qc);
            m_quantized_copy[dot] = copy;
            m_folded.insert(n.get());
        }
    }

    void HIPExecutable::assign_layouts()
    {
        pass::PassConfig config;
        auto en = config.get_enables().find("HIPLayout");
        if (en != config.get_enables().end() && !en->second)
            return;
        const auto ops = m_function->get_ordered_ops();
        unordered_map<const Node*, const Node*> parent;
        for (const auto& n : ops)
            parent[n.get()] = n.get();
        function<const Node*(const Node*)> find = [&](const Node* x) {
            while (parent[x] != x)
                x = parent[x] = parent[parent[x]];
            return x;
        };
        auto unite = [&](const Node* a, const Node* b) { parent[find(a)] = find(b); };
        // classes
        for (const auto& n : ops)
        {
            for (size_t i : tied_inputs(n.get()))
                unite(n->input_value(i).get_node(), n.get());
            const int si = conv_sum_input(n.get());
            if (si >= 0)
                unite(n->input_value(si).get_node(), n.get());
        }
        // pins
        unordered_map<const Node*, bool> pinned;
        auto pin = [&](const Node* x) { pinned[find(x)] = true; };
        for (const auto& n : ops)
        {
            const Node* p = n.get();
            const bool conv = is_conv(p);
            const vector<size_t> tied = tied_inputs(p);
            if (!conv && tied.empty())
                pin(p); // produces nGraph's layout (or has none)
            if (p->get_output_size() != 1 || p->get_output_shape(0).size() < 3)
                pin(p);
            for (size_t i = 0; i < p->get_input_size(); ++i)
            {
                const bool free_read = (conv && (i == 0 || static_cast<int>(i) == conv_sum_input(p))) || (i == 0 && pool_to_points(p));
                const bool tied_read = find(p->input_value(i).get_node()) == find(p) && !tied.empty();
                if (!free_read && !tied_read)
                    pin(p->input_value(i).get_node());
                if (p->input_value(i).get_index() != 0)
                    pin(p->input_value(i).get_node());
            }
        }
        for (const auto& n : ops)
            if (!pinned.count(find(n.get())))
                m_nxc[n.get()] = true;
    }

    HIPExecutable::ConvCall HIPExecutable::conv_call(const shared_ptr<Node>& n) const
    {
        ConvCall c;
        ConvAttrs attrs;
        // input positions per op (src/ngraph/op/experimental/quantized_conv_bias.cpp, quantized_conv_relu.cpp)
        bool relu = false;
        if (auto q = as_type_ptr<op::v0::QuantizedConvolution>(n))
        {
            attrs = conv_attrs(*q);
            c.plain = true;
        }
        else if (auto qb = as_type_ptr<op::v0::QuantizedConvolutionBias>(n))
        {
            attrs = conv_attrs(*qb);
            c.bias_i = 2, c.scale_i = 3, relu = qb->with_relu();
        }
        else if (auto qr = as_type_ptr<op::v0::QuantizedConvolutionRelu>(n))
        {
            attrs = conv_attrs(*qr);
            c.scale_i = 2, relu = true;
        }
        else if (auto qa = as_type_ptr<op::v0::QuantizedConvolutionBiasAdd>(n))
        {
            attrs = conv_attrs(*qa);
            c.bias_i = 2, c.sum_i = 3, c.scale_i = 4, c.sum_scale_i = 5, relu = qa->with_relu();
        }
        else if (auto qs = as_type_ptr<op::v0::QuantizedConvolutionBiasSignedAdd>(n))
        {
            attrs = conv_attrs(*qs);
            c.bias_i = 2, c.sum_i = 3, c.scale_i = 4, c.sum_scale_i = 5, relu = qs->with_relu();
        }
        fill_conv_desc(c.d, *n, attrs);
        c.d.data_layout = nxc(n->input_value(0).get_node()) ? HIPQ_LAYOUT_NXC : HIPQ_LAYOUT_NCX;
        c.d.out_layout = nxc(n.get()) ? HIPQ_LAYOUT_NXC : HIPQ_LAYOUT_NCX; // the sum input is in the output's class
        memset(&c.f, 0, sizeof(c.f));
        if (c.plain)
            return c;
        c.f.has_bias = c.bias_i >= 0;
        c.f.has_sum = c.sum_i >= 0;
        c.f.sum_t = c.sum_i >= 0 ? dtype_of(n->get_input_element_type(c.sum_i)) : HIPQ_U8;
        c.f.with_relu = relu;
        c.f.scale_count = static_cast<int64_t>(shape_size(n->get_input_shape(c.scale_i)));
        if (c.f.scale_count != 1 && c.f.scale_count != c.d.K)
            throw ngraph_error("HIP backend: requantization scale must be a scalar or have one entry per output channel");
        if (c.sum_scale_i >= 0 && shape_size(n->get_input_shape(c.sum_scale_i)) != 1)
            throw ngraph_error("HIP backend: sum scale must be a scalar");
        return c;
    }

    // A constant filter whose zero point is a constant 0 (the fused ops have none) is packed once at
    // compile time; the nGraph CPU backend makes the same demand of its fast path
    // (src/ngraph/runtime/cpu/pass/cpu_assignment.cpp:801-825).  Null when there is nothing to pack.
    shared_ptr<DeviceBlock> HIPExecutable::packed_filter(const shared_ptr<Node>& n, const ConvCall& c)
    {
        shared_ptr<DeviceBlock> packed;
        const bool filter_const = n->get_argument(1)->is_constant();
        const bool zp_zero = c.plain ? constant_is_zero(n->input_value(5)) : true;
        const size_t packed_bytes = hipq_conv_packed_filter_bytes(&c.d);
        if (filter_const && zp_zero && packed_bytes)
        {
            packed = alloc(packed_bytes);
            check(hipq_conv_pack_filter(&c.d, constant_ptr(n->input_value(1)), packed->ptr, m_stream), "filter packing");
        }
        return packed;
    }

    void HIPExecutable::lower_conv(const shared_ptr<Node>& n, Step& st)
    {
        const ConvCall c = conv_call(n);
        const hipq_conv_desc_t d = c.d;
        const shared_ptr<DeviceBlock> packed = packed_filter(n, c);
        if (c.plain)
        {
            st.launch = [d, packed](const vector<void*>& in, void* out, void* stream) {
                check(hipq_quantized_convolution(&d, in[0], in[1], packed ? packed->ptr : nullptr, static_cast<const float*>(in[2]), in[3],
                                                 static_cast<const float*>(in[4]), in[5], static_cast<const float*>(in[6]), in[7], out, stream),
                      "QuantizedConvolution");
            };
            return;
        }
        const hipq_fused_desc_t f = c.f;
        const int bias_i = c.bias_i, sum_i = c.sum_i, scale_i = c.scale_i, sum_scale_i = c.sum_scale_i;
        const string name = n->get_type_name();
        st.launch = [d, f, packed, bias_i, sum_i, scale_i, sum_scale_i, name](const vector<void*>& in, void* out, void* stream) {
            check(hipq_quantized_convolution_fused(&d, &f, in[0], in[1], packed ? packed->ptr : nullptr,
                                                   bias_i >= 0 ? static_cast<const int32_t*>(in[bias_i]) : nullptr,
                                                   sum_i >= 0 ? in[sum_i] : nullptr, static_cast<const float*>(in[scale_i]),
                                                   sum_scale_i >= 0 ? static_cast<const float*>(in[sum_scale_i]) : nullptr, out, stream),
                  name.c_str());
        };
    }

    void HIPExecutable::lower_dot(const shared_ptr<Node>& n, Step& st, const hipq_quant_out_t* gelu_quantize, int gelu_quantize_at)
    {
        hipq_dot_desc_t d;
        memset(&d, 0, sizeof(d));
        const Shape& s0 = n->get_input_shape(0);
        const Shape& s1 = n->get_input_shape(1);
        d.a_t = dtype_of(n->get_input_element_type(0));
        d.b_t = dtype_of(n->get_input_element_type(1));
        d.out_t = dtype_of(n->get_output_element_type(0));
        if (auto q = as_type_ptr<op::v0::QuantizedDot>(n))
        {
            // the INTERPRETER runs every QuantizedDot with one reduction axis (int_executable.hpp:1583)
            if (q->get_reduction_axes_count() != 1)
                throw unsupported_op("HIP backend: QuantizedDot with reduction_axes_count != 1");
            d.b_layout = HIPQ_B_KN;
            d.K = static_cast<int64_t>(s1.at(0));
            d.M = static_cast<int64_t>(shape_size(s0) / (s0.empty() ? 1 : s0.back() ? s0.back() : 1));
            d.N = static_cast<int64_t>(shape_size(s1) / (s1[0] ? s1[0] : 1));
            shared_ptr<DeviceBlock> packed;
            size_t pb = hipq_dot_packed_bytes(&d);
            if (pb && n->get_argument(1)->is_constant() && constant_is_zero(n->input_value(5)))
            {
                packed = alloc(pb);
                check(hipq_dot_pack(&d, constant_ptr(n->input_value(1)), packed->ptr, m_stream), "QuantizedDot operand packing");
            }
            st.launch = [d, packed](const vector<void*>& in, void* out, void* stream) {
                // without a prepacked operand the direct kernel runs unless the zero point is known to be 0
                check(hipq_quantized_dot(&d, in[0], in[1], packed ? packed->ptr : nullptr, static_cast<const float*>(in[2]), in[3],
                                         static_cast<const float*>(in[4]), in[5], static_cast<const float*>(in[6]), in[7], out, stream),
                      "QuantizedDot");
            };
            return;
        }
        auto qb = as_type_ptr<op::v0::QuantizedDotBias>(n);
        d.b_layout = HIPQ_B_NK;
        d.M = static_cast<int64_t>(s0.at(0));
        d.K = static_cast<int64_t>(s0.at(1));
        d.N = static_cast<int64_t>(s1.at(0));
        hipq_fused_desc_t f;
        memset(&f, 0, sizeof(f));
        f.has_bias = 1;
        f.with_relu = qb->with_relu();
        f.scale_count = static_cast<int64_t>(shape_size(n->get_input_shape(3)));
        if (f.scale_count != 1 && f.scale_count != d.N)
            throw ngraph_error("HIP backend: QuantizedDotBias scale must be a scalar or have one entry per output column");
        shared_ptr<DeviceBlock> packed;
        size_t pb = hipq_dot_packed_bytes(&d);
        if (pb && n->get_argument(1)->is_constant())
        {
            packed = alloc(pb);
            check(hipq_dot_pack(&d, constant_ptr(n->input_value(1)), packed->ptr, m_stream), "QuantizedDotBias weight packing");
        }
        if (gelu_quantize)
        {
            // Quantize(Gelu(product)): the bytes go to the folded Quantize's value; the product's own value stays unwritten
            const hipq_quant_out_t q0 = *gelu_quantize;
            st.launch = [d, f, packed, q0, gelu_quantize_at](const vector<void*>& in, void*, void* stream) {
                hipq_quant_out_t q = q0;
                q.out = in[gelu_quantize_at];
                check(hipq_quantized_dot_bias_gelu_quantize(&d, &f, in[0], in[1], packed ? packed->ptr : nullptr, static_cast<const int32_t*>(in[2]), static_cast<const float*>(in[3]), &q, stream),
                      "QuantizedDotBias with Gelu and Quantize");
            };
            return;
        }
        st.launch = [d, f, packed](const vector<void*>& in, void* out, void* stream) {
            check(hipq_quantized_dot_bias(&d, &f, in[0], in[1], packed ? packed->ptr : nullptr, static_cast<const int32_t*>(in[2]),
                                          static_cast<const float*>(in[3]), out, stream),
                  "QuantizedDotBias");
        };
    }

    int binary_code(const Node& n)
    {
        const auto& ti = n.get_type_info();
        if (ti == op::v1::Add::type_info)
            return HIPQ_OP_ADD;
        if (ti == op::v1::Subtract::type_info)
            return HIPQ_OP_SUBTRACT;
        if (ti == op::v1::Multiply::type_info)
            return HIPQ_OP_MULTIPLY;
        if (ti == op::v1::Divide::type_info)
        {
            // integer division floors unless the op says otherwise (src/ngraph/op/divide.hpp:72,
            // src/ngraph/runtime/reference/divide.hpp:41-60); floats divide the same way under both
            const auto* div = static_cast<const op::v1::Divide*>(&n);
            return (div->is_pythondiv() && !n.get_output_element_type(0).is_real()) ? HIPQ_OP_DIVIDE_FLOOR : HIPQ_OP_DIVIDE;
        }
        if (ti == op::v1::Maximum::type_info)
            return HIPQ_OP_MAXIMUM;
        if (ti == op::v1::Minimum::type_info)
            return HIPQ_OP_MINIMUM;
        return -1;
    }

    // MaxPool / AvgPool over [N, C, spatial...] (src/ngraph/runtime/reference/max_pool.hpp:127-222, avg_pool.hpp:128-250)
    hipq_pool_desc_t HIPExecutable::pool_desc(const shared_ptr<Node>& n) const
    {
        hipq_pool_desc_t d;
        memset(&d, 0, sizeof(d));
        const Shape& in = n->get_input_shape(0);
        if (in.size() < 3 || in.size() > 5)
            throw unsupported_op("HIP backend: pooling with " + to_string(in.size() < 2 ? 0 : in.size() - 2) + " spatial dimensions");
        const Shape *window, *pb, *pa;
        const Strides* strides;
        if (auto mp = as_type_ptr<op::v0::MaxPool>(n))
        {
            d.op = HIPQ_POOL_MAX;
            window = &mp->get_window_shape();
            strides = &mp->get_window_movement_strides();
            pb = &mp->get_padding_below();
            pa = &mp->get_padding_above();
        }
        else
        {
            auto ap = as_type_ptr<op::v0::AvgPool>(n);
            d.op = HIPQ_POOL_AVG;
            d.include_padding = ap->get_include_padding_in_avg_computation() ? 1 : 0;
            window = &ap->get_window_shape();
            strides = &ap->get_window_movement_strides();
            pb = &ap->get_padding_below();
            pa = &ap->get_padding_above();
        }
        d.dtype = dtype_of(n->get_output_element_type(0));
        // input and output share a class, except where the output is points (the same bytes either way)
        d.layout = nxc(pool_to_points(n.get()) ? n->input_value(0).get_node() : n.get()) ? HIPQ_LAYOUT_NXC : HIPQ_LAYOUT_NCX;
        d.n_spatial = static_cast<int32_t>(in.size() - 2);
        d.N = static_cast<int64_t>(in[0]);
        d.C = static_cast<int64_t>(in[1]);
        for (int i = 0; i < d.n_spatial; ++i)
        {
            d.in_sp[i] = static_cast<int64_t>(in[2 + i]);
            d.window[i] = static_cast<int64_t>((*window)[i]);
            d.stride[i] = static_cast<int64_t>((*strides)[i]);
            d.pad_below[i] = static_cast<int64_t>((*pb)[i]);
            d.pad_above[i] = static_cast<int64_t>((*pa)[i]);
        }
        check(hipq_pool_infer_output(&d), n->description().c_str());
        const Shape& out = n->get_output_shape(0);
        for (int i = 0; i < d.n_spatial; ++i)
            if (d.out_sp[i] != static_cast<int64_t>(out[2 + i]))
                throw runtime_error("HIP backend: pooling output shape disagrees with the node's");
        return d;
    }

    void HIPExecutable::lower_pool(const shared_ptr<Node>& n, Step& st)
    {
        const hipq_pool_desc_t d = pool_desc(n);
        const auto fused = m_pool_of_conv.find(n.get());
        if (fused != m_pool_of_conv.end())
        {
            // the step's inputs are the convolution's (lower): data, filter, bias / scale
            const ConvCall c = conv_call(fused->second);
            const shared_ptr<DeviceBlock> packed = packed_filter(fused->second, c);
            if (!packed)
                throw runtime_error("HIP backend: fused convolution + MaxPool without a packed filter");
            const hipq_conv_desc_t cd = c.d;
            const hipq_fused_desc_t cf = c.f;
            const int bias_i = c.bias_i, scale_i = c.scale_i;
            st.launch = [cd, cf, d, packed, bias_i, scale_i](const vector<void*>& in, void* out, void* stream) {
                check(hipq_quantized_convolution_fused_max_pool(&cd, &cf, &d, in[0], packed->ptr, bias_i >= 0 ? static_cast<const int32_t*>(in[bias_i]) : nullptr,
                                                                static_cast<const float*>(in[scale_i]), out, stream),
                      "QuantizedConvolutionBias + MaxPool");
            };
            return;
        }
        st.launch = [d](const vector<void*>& in, void* out, void* stream) { check(hipq_pool(&d, in[0], out, stream), "pooling"); };
    }

    bool backend_supports(const Node& n)
    {
        static const vector<NodeTypeInfo> ops = {
            op::v0::Parameter::type_info, op::v0::Constant::type_info, op::v0::Result::type_info, op::v0::Quantize::type_info,
            op::v0::Dequantize::type_info, op::v0::QuantizedConvolution::type_info, op::v0::QuantizedConvolutionBias::type_info,
            op::v0::QuantizedConvolutionRelu::type_info, op::v0::QuantizedConvolutionBiasAdd::type_info,
            op::v0::QuantizedConvolutionBiasSignedAdd::type_info, op::v0::QuantizedDot::type_info, op::v0::QuantizedDotBias::type_info,
            op::v0::Abs::type_info, op::v0::Relu::type_info, op::v0::Convert::type_info, op::v0::Broadcast::type_info,
            op::v0::Reshape::type_info, op::v1::Add::type_info, op::v1::Subtract::type_info, op::v1::Multiply::type_info,
            op::v1::Divide::type_info, op::v1::Maximum::type_info, op::v1::Minimum::type_info, op::v0::MaxPool::type_info,
            op::v0::AvgPool::type_info, op::v0::Concat::type_info, op::v0::Slice::type_info, op::v0::Softmax::type_info, op::v0::Erf::type_info,
            op::v0::Gelu::type_info, op::v0::LayerNorm::type_info, op::v0::BatchMatMul::type_info, op::v0::BatchMatMulTranspose::type_info};
        for (const auto& ti : ops)
            if (n.get_type_info() == ti)
                return true;
        return false;
    }

    void HIPExecutable::lower(const shared_ptr<Node>& n)
    {
        if (!backend_supports(*n))
            throw unsupported_op(string("Unsupported op '") + n->description() + "'");
        // one output a step, except LayerNorm with its statistics: further outputs get the following
        // value ids and reach the launch as pointers after the inputs
        if (n->get_output_size() != 1 && !is_type<op::v0::LayerNorm>(n))
            throw unsupported_op(string("HIP backend: op '") + n->description() + "' with " + to_string(n->get_output_size()) + " outputs");
        // folded into a neighbour: no launch and (Multiply, Add) no value; a folded Quantize got its
        // value when its producer was lowered
        if (m_folded.count(n.get()))
            return;
        const auto et = n->get_output_element_type(0);
        const size_t bytes = shape_size(n->get_output_shape(0)) * et.size();
        const int id = static_cast<int>(m_value_ptr.size());

        if (n->is_output())
        {
            // a Result aliases the value it returns
            m_value_of[n.get()] = value_of(n->input_value(0));
            m_value_uses[value_of(n->input_value(0))] += 1;
            return;
        }
        // Ops that change what the bytes are called, not the bytes: Convert between the two 8-bit
        // integer types (a static_cast keeps the bits; the reference's CPU backend runs it in place,
        // src/ngraph/runtime/cpu/pass/cpu_assignment.cpp:983-997) and Reshape without a transposition.
        // The node shares its input's value: no launch, no memory.
        {
            bool same_bytes = false;
            if (is_type<op::v0::Convert>(n))
            {
                const auto it = n->get_input_element_type(0);
                same_bytes = (it == element::i8 || it == element::u8) && (et == element::i8 || et == element::u8);
            }
            else if (auto r = as_type_ptr<op::v0::Reshape>(n))
            {
                same_bytes = true;
                const auto& order = r->get_input_order();
                for (size_t i = 0; i < order.size(); ++i)
                    same_bytes = same_bytes && order[i] == i;
                // a transposition-free Reshape of a tensor kept channels-last would change the element
                // order nGraph defines for it unless the tensor has no spatial extent left
                if (same_bytes && nxc(n->input_value(0).get_node()))
                {
                    const Shape& is = n->get_input_shape(0);
                    size_t spatial = 1;
                    for (size_t i = 2; i < is.size(); ++i)
                        spatial *= is[i];
                    same_bytes = spatial == 1 || is.at(1) == 1;
                }
            }
            if (same_bytes)
            {
                m_value_of[n.get()] = value_of(n->input_value(0));
                return;
            }
        }
        m_value_of[n.get()] = id;
        m_value_ptr.push_back(nullptr);
        m_value_bytes.push_back(bytes);
        m_value_uses.push_back(0);
        m_value_external.push_back(n->is_parameter() || n->is_constant());
        if (n->is_parameter())
            return; // bound per call
        if (auto c = as_type_ptr<op::v0::Constant>(n))
        {
            auto block = alloc(bytes);
            check(hipq_memcpy_h2d(block->ptr, c->get_data_ptr(), bytes, m_stream), "constant upload");
            m_value_ptr[id] = block->ptr;
            return;
        }
        m_value_ptr[id] = alloc(bytes)->ptr;

        Step st;
        st.node = n;
        st.output = id;
        const auto attention = m_attention.find(n.get());
        if (attention != m_attention.end())
        {
            // the folded scores / Softmax chain in front of input 0: the launch reads q, k and v
            for (const Output<Node>& o : {attention->second.q, attention->second.k, attention->second.v})
            {
                st.inputs.push_back(value_of(o));
                m_value_uses[st.inputs.back()] += 1;
            }
        }
        const auto pool_of_conv = m_pool_of_conv.find(n.get());
        if (pool_of_conv != m_pool_of_conv.end())
        {
            // the folded convolution in front of input 0: the launch reads its data, filter, bias and scale
            for (size_t i = 0; i < pool_of_conv->second->get_input_size(); ++i)
            {
                st.inputs.push_back(value_of(pool_of_conv->second->input_value(i)));
                m_value_uses[st.inputs.back()] += 1;
            }
        }
        for (size_t i = 0; attention == m_attention.end() && pool_of_conv == m_pool_of_conv.end() && i < n->get_input_size(); ++i)
        {
            // (a folded Multiply / Add in front of input 0: the consumer reads the folded node's inputs instead)
            const auto sp = m_softmax_of_product.find(n.get());
            const auto ls = m_layer_norm_of_sum.find(n.get());
            if (i == 0 && sp != m_softmax_of_product.end())
                st.inputs.push_back(value_of(sp->second.x));
            else if (i == 0 && ls != m_layer_norm_of_sum.end())
                st.inputs.push_back(value_of(ls->second.first));
            else
                st.inputs.push_back(value_of(n->input_value(i)));
            m_value_uses[st.inputs.back()] += 1;
        }
        for (size_t o = 1; o < n->get_output_size(); ++o)
        {
            const size_t obytes = shape_size(n->get_output_shape(o)) * n->get_output_element_type(o).size();
            m_value_ptr.push_back(alloc(obytes)->ptr);
            m_value_bytes.push_back(obytes);
            m_value_uses.push_back(0);
            m_value_external.push_back(false);
            st.inputs.push_back(id + static_cast<int>(o)); // written, not read: no use counted
        }
        // glue fusion: the second addend of a folded Add, then the quantized copy a folded Quantize stands for
        int addend_at = -1, qcopy_at = -1;
        hipq_quant_out_t qcopy;
        memset(&qcopy, 0, sizeof(qcopy));
        bool qcopy_only = false;
        {
            const auto ls = m_layer_norm_of_sum.find(n.get());
            if (ls != m_layer_norm_of_sum.end())
            {
                addend_at = static_cast<int>(st.inputs.size());
                st.inputs.push_back(value_of(ls->second.second));
                m_value_uses[st.inputs.back()] += 1;
            }
            const auto qc = m_quantized_copy.find(n.get());
            if (qc != m_quantized_copy.end())
            {
                const shared_ptr<Node>& qn = qc->second.quantize;
                const size_t qbytes = shape_size(qn->get_output_shape(0));
                const int qid = static_cast<int>(m_value_ptr.size());
                m_value_of[qn.get()] = qid;
                m_value_ptr.push_back(alloc(qbytes)->ptr);
                m_value_bytes.push_back(qbytes);
                m_value_uses.push_back(0);
                m_value_external.push_back(false);
                qcopy_at = static_cast<int>(st.inputs.size());
                st.inputs.push_back(qid); // written, not read: no use counted
                auto scalars = alloc(8);
                unsigned char host[8] = {0};
                memcpy(host, &qc->second.scale, sizeof(float));
                host[4] = static_cast<unsigned char>(qc->second.zero_point & 0xFF);
                check(hipq_memcpy_h2d(scalars->ptr, host, 8, m_stream), "constant upload");
                qcopy.scale = static_cast<const float*>(scalars->ptr);
                qcopy.zero_point = static_cast<const unsigned char*>(scalars->ptr) + 4;
                qcopy.quant_t = dtype_of(qn->get_output_element_type(0));
                qcopy.round_mode = static_cast<int32_t>(static_cast<const op::v0::Quantize*>(qn.get())->get_round_mode());
                qcopy_only = qc->second.only_user;
            }
        }
        const int64_t count = static_cast<int64_t>(shape_size(n->get_output_shape(0)));
        const int dt = dtype_of(et);

        if (auto q = as_type_ptr<op::v0::Quantize>(n))
        {
            hipq_quant_desc_t d;
            memset(&d, 0, sizeof(d));
            d.real_t = dtype_of(n->get_input_element_type(0));
            d.quant_t = dt;
            d.round_mode = static_cast<int32_t>(q->get_round_mode());
            const Shape& s = n->get_input_shape(0);
            if (s.size() > HIPQ_MAX_RANK)
                throw unsupported_op("HIP backend: Quantize rank beyond 8");
            d.rank = static_cast<int32_t>(s.size());
            for (size_t i = 0; i < s.size(); ++i)
                d.shape[i] = static_cast<int64_t>(s[i]);
            for (size_t a : q->get_axes())
                d.axes_mask |= 1u << a;
            st.launch = [d](const vector<void*>& in, void* out, void* stream) { check(hipq_quantize(&d, in[0], in[1], in[2], out, stream), "Quantize"); };
        }
        else if (auto dq = as_type_ptr<op::v0::Dequantize>(n))
        {
            hipq_quant_desc_t d;
            memset(&d, 0, sizeof(d));
            d.real_t = dt;
            d.quant_t = dtype_of(n->get_input_element_type(0));
            const Shape& s = n->get_input_shape(0);
            if (s.size() > HIPQ_MAX_RANK)
                throw unsupported_op("HIP backend: Dequantize rank beyond 8");
            d.rank = static_cast<int32_t>(s.size());
            for (size_t i = 0; i < s.size(); ++i)
                d.shape[i] = static_cast<int64_t>(s[i]);
            for (size_t a : dq->get_axes())
                d.axes_mask |= 1u << a;
            st.launch = [d](const vector<void*>& in, void* out, void* stream) { check(hipq_dequantize(&d, in[0], in[1], in[2], out, stream), "Dequantize"); };
        }
        else if (is_type<op::v0::QuantizedConvolution>(n) || is_type<op::v0::QuantizedConvolutionBias>(n) ||
                 is_type<op::v0::QuantizedConvolutionRelu>(n) || is_type<op::v0::QuantizedConvolutionBiasAdd>(n) ||
                 is_type<op::v0::QuantizedConvolutionBiasSignedAdd>(n))
        {
            lower_conv(n, st);
        }
        else if (is_type<op::v0::QuantizedDot>(n) || is_type<op::v0::QuantizedDotBias>(n))
        {
            lower_dot(n, st, qcopy_at >= 0 ? &qcopy : nullptr, qcopy_at);
        }
        else if (binary_code(*n) >= 0)
        {
            const int op = binary_code(*n);
            const int64_t an = static_cast<int64_t>(shape_size(n->get_input_shape(0)));
            const int64_t bn = static_cast<int64_t>(shape_size(n->get_input_shape(1)));
            st.launch = [op, dt, an, bn, count](const vector<void*>& in, void* out, void* stream) {
                check(hipq_binary(op, dt, in[0], an == count ? an : 1, in[1], bn == count ? bn : 1, out, count, stream), "elementwise");
            };
        }
        else if (is_type<op::v0::Abs>(n) || is_type<op::v0::Relu>(n))
        {
            const int op = is_type<op::v0::Abs>(n) ? HIPQ_OP_ABS : HIPQ_OP_RELU;
            st.launch = [op, dt, count](const vector<void*>& in, void* out, void* stream) { check(hipq_unary(op, dt, in[0], out, count, stream), "unary"); };
        }
        else if (is_type<op::v0::Convert>(n))
        {
            const int it = dtype_of(n->get_input_element_type(0));
            st.launch = [it, dt, count](const vector<void*>& in, void* out, void* stream) { check(hipq_convert(it, dt, in[0], out, count, stream), "Convert"); };
        }
        else if (auto b = as_type_ptr<op::v0::Broadcast>(n))
        {
            const Shape& s = b->get_broadcast_shape();
            if (s.size() > HIPQ_MAX_RANK)
                throw unsupported_op("HIP backend: Broadcast rank beyond 8");
            vector<int64_t> shape(s.begin(), s.end());
            uint32_t mask = 0;
            for (size_t a : b->get_broadcast_axes())
                mask |= 1u << a;
            const int eb = static_cast<int>(et.size());
            st.launch = [shape, mask, eb](const vector<void*>& in, void* out, void* stream) {
                check(hipq_broadcast(eb, in[0], out, static_cast<int32_t>(shape.size()), shape.data(), mask, stream), "Broadcast");
            };
        }
        else if (auto r = as_type_ptr<op::v0::Reshape>(n))
        {
            const Shape& s = n->get_input_shape(0);
            if (s.size() > HIPQ_MAX_RANK)
                throw unsupported_op("HIP backend: Reshape rank beyond 8");
            vector<int64_t> shape(s.begin(), s.end());
            vector<int32_t> order(r->get_input_order().begin(), r->get_input_order().end());
            const int eb = static_cast<int>(et.size());
            st.launch = [shape, order, eb](const vector<void*>& in, void* out, void* stream) {
                check(hipq_permute(eb, in[0], out, static_cast<int32_t>(shape.size()), shape.data(), order.data(), stream), "Reshape");
            };
        }
        else if (is_type<op::v0::MaxPool>(n) || is_type<op::v0::AvgPool>(n))
        {
            lower_pool(n, st);
        }
        else if (auto sm = as_type_ptr<op::v0::Softmax>(n))
        {
            // src/ngraph/runtime/reference/softmax.hpp:31-57; the library takes a contiguous run of axes
            if (et != element::f32)
                throw unsupported_op("HIP backend: Softmax on " + et.get_type_name());
            const Shape& s = n->get_input_shape(0);
            const AxisSet& axes = sm->get_axes();
            const size_t first = *axes.begin(), last = *axes.rbegin();
            if (last - first + 1 != axes.size())
                throw unsupported_op("HIP backend: Softmax over axes that are not a contiguous run");
            int64_t outer = 1, axis = 1, inner = 1;
            for (size_t i = 0; i < s.size(); ++i)
                (i < first ? outer : (i <= last ? axis : inner)) *= static_cast<int64_t>(s[i]);
            const auto product = m_softmax_of_product.find(n.get());
            if (product != m_softmax_of_product.end())
            {
                // Softmax(Multiply(x, c)): the factor as a device scalar of this executable
                auto block = alloc(sizeof(float));
                check(hipq_memcpy_h2d(block->ptr, &product->second.factor, sizeof(float), m_stream), "constant upload");
                const float* factor = static_cast<const float*>(block->ptr);
                st.launch = [outer, axis, inner, factor](const vector<void*>& in, void* out, void* stream) {
                    check(hipq_softmax_scaled_f32(static_cast<const float*>(in[0]), factor, static_cast<float*>(out), outer, axis, inner, stream), "Softmax of a product");
                };
            }
            else
                st.launch = [outer, axis, inner](const vector<void*>& in, void* out, void* stream) {
                    check(hipq_softmax_f32(static_cast<const float*>(in[0]), static_cast<float*>(out), outer, axis, inner, stream), "Softmax");
                };
        }
        else if (is_type<op::v0::Erf>(n) || is_type<op::v0::Gelu>(n))
        {
            // src/ngraph/runtime/reference/erf.hpp:29-35; src/ngraph/op/gelu.cpp:46-60
            if (et != element::f32)
                throw unsupported_op("HIP backend: " + n->description() + " on " + et.get_type_name());
            const int64_t count = static_cast<int64_t>(shape_size(n->get_output_shape(0)));
            const bool gelu = is_type<op::v0::Gelu>(n);
            if (gelu && qcopy_at >= 0)
                st.launch = [count, qcopy, qcopy_at, qcopy_only](const vector<void*>& in, void* out, void* stream) {
                    hipq_quant_out_t q = qcopy;
                    q.out = in[qcopy_at];
                    check(hipq_gelu_quantize_f32(static_cast<const float*>(in[0]), qcopy_only ? nullptr : static_cast<float*>(out), &q, count, stream), "Gelu with its Quantize");
                };
            else
                st.launch = [count, gelu](const vector<void*>& in, void* out, void* stream) {
                    if (gelu)
                        check(hipq_gelu_f32(static_cast<const float*>(in[0]), static_cast<float*>(out), count, stream), "Gelu");
                    else
                        check(hipq_erf_f32(static_cast<const float*>(in[0]), static_cast<float*>(out), count, stream), "Erf");
                };
        }
        else if (auto ln = as_type_ptr<op::v0::LayerNorm>(n))
        {
            // src/ngraph/op/layer_norm.cpp:68-150; with keep_stats the mean and variance tensors follow the inputs
            if (et != element::f32)
                throw unsupported_op("HIP backend: LayerNorm on " + et.get_type_name());
            const Shape& s = n->get_input_shape(0);
            const int64_t rank = static_cast<int64_t>(s.size());
            const int64_t n_axis = ln->get_begin_norm_axis() >= 0 ? ln->get_begin_norm_axis() : rank + ln->get_begin_norm_axis();
            int64_t rows = 1, cols = 1;
            for (int64_t i = 0; i < rank; ++i)
                (i < n_axis ? rows : cols) *= static_cast<int64_t>(s[i]);
            const bool affine = ln->get_use_affine();
            if (affine && static_cast<int64_t>(shape_size(n->get_input_shape(1))) != cols)
                throw unsupported_op("HIP backend: LayerNorm scale that does not cover the normalised axes");
            const double eps = ln->get_epsilon();
            const bool stats = ln->get_keep_stats();
            const size_t first_stat = affine ? 3 : 1;
            if (addend_at >= 0 || qcopy_at >= 0)
                st.launch = [rows, cols, affine, eps, addend_at, qcopy, qcopy_at](const vector<void*>& in, void* out, void* stream) {
                    hipq_quant_out_t q = qcopy;
                    if (qcopy_at >= 0)
                        q.out = in[qcopy_at];
                    check(hipq_add_layer_norm_f32(static_cast<const float*>(in[0]), addend_at >= 0 ? static_cast<const float*>(in[addend_at]) : nullptr,
                                                  affine ? static_cast<const float*>(in[1]) : nullptr, affine ? static_cast<const float*>(in[2]) : nullptr, static_cast<float*>(out),
                                                  qcopy_at >= 0 ? &q : nullptr, rows, cols, eps, stream),
                          "LayerNorm with its Add / Quantize");
                };
            else
                st.launch = [rows, cols, affine, eps, stats, first_stat](const vector<void*>& in, void* out, void* stream) {
                    check(hipq_layer_norm_f32(static_cast<const float*>(in[0]), affine ? static_cast<const float*>(in[1]) : nullptr, affine ? static_cast<const float*>(in[2]) : nullptr,
                                              static_cast<float*>(out), stats ? static_cast<float*>(in[first_stat]) : nullptr, stats ? static_cast<float*>(in[first_stat + 1]) : nullptr,
                                              rows, cols, eps, stream),
                          "LayerNorm");
                };
        }
        else if (is_type<op::v0::BatchMatMul>(n) || is_type<op::v0::BatchMatMulTranspose>(n))
        {
            // src/ngraph/runtime/reference/batch_mat_mul.hpp:31-57
            if (et != element::f32)
                throw unsupported_op("HIP backend: " + n->description() + " on " + et.get_type_name());
            bool t0 = false, t1 = false;
            if (auto bt = as_type_ptr<op::v0::BatchMatMulTranspose>(n))
            {
                t0 = bt->get_transpose_arg0();
                t1 = bt->get_transpose_arg1();
            }
            const Shape& a = n->get_input_shape(0);
            const Shape& o = n->get_output_shape(0);
            const int64_t batch = static_cast<int64_t>(o[0]), M = static_cast<int64_t>(o[1]), N = static_cast<int64_t>(o[2]), K = static_cast<int64_t>(t0 ? a[1] : a[2]);
            if (attention != m_attention.end())
            {
                // dense [batch][rows][64] operands and result: one batch level, rows 64 apart
                const float* factor = nullptr;
                if (attention->second.scaled)
                {
                    auto block = alloc(sizeof(float));
                    check(hipq_memcpy_h2d(block->ptr, &attention->second.factor, sizeof(float), m_stream), "constant upload");
                    factor = static_cast<const float*>(block->ptr);
                }
                const int64_t keys = K, depth = N;
                const hipq_attention_view_t view{1, M * depth, 0, depth, keys * depth, 0, depth, keys * depth, 0, depth, M * depth, 0, depth};
                st.launch = [batch, M, keys, depth, factor, view](const vector<void*>& in, void* out, void* stream) {
                    check(hipq_attention_f32(static_cast<const float*>(in[0]), static_cast<const float*>(in[1]), static_cast<const float*>(in[2]), factor, static_cast<float*>(out), &view, nullptr,
                                             batch, M, keys, depth, stream),
                          "attention");
                };
            }
            else
                st.launch = [batch, M, K, N, t0, t1](const vector<void*>& in, void* out, void* stream) {
                    check(hipq_batch_matmul_f32(static_cast<const float*>(in[0]), static_cast<const float*>(in[1]), static_cast<float*>(out), batch, M, K, N, t0 ? 1 : 0, t1 ? 1 : 0, stream),
                          "BatchMatMul");
                };
        }
        else if (auto sl = as_type_ptr<op::v0::Slice>(n))
        {
            // src/ngraph/runtime/reference/slice.hpp:30-66
            const int32_t eb = static_cast<int32_t>(et.size());
            const Shape& is = n->get_input_shape(0);
            if (is.size() > HIPQ_MAX_RANK)
                throw unsupported_op("HIP backend: Slice of rank " + to_string(is.size()));
            const vector<int64_t> shape(is.begin(), is.end()), lower(sl->get_lower_bounds().begin(), sl->get_lower_bounds().end()),
                upper(sl->get_upper_bounds().begin(), sl->get_upper_bounds().end()), strides(sl->get_strides().begin(), sl->get_strides().end());
            st.launch = [eb, shape, lower, upper, strides](const vector<void*>& in, void* out, void* stream) {
                check(hipq_slice(eb, in[0], out, static_cast<int32_t>(shape.size()), shape.data(), lower.data(), upper.data(), strides.data(), stream), "Slice");
            };
        }
        else if (auto cc = as_type_ptr<op::v0::Concat>(n))
        {
            const size_t axis = static_cast<size_t>(cc->get_concatenation_axis());
            const Shape& os = n->get_output_shape(0);
            // the order the axes have in memory: nGraph's, or batch, spatial..., channels
            vector<size_t> order;
            for (size_t a = 0; a < os.size(); ++a)
                if (!(nxc(n.get()) && a == 1))
                    order.push_back(a);
            if (nxc(n.get()))
                order.push_back(1);
            int64_t outer = 1, inner = 1;
            bool before = true;
            for (size_t a : order)
            {
                if (a == axis)
                    before = false;
                else
                    (before ? outer : inner) *= static_cast<int64_t>(os[a]);
            }
            vector<int64_t> extents;
            for (size_t i = 0; i < n->get_input_size(); ++i)
                extents.push_back(static_cast<int64_t>(n->get_input_shape(i)[axis]));
            const int eb = static_cast<int>(et.size());
            st.launch = [extents, outer, inner, eb](const vector<void*>& in, void* out, void* stream) {
                check(hipq_concat(eb, static_cast<int32_t>(extents.size()), const_cast<const void* const*>(in.data()), extents.data(), outer, inner, out, stream), "Concat");
            };
        }
        else
        {
            throw unsupported_op(string("Unsupported op '") + n->description() + "'");
        }
        m_steps.push_back(move(st));
    }

    HIPExecutable::HIPExecutable(const shared_ptr<Function>& func, int device, bool enable_performance_data)
        : m_device(device), m_perf(enable_performance_data)
    {
        check(hipq_set_device(m_device), "HIP backend");
        check(hipq_stream_create(&m_stream), "stream creation");
        // work on a private copy: compile must not change the caller's graph
        m_function = clone_function(*func);
        // a pass named in NGRAPH_PASS_ENABLES with 0 is left out, like the reference CPU backend's
        // knobbed passes (src/ngraph/runtime/cpu/cpu_external_function.cpp:215-226)
        pass::Manager pm;
        const auto& knobs = pm.get_pass_config().get_enables();
        const auto fusion = knobs.find("HIPQuantFusion");
        if (fusion == knobs.end() || fusion->second)
            pm.register_pass<runtime::hip::pass::HIPQuantFusion>();
        pm.register_pass<pass::ConstantFolding>();
        pm.run_passes(m_function);
        assign_layouts();
        plan_glue_fusion();
        for (const auto& n : m_function->get_ordered_ops())
            lower(n);
        for (const auto& p : m_function->get_parameters())
            m_param_value.push_back(m_value_of.at(p.get()));
        for (const auto& r : m_function->get_results())
            m_result_value.push_back(m_value_of.at(r.get()));
        check(hipq_stream_sync(m_stream), "compile-time uploads");
        if (m_perf)
        {
            m_events.resize(m_steps.size() + 1, nullptr);
            for (auto& e : m_events)
                check(hipq_event_create(&e), "event creation");
            m_step_us.assign(m_steps.size(), 0.0);
        }
        {
            pass::PassConfig config;
            auto en = config.get_enables().find("HIPGraph");
            m_use_graph = !m_perf && !(en != config.get_enables().end() && !en->second);
        }
        // validation is against the caller's function (same parameter / result signature)
        set_parameters_and_results(*func);
    }

    HIPExecutable::~HIPExecutable()
    {
        for (auto e : m_events)
            hipq_event_destroy(e);
        if (m_graph)
            hipq_graph_destroy(m_graph);
        if (m_stream)
        {
            hipq_stream_sync(m_stream);
            hipq_stream_destroy(m_stream);
        }
    }

    bool HIPExecutable::call(const vector<shared_ptr<runtime::Tensor>>& outputs, const vector<shared_ptr<runtime::Tensor>>& inputs)
    {
        lock_guard<mutex> lock(m_mutex);
        check(hipq_set_device(m_device), "HIP backend");
        if (inputs.size() != m_param_value.size() || outputs.size() != m_result_value.size())
            throw runtime_error("HIP backend: wrong number of call arguments");
        vector<void*> ptr = m_value_ptr;
        for (size_t i = 0; i < inputs.size(); ++i)
        {
            auto t = dynamic_pointer_cast<HIPTensor>(inputs[i]);
            if (!t)
                throw runtime_error("HIP backend: input " + to_string(i) + " is not a tensor of this backend");
            ptr[m_param_value[i]] = t->device_ptr();
        }
        // a value consumed only by one Result is produced straight into the caller's tensor
        vector<void*> out_ptr(outputs.size());
        vector<bool> direct(outputs.size(), false);
        for (size_t i = 0; i < outputs.size(); ++i)
        {
            auto t = dynamic_pointer_cast<HIPTensor>(outputs[i]);
            if (!t)
                throw runtime_error("HIP backend: output " + to_string(i) + " is not a tensor of this backend");
            out_ptr[i] = t->device_ptr();
            const int v = m_result_value[i];
            if (m_value_uses[v] == 1 && !m_value_external[v])
            {
                ptr[v] = out_ptr[i];
                direct[i] = true;
            }
        }
        auto issue = [&]() {
            vector<void*> in;
            for (size_t s = 0; s < m_steps.size(); ++s)
            {
                const Step& st = m_steps[s];
                in.clear();
                for (int v : st.inputs)
                    in.push_back(ptr[v]);
                if (m_perf)
                    check(hipq_event_record(m_events[s], m_stream), "event record");
                st.launch(in, ptr[st.output], m_stream);
            }
            if (m_perf)
                check(hipq_event_record(m_events[m_steps.size()], m_stream), "event record");
            for (size_t i = 0; i < outputs.size(); ++i)
                if (!direct[i])
                    check(hipq_memcpy_d2d(out_ptr[i], ptr[m_result_value[i]], m_value_bytes[m_result_value[i]], m_stream), "result copy");
        };
        // The launch sequence of a call depends only on the tensor addresses: the first call with a
        // set of addresses runs eagerly (and lets the library size its workspace), the second is
        // captured into a HIP graph, later ones replay it -- one launch instead of one per op.
        vector<void*> key;
        for (size_t i = 0; i < inputs.size(); ++i)
            key.push_back(ptr[m_param_value[i]]);
        key.insert(key.end(), out_ptr.begin(), out_ptr.end());
        if (m_use_graph && m_graph && key == m_graph_key && hipq_workspace_epoch() == m_graph_epoch)
            check(hipq_graph_launch(m_graph, m_stream), "graph launch");
        else if (m_use_graph && !m_steps.empty() && key == m_last_key)
        {
            if (m_graph)
            {
                hipq_graph_destroy(m_graph);
                m_graph = nullptr;
            }
            check(hipq_capture_begin(m_stream), "stream capture");
            try
            {
                issue();
            }
            catch (...)
            {
                void* dropped = nullptr;
                hipq_capture_end(m_stream, &dropped);
                hipq_graph_destroy(dropped);
                throw;
            }
            check(hipq_capture_end(m_stream, &m_graph), "stream capture");
            m_graph_key = key;
            m_graph_epoch = hipq_workspace_epoch();
            check(hipq_graph_launch(m_graph, m_stream), "graph launch");
        }
        else
            issue();
        m_last_key = key;
        check(hipq_stream_sync(m_stream), "Executable::call");
        if (m_perf)
        {
            for (size_t s = 0; s < m_steps.size(); ++s)
            {
                float ms = 0;
                check(hipq_event_elapsed_ms(m_events[s], m_events[s + 1], &ms), "event timing");
                m_step_us[s] += ms * 1e3;
            }
            ++m_calls;
        }
        for (auto& t : outputs)
            t->set_stale(false);
        return true;
    }

    vector<runtime::PerformanceCounter> HIPExecutable::get_performance_data() const
    {
        vector<runtime::PerformanceCounter> rc;
        if (m_perf)
            for (size_t s = 0; s < m_steps.size(); ++s)
                rc.emplace_back(m_steps[s].node, static_cast<size_t>(m_step_us[s]), m_calls);
        return rc;
    }

    // ------------------------------------------------------------------ backend
    class HIPBackend : public runtime::Backend
    {
    public:
        explicit HIPBackend(const string& config) : m_device(0)
        {
            // "HIP:<device ordinal>"
            if (!config.empty())
            {
                size_t used = 0;
                try
                {
                    m_device = stoi(config, &used);
                }
                catch (const exception&)
                {
                    used = 0;
                }
                if (used != config.size() || m_device < 0)
                    throw runtime_error("HIP backend: cannot read device ordinal from '" + config + "'");
            }
            int rc = hipq_set_device(m_device);
            if (rc != HIPQ_OK)
                throw runtime_error(string("HIP backend: device ") + to_string(m_device) + " is not usable: " + hipq_last_error());
        }
        shared_ptr<runtime::Tensor> create_tensor() override { throw runtime_error("HIP backend does not support dynamic tensors"); }
        shared_ptr<runtime::Tensor> create_tensor(const element::Type& et, const Shape& shape) override
        {
            use_device();
            return make_shared<HIPTensor>(et, shape);
        }
        // memory_pointer is device memory owned by the caller
        shared_ptr<runtime::Tensor> create_tensor(const element::Type& et, const Shape& shape, void* memory_pointer) override
        {
            use_device();
            return make_shared<HIPTensor>(et, shape, memory_pointer);
        }
        shared_ptr<runtime::Executable> compile(shared_ptr<Function> func, bool enable_performance_data = false) override
        {
            lock_guard<mutex> lock(m_mutex);
            auto it = m_cache.find(func);
            if (it != m_cache.end() && !enable_performance_data)
                return it->second;
            auto exec = make_shared<HIPExecutable>(func, m_device, enable_performance_data);
            if (!enable_performance_data)
                m_cache[func] = exec;
            return exec;
        }
        void remove_compiled_function(shared_ptr<runtime::Executable> exec) override
        {
            lock_guard<mutex> lock(m_mutex);
            for (auto it = m_cache.begin(); it != m_cache.end(); ++it)
                if (it->second == exec)
                {
                    m_cache.erase(it);
                    break;
                }
        }
        bool is_supported(const Node& node) const override { return backend_supports(node); }
        bool is_supported_property(const Property prop) const override { return prop == Property::memory_attach; }
        bool is_device_memory(void*) override { return true; }
        string get_version() const override { return "hipq-" + to_string(hipq_version()); }

    private:
        void use_device() { check(hipq_set_device(m_device), "HIP backend"); }
        int m_device;
        mutex m_mutex;
        map<shared_ptr<Function>, shared_ptr<runtime::Executable>> m_cache;
    };
}

// Found by BackendManager through dlsym("ngraph_register_hip_backend")
// (src/ngraph/runtime/backend_manager.cpp:106-113 of the nGraph tree).
extern "C" HIP_BACKEND_API void ngraph_register_hip_backend()
{
    runtime::BackendManager::register_backend("HIP", [](const string& config) { return make_shared<HIPBackend>(config); });
}
