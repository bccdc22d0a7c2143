// Pass manager, pass configuration and constant folding, as far as the int8 path uses them.
// Mirrors src/ngraph/pass/{manager.hpp,manager.cpp:48-170,pass.hpp,pass_config.{hpp,cpp:27-84},
// constant_folding.hpp} of the nGraph tree.
#pragma once

#include <map>
#include <typeinfo>

#include "ngraph/ops.hpp"

namespace ngraph
{
    namespace pass
    {
        // NGRAPH_PASS_ENABLES="Name:0;Other:1", NGRAPH_PASS_ATTRIBUTES="Key=1;Other=0"
        class NGRAPH_API PassConfig
        {
        public:
            PassConfig();
            const std::map<std::string, bool>& get_enables() const { return m_pass_enables; }
            void set_pass_enable(const std::string& name, bool enable) { m_pass_enables[name] = enable; }
            bool get_pass_enable(const std::string& name) const;
            void set_pass_attribute(const std::string& name, bool enable) { m_pass_attributes[name] = enable; }
            bool get_pass_attribute(const std::string& name) const;

        private:
            std::map<std::string, bool> m_pass_enables;
            std::map<std::string, bool> m_pass_attributes;
        };

        // as in src/ngraph/pass/pass.hpp:72-99: a pass has no name of its own; which passes run is the
        // registering backend's decision (it consults PassConfig the way REGISTER_KNOBBED_PASS does,
        // src/ngraph/runtime/cpu/cpu_external_function.cpp:215-226)
        class NGRAPH_API PassBase
        {
        public:
            virtual ~PassBase() {}
        };

        class NGRAPH_API FunctionPass : public PassBase
        {
        public:
            // returns true when the function was modified
            virtual bool run_on_function(std::shared_ptr<Function> f) = 0;
        };

        class NGRAPH_API Manager
        {
        public:
            Manager() = default;
            template <typename T, class... Args>
            void register_pass(Args&&... args)
            {
                m_passes.push_back(std::make_shared<T>(std::forward<Args>(args)...));
            }
            // runs the registered passes in order
            void run_passes(std::shared_ptr<Function> f);
            PassConfig& get_pass_config() { return m_config; }
            void set_pass_config(const PassConfig& c) { m_config = c; }

        private:
            std::vector<std::shared_ptr<FunctionPass>> m_passes;
            PassConfig m_config;
        };

        // Evaluates on the host every node whose inputs are all Constants, for the ops of the
        // scale sub-graphs (Abs, Add, Subtract, Multiply, Divide, Maximum, Minimum, Broadcast,
        // Convert, Relu), and replaces it by a Constant.
        class NGRAPH_API ConstantFolding : public FunctionPass
        {
        public:
            bool run_on_function(std::shared_ptr<Function> f) override;
        };
    }
}
