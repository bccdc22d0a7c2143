// runtime::Tensor and runtime::HostTensor.
// Mirrors src/ngraph/runtime/tensor.hpp:32-120 and host_tensor.hpp:41-135 of the nGraph tree.
#pragma once

#include "ngraph/core.hpp"

namespace ngraph
{
    namespace runtime
    {
        class NGRAPH_API Tensor
        {
        protected:
            explicit Tensor(const std::shared_ptr<descriptor::Tensor>& descriptor) : m_descriptor(descriptor), m_stale(true) {}

        public:
            virtual ~Tensor() {}
            virtual const Shape& get_shape() const { return m_descriptor->get_shape(); }
            const PartialShape& get_partial_shape() const { return m_descriptor->get_shape(); }
            virtual const element::Type& get_element_type() const { return m_descriptor->get_element_type(); }
            virtual size_t get_element_count() const { return shape_size(m_descriptor->get_shape()); }
            virtual size_t get_size_in_bytes() const { return m_descriptor->size(); }
            const std::string& get_name() const { return m_descriptor->get_name(); }
            bool get_stale() const { return m_stale; }
            void set_stale(bool val) { m_stale = val; }
            // n is in bytes and must be the whole tensor
            virtual void write(const void* p, size_t n) = 0;
            virtual void read(void* p, size_t n) const = 0;
            virtual void wait_for_read_ready() {}
            virtual void wait_for_write_ready() {}
            // bounces through host memory unless a backend overrides it
            virtual void copy_from(const Tensor& source);

        protected:
            std::shared_ptr<descriptor::Tensor> m_descriptor;
            bool m_stale;
        };

        class NGRAPH_API HostTensor : public Tensor
        {
        public:
            HostTensor(const element::Type& element_type, const Shape& shape, void* memory_pointer = nullptr, const std::string& name = "");
            ~HostTensor() override;
            void write(const void* p, size_t n) override;
            void read(void* p, size_t n) const override;
            void* get_data_ptr() { return m_data; }
            const void* get_data_ptr() const { return m_data; }
            template <typename T>
            T* get_data_ptr()
            {
                return static_cast<T*>(m_data);
            }

        private:
            void* m_data;
            bool m_owned;
        };
    }
}
