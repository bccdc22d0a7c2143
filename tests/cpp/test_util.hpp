// copy_data / read_vector as in the reference's test/util/test_tools.hpp:79-110
#pragma once

#include "mini_test.hpp"
#include "ngraph/ngraph.hpp"

template <typename T>
void copy_data(const std::shared_ptr<ngraph::runtime::Tensor>& tv, const std::vector<T>& data)
{
    tv->write(data.data(), data.size() * sizeof(T));
}

template <typename T>
std::vector<T> read_vector(const std::shared_ptr<ngraph::runtime::Tensor>& tv)
{
    if (ngraph::element::from<T>() != tv->get_element_type())
        throw std::invalid_argument("read_vector type must match Tensor type");
    std::vector<T> rc(tv->get_element_count());
    tv->read(rc.data(), rc.size() * sizeof(T));
    return rc;
}

inline void constant_fold(const std::shared_ptr<ngraph::Function>& f)
{
    ngraph::pass::Manager pm;
    pm.register_pass<ngraph::pass::ConstantFolding>();
    pm.run_passes(f);
}

template <typename T>
size_t count_ops_of_type(const std::shared_ptr<ngraph::Function>& f)
{
    size_t n = 0;
    for (const auto& op : f->get_ordered_ops())
        if (ngraph::is_type<T>(op))
            ++n;
    return n;
}
