// hip_backend_tests [--cpu | --gpu | --all] [--list] [--exact] [substring or, with --exact, suite.name]
// hip_backend_tests --bench [--calls N] [--warmup N] [--only conv|resnet50]   (bench_backend.cpp)
#include "mini_test.hpp"

int run_backend_bench(int argc, char** argv);

int main(int argc, char** argv)
{
    if (argc > 1 && std::string(argv[1]) == "--bench")
        return run_backend_bench(argc, argv);
    bool want_cpu = true, want_gpu = false, list = false, exact = false;
    std::string filter;
    for (int i = 1; i < argc; ++i)
    {
        std::string a = argv[i];
        if (a == "--cpu")
            want_cpu = true, want_gpu = false;
        else if (a == "--gpu")
            want_cpu = false, want_gpu = true;
        else if (a == "--all")
            want_cpu = want_gpu = true;
        else if (a == "--list")
            list = true;
        else if (a == "--exact")
            exact = true;
        else
            filter = a;
    }
    if (list)
    {
        for (const auto& c : mini_test::registry())
            std::cout << (c.needs_gpu ? "gpu " : "cpu ") << c.suite << "." << c.name << std::endl;
        return 0;
    }
    int ran = 0;
    for (const auto& c : mini_test::registry())
    {
        if ((c.needs_gpu && !want_gpu) || (!c.needs_gpu && !want_cpu))
            continue;
        std::string full = c.suite + "." + c.name;
        if (!filter.empty() && (exact ? full != filter : full.find(filter) == std::string::npos))
            continue;
        std::cout << "[ RUN      ] " << full << std::endl;
        int before = mini_test::failures();
        try
        {
            c.fn();
        }
        catch (const std::exception& e)
        {
            mini_test::fail(__FILE__, __LINE__, full + " threw: " + e.what());
        }
        std::cout << (mini_test::failures() == before ? "[       OK ] " : "[  FAILED  ] ") << full << std::endl;
        ++ran;
    }
    std::cout << ran << " tests ran, " << mini_test::failures() << " failures" << std::endl;
    return mini_test::failures() == 0 && ran > 0 ? 0 : 1;
}
