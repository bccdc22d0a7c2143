// A few lines of test harness (no googletest on this image): TEST registration, EXPECT macros.
#pragma once

#include <cmath>
#include <cstdio>
#include <cstring>
#include <functional>
#include <iostream>
#include <sstream>
#include <string>
#include <vector>

namespace mini_test
{
    struct Case
    {
        std::string suite, name;
        bool needs_gpu;
        std::function<void()> fn;
    };
    inline std::vector<Case>& registry()
    {
        static std::vector<Case> r;
        return r;
    }
    inline int& failures()
    {
        static int f = 0;
        return f;
    }
    struct Registrar
    {
        Registrar(const char* suite, const char* name, bool gpu, std::function<void()> fn) { registry().push_back({suite, name, gpu, fn}); }
    };
    template <typename T>
    std::string show(const std::vector<T>& v)
    {
        std::ostringstream ss;
        ss << "{";
        for (size_t i = 0; i < v.size(); ++i)
            ss << (i ? ", " : "") << +v[i];
        ss << "}";
        return ss.str();
    }
    inline void fail(const char* file, int line, const std::string& msg)
    {
        ++failures();
        std::cout << file << ":" << line << ": FAILURE: " << msg << std::endl;
    }
}

#define MT_CONCAT2(a, b) a##b
#define MT_CONCAT(a, b) MT_CONCAT2(a, b)

// GPU_TEST needs a device (runs with --gpu); CPU_TEST runs anywhere (--cpu)
#define GPU_TEST(suite, name)                                                                      \
    static void MT_CONCAT(suite##_##name, _body)();                                                \
    static mini_test::Registrar MT_CONCAT(suite##_##name, _reg)(#suite, #name, true, MT_CONCAT(suite##_##name, _body));          \
    static void MT_CONCAT(suite##_##name, _body)()
#define CPU_TEST(suite, name)                                                                      \
    static void MT_CONCAT(suite##_##name, _body)();                                                \
    static mini_test::Registrar MT_CONCAT(suite##_##name, _reg)(#suite, #name, false, MT_CONCAT(suite##_##name, _body));         \
    static void MT_CONCAT(suite##_##name, _body)()

#define EXPECT_TRUE(cond)                                                                          \
    do                                                                                             \
    {                                                                                              \
        if (!(cond))                                                                               \
            mini_test::fail(__FILE__, __LINE__, "expected true: " #cond);                          \
    } while (0)
#define EXPECT_FALSE(cond) EXPECT_TRUE(!(cond))
#define EXPECT_EQ(a, b)                                                                            \
    do                                                                                             \
    {                                                                                              \
        if (!((a) == (b)))                                                                         \
            mini_test::fail(__FILE__, __LINE__, "expected equality of " #a " and " #b);           \
    } while (0)
#define EXPECT_VEC_EQ(expected, actual)                                                            \
    do                                                                                             \
    {                                                                                              \
        auto e_ = (expected);                                                                      \
        auto a_ = (actual);                                                                        \
        if (!(e_ == a_))                                                                           \
            mini_test::fail(__FILE__, __LINE__, "expected " + mini_test::show(e_) + " got " + mini_test::show(a_));             \
    } while (0)
#define EXPECT_THROW(stmt, type)                                                                   \
    do                                                                                             \
    {                                                                                              \
        bool ok_ = false;                                                                          \
        try                                                                                        \
        {                                                                                          \
            stmt;                                                                                  \
        }                                                                                          \
        catch (const type&)                                                                        \
        {                                                                                          \
            ok_ = true;                                                                            \
        }                                                                                          \
        catch (...)                                                                                \
        {                                                                                          \
        }                                                                                          \
        if (!ok_)                                                                                  \
            mini_test::fail(__FILE__, __LINE__, "expected " #stmt " to throw " #type);            \
    } while (0)
#define EXPECT_ANY_THROW(stmt)                                                                     \
    do                                                                                             \
    {                                                                                              \
        bool ok_ = false;                                                                          \
        try                                                                                        \
        {                                                                                          \
            stmt;                                                                                  \
        }                                                                                          \
        catch (...)                                                                                \
        {                                                                                          \
            ok_ = true;                                                                            \
        }                                                                                          \
        if (!ok_)                                                                                  \
            mini_test::fail(__FILE__, __LINE__, "expected " #stmt " to throw");                    \
    } while (0)
#define EXPECT_NO_THROW(stmt)                                                                      \
    do                                                                                             \
    {                                                                                              \
        try                                                                                        \
        {                                                                                          \
            stmt;                                                                                  \
        }                                                                                          \
        catch (const std::exception& e_)                                                           \
        {                                                                                          \
            mini_test::fail(__FILE__, __LINE__, std::string("unexpected exception: ") + e_.what()); \
        }                                                                                          \
    } while (0)
