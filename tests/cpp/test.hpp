// Minimal test registry for the host-layer tests: TEST_CASE(name) { EXPECT(cond); ... }.
// `prog` runs every case, `prog name...` the named ones, `prog --list` prints the names.
#ifndef TESTS_CPP_TEST_HPP
#define TESTS_CPP_TEST_HPP

#include <cstring>
#include <exception>
#include <functional>
#include <iostream>
#include <string>
#include <vector>

namespace test {

struct failure : std::exception
{
    std::string msg;
    explicit failure(std::string m) : msg(std::move(m)) {}
    const char* what() const noexcept override { return msg.c_str(); }
};

inline std::vector<std::pair<std::string, std::function<void()>>>& cases()
{
    static std::vector<std::pair<std::string, std::function<void()>>> c;
    return c;
}

struct registrar
{
    registrar(const char* name, std::function<void()> f) { cases().emplace_back(name, std::move(f)); }
};

template <class F>
bool throws(F f)
{
    try
    {
        f();
    }
    catch(const std::exception&)
    {
        return true;
    }
    return false;
}

inline int run(int argc, char** argv)
{
    std::vector<std::string> only;
    for(int i = 1; i < argc; i++)
    {
        if(std::strcmp(argv[i], "--list") == 0)
        {
            for(auto& c : cases())
                std::cout << c.first << "\n";
            return 0;
        }
        only.emplace_back(argv[i]);
    }
    int failed = 0;
    int ran    = 0;
    for(auto& c : cases())
    {
        if(not only.empty() and std::find(only.begin(), only.end(), c.first) == only.end())
            continue;
        ran++;
        std::cout << "[ RUN  ] " << c.first << std::endl;
        try
        {
            c.second();
            std::cout << "[  OK  ] " << c.first << std::endl;
        }
        catch(const std::exception& e)
        {
            failed++;
            std::cout << "[ FAIL ] " << c.first << ": " << e.what() << std::endl;
        }
    }
    std::cout << ran - failed << " passed, " << failed << " failed" << std::endl;
    if(ran == 0)
        return 2;
    return failed == 0 ? 0 : 1;
}

} // namespace test

#define TEST_CASE(name)                                             \
    static void name();                                             \
    static const test::registrar test_registrar_##name{#name, name}; \
    static void name()

#define EXPECT(...)                                                                          \
    do                                                                                       \
    {                                                                                        \
        if(not(__VA_ARGS__))                                                                 \
            throw test::failure(std::string(__FILE__) + ":" + std::to_string(__LINE__) +     \
                                ": EXPECT(" #__VA_ARGS__ ") failed");                        \
    } while(0)

#endif
