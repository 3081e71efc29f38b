// Error convention of the Acrotensor API: every failed precondition throws std::runtime_error carrying
// "<file>:  <line>  <message>".  Mirrors the contract of the reference's util/Error.hpp:15-23
// (ACROBATIC_ASSERT with one or two arguments, acro::throw_error).
#ifndef ACRO_HIP_ERROR_HPP
#define ACRO_HIP_ERROR_HPP

#include <stdexcept>
#include <string>

namespace acro
{

[[noreturn]] inline void throw_error(const std::string &what)
{
    throw std::runtime_error(what);
}

namespace detail
{
inline std::string where(const char *file, int line)
{
    return std::string(file) + ":  " + std::to_string(line);
}
inline void fail(const char *file, int line)
{
    throw_error(where(file, line));
}
inline void fail(const char *file, int line, const std::string &msg)
{
    throw_error(where(file, line) + "  " + msg);
}
}  // namespace detail

}  // namespace acro

// ACROBATIC_ASSERT(cond) or ACROBATIC_ASSERT(cond, message)
#define ACROBATIC_ASSERT(EX, ...)                                        \
    do                                                                   \
    {                                                                    \
        if (!(EX)) ::acro::detail::fail(__FILE__, __LINE__, ##__VA_ARGS__); \
    } while (0)

#endif
