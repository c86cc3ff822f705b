// Argument-check convention of the library: a failed check prints one line on stderr, latches a
// process-wide flag and lets the caller return early; nothing aborts and nothing throws.
// Message format and stickiness follow reference src/utils/check.h:36-56 and src/utils/check.cpp:16.
#pragma once
#include <sstream>
#include <string>

namespace kutacc {
extern bool kutacc_check_err_set;

namespace internal {
void emit_check_failure(const char *func, const char *file, int line, const std::string &detail);

template <typename... Parts>
inline std::string join_parts(Parts &&...parts)
{
    std::ostringstream os;
    (void)std::initializer_list<int>{((os << parts), 0)...};
    return os.str();
}
} // namespace internal
} // namespace kutacc

#define KUTACC_CHECK(cond, ...)                                                                  \
    do {                                                                                         \
        if (__builtin_expect(!(cond), 0)) {                                                      \
            ::kutacc::internal::emit_check_failure(__func__, __FILE__, __LINE__,                 \
                                                   ::kutacc::internal::join_parts(__VA_ARGS__)); \
        }                                                                                        \
    } while (0)

#define KUTACC_FAILED() (::kutacc::kutacc_check_err_set)
