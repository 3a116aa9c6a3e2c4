// Error macros with Deep8's names and exception types (deep8/include/basic/Exception.h:6-30):
// argument / shape / dtype / device mismatches raise std::invalid_argument, everything else
// std::runtime_error; the text is "file:line: message.".  D8_CHECK converts a non-zero code of
// the C ABI into the runtime_error Deep8's CUDA_CHECK raises (basic/GPUException.h:15-24).
#ifndef DEEP8_HOST_EXCEPTION_H
#define DEEP8_HOST_EXCEPTION_H

#include <sstream>
#include <stdexcept>
#include <string>

namespace Deep8 {

template <typename E>
[[noreturn]] inline void raise(const char *file, int line, const std::string &message) {
    std::ostringstream text;
    text << file << ":" << line << ": " << message << ".";
    throw E(text.str());
}

}  // namespace Deep8

#define DEEP8_MESSAGE(message) (static_cast<std::ostringstream &>(std::ostringstream().flush() << message).str())

#define DEEP8_RUNTIME_ERROR(message) ::Deep8::raise<std::runtime_error>(__FILE__, __LINE__, DEEP8_MESSAGE(message))

#define DEEP8_ASSERT(condition, message) \
    if (!(condition)) ::Deep8::raise<std::runtime_error>(__FILE__, __LINE__, DEEP8_MESSAGE(message))

#define DEEP8_ARGUMENT_CHECK(condition, message) \
    if (!(condition)) ::Deep8::raise<std::invalid_argument>(__FILE__, __LINE__, DEEP8_MESSAGE(message))

// a call into libdeep8_hip.so
#define D8_CHECK(call)                                                                                  \
    do {                                                                                                \
        int d8_rc_ = (call);                                                                            \
        if (d8_rc_ != 0)                                                                                \
            DEEP8_RUNTIME_ERROR("the HIP path get a error: " << #call << "," << d8_last_error()         \
                                                            << " (code " << d8_rc_ << ")");            \
    } while (0)

#endif
