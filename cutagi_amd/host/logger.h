// Error convention of the host classes: LOG(LogLevel::ERROR, msg) prints the
// message and throws std::runtime_error, like the reference's logger
// (src/custom_logger.cpp:46-61); lower levels only print.
#pragma once
#include <iostream>
#include <stdexcept>
#include <string>

namespace tagi_host {

enum class LogLevel { DEBUG, INFO, WARNING, ERROR };

inline void log_message(LogLevel level, const char *file, int line, const std::string &msg) {
    static const char *names[] = {"[DEBUG]", "[INFO]", "[WARNING]", "[ERROR]"};
    if (level == LogLevel::ERROR) {
        std::cerr << names[(int)level] << " " << file << ":" << line << " - " << msg << std::endl;
        throw std::runtime_error(msg);
    }
    std::cout << names[(int)level] << " - " << msg << std::endl;
}

}  // namespace tagi_host

#define LOG(level, msg) ::tagi_host::log_message(level, __FILE__, __LINE__, msg)

// A failed HIP runtime or C-ABI call becomes LOG(ERROR), i.e. an exception.
#define HIP_OK(expr)                                                                  \
    do {                                                                              \
        hipError_t _e = (expr);                                                       \
        if (_e != hipSuccess)                                                         \
            LOG(::tagi_host::LogLevel::ERROR, std::string(#expr) + ": " + hipGetErrorString(_e)); \
    } while (0)
#define TAGI_OK_OR_THROW(expr)                                                        \
    do {                                                                              \
        int _rc = (expr);                                                             \
        if (_rc != TAGI_OK)                                                           \
            LOG(::tagi_host::LogLevel::ERROR, std::string(#expr) + ": " + tagi_hip_error_string(_rc)); \
    } while (0)
