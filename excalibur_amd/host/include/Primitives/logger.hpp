// glog-style logging with the reference's failure policy: a FATAL message prints and terminates
// the process; nothing throws (reference include/Primitives/logger.hpp:101-118,162-204 and the
// statement of that policy in include/Primitives/memory.hpp:27-31).
#pragma once
#include <cstdlib>
#include <exception>
#include <iostream>
#include <sstream>

namespace glasssix {
enum log_severity { INFO = 0, WARNING = 1, ERROR = 2, FATAL = 3 };

class log_message {
public:
    log_message(const char* file, int line, log_severity sev) : sev_(sev) {
        static const char* names[] = {"INFO", "WARNING", "ERROR", "FATAL"};
        ss_ << "[" << file << ":" << line << "][" << names[sev] << "] ";
    }
    ~log_message() {
        std::cerr << ss_.str() << std::endl;
        if (sev_ == FATAL) std::terminate();
    }
    std::ostream& stream() { return ss_; }

private:
    std::ostringstream ss_;
    log_severity sev_;
};
}  // namespace glasssix

#define LOG(sev) ::glasssix::log_message(__FILE__, __LINE__, ::glasssix::sev).stream()
#define CHECK(cond) \
    if (!(cond)) LOG(FATAL) << "Check failed: " #cond " "
#define CHECK_OP(a, b, op) \
    if (!((a)op(b))) LOG(FATAL) << "Check failed: " #a " " #op " " #b " (" << (a) << " vs " << (b) << ") "
#define CHECK_EQ(a, b) CHECK_OP(a, b, ==)
#define CHECK_NE(a, b) CHECK_OP(a, b, !=)
#define CHECK_LE(a, b) CHECK_OP(a, b, <=)
#define CHECK_LT(a, b) CHECK_OP(a, b, <)
#define CHECK_GE(a, b) CHECK_OP(a, b, >=)
#define CHECK_GT(a, b) CHECK_OP(a, b, >)
#define NOT_IMPLEMENTED LOG(FATAL) << "Not Implemented Yet"
#define NO_GPU LOG(FATAL) << "This operator has no device code."
#define NO_CPU LOG(FATAL) << "This backend computes on an MI355X only: construct the pipeline with device >= 0."
#define DISABLE_COPY_AND_ASSIGN(classname) \
    classname(const classname&) = delete;  \
    classname& operator=(const classname&) = delete
