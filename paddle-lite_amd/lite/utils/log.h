// LOG / CHECK in the shape the reference's kernels and ops use them
// (lite/utils/log/logging.h).  FATAL throws lite::FatalError (the reference's
// LITE_WITH_EXCEPTION behaviour) so that host tests can observe it.
#pragma once

#include <iostream>
#include <sstream>
#include <stdexcept>
#include <string>

namespace paddle {
namespace lite {

struct FatalError : std::runtime_error {
  explicit FatalError(const std::string& what) : std::runtime_error(what) {}
};

namespace logging {

enum Severity { INFO = 0, WARNING = 1, ERROR = 2, FATAL = 3 };

class Message {
 public:
  Message(const char* file, int line, Severity s) : severity_(s) { stream_ << "[" << file << ":" << line << "] "; }
  ~Message() noexcept(false) {
    if (severity_ == FATAL) throw FatalError(stream_.str());
    if (severity_ >= WARNING) std::cerr << stream_.str() << std::endl;
  }
  std::ostream& stream() { return stream_; }

 private:
  std::ostringstream stream_;
  Severity severity_;
};

// Swallows the stream expression of a CHECK that holds.
struct Voidify {
  void operator&(std::ostream&) {}
};

}  // namespace logging
}  // namespace lite
}  // namespace paddle

#define LOG(severity) paddle::lite::logging::Message(__FILE__, __LINE__, paddle::lite::logging::severity).stream()
#define VLOG(level) \
  if (false) LOG(INFO)
#define CHECK(cond) \
  (cond) ? (void)0 : paddle::lite::logging::Voidify() & LOG(FATAL) << "Check failed: " #cond " "
#define CHECK_EQ(a, b) CHECK((a) == (b))
#define CHECK_NE(a, b) CHECK((a) != (b))
#define CHECK_GE(a, b) CHECK((a) >= (b))
#define CHECK_GT(a, b) CHECK((a) > (b))
#define CHECK_LE(a, b) CHECK((a) <= (b))
#define CHECK_LT(a, b) CHECK((a) < (b))
#define CHECK_OR_FALSE(cond) \
  if (!(cond)) return false
