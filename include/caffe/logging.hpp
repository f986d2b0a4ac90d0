/*
 * Logging and checks for the Mini-Caffe host API.
 *
 * Same contract as the reference's dmlc-style macros (reference
 * include/caffe/logging.hpp:115-141,200-213): LOG(INFO|WARNING|ERROR) write a
 * line to stderr, LOG(FATAL) and every failed CHECK* throw caffe::Error (a
 * std::runtime_error) carrying "file:line: message".  The C ABI turns that
 * exception into a -1 return code plus CaffeGetLastError().
 */
#ifndef CAFFE_LOGGING_HPP_
#define CAFFE_LOGGING_HPP_

#include <iostream>
#include <sstream>
#include <stdexcept>
#include <string>

namespace caffe {

struct Error : public std::runtime_error {
  explicit Error(const std::string& s) : std::runtime_error(s) {}
};

namespace log_detail {

class Line {
 public:
  Line(const char* file, int line, const char* level, bool fatal) : fatal_(fatal) {
    if (fatal) {
      os_ << file << ":" << line << ": ";
    } else {
      os_ << "[" << level << "] " << file << ":" << line << ": ";
    }
  }
  // Throwing from a destructor is deliberate (and the reference does the same):
  // the message is complete only once the full << chain has run.
  ~Line() noexcept(false) {
    if (fatal_) throw Error(os_.str());
    std::cerr << os_.str() << std::endl;
  }
  std::ostringstream& stream() { return os_; }

 private:
  std::ostringstream os_;
  bool fatal_;
};

struct Voidify {
  void operator&(std::ostream&) {}
};

}  // namespace log_detail
}  // namespace caffe

#define CAFFE_LOG_INFO ::caffe::log_detail::Line(__FILE__, __LINE__, "INFO", false)
#define CAFFE_LOG_WARNING ::caffe::log_detail::Line(__FILE__, __LINE__, "WARNING", false)
#define CAFFE_LOG_ERROR ::caffe::log_detail::Line(__FILE__, __LINE__, "ERROR", false)
#define CAFFE_LOG_FATAL ::caffe::log_detail::Line(__FILE__, __LINE__, "FATAL", true)
#define LOG(severity) CAFFE_LOG_##severity.stream()

#define CHECK(cond) \
  if (!(cond)) CAFFE_LOG_FATAL.stream() << "Check failed: " #cond << ' '
#define CAFFE_CHECK_OP(a, b, op)                                                       \
  if (!((a)op(b)))                                                                     \
  CAFFE_LOG_FATAL.stream() << "Check failed: " #a " " #op " " #b " (" << (a) << " vs. " \
                           << (b) << ") "
#define CHECK_EQ(a, b) CAFFE_CHECK_OP(a, b, ==)
#define CHECK_NE(a, b) CAFFE_CHECK_OP(a, b, !=)
#define CHECK_LT(a, b) CAFFE_CHECK_OP(a, b, <)
#define CHECK_LE(a, b) CAFFE_CHECK_OP(a, b, <=)
#define CHECK_GT(a, b) CAFFE_CHECK_OP(a, b, >)
#define CHECK_GE(a, b) CAFFE_CHECK_OP(a, b, >=)
#define CHECK_NOTNULL(p) \
  ((p) == nullptr ? (CAFFE_LOG_FATAL.stream() << "Check notnull: " #p << ' ', (p)) : (p))

#ifdef NDEBUG
#define DLOG(severity) \
  true ? (void)0 : ::caffe::log_detail::Voidify() & LOG(severity)
#else
#define DLOG(severity) LOG(severity)
#endif

#endif  // CAFFE_LOGGING_HPP_
