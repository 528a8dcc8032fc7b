/*
 * Minimal glog-style checks and logging for the mshadow API.
 *
 * Behaviour follows mshadow/logging.h:62-229 of the reference: CHECK(x) << "msg"
 * evaluates the message only on failure; LOG(FATAL) aborts the process unless
 * DMLC_LOG_FATAL_THROW is 1, in which case it throws dmlc::Error (:183-216); other
 * severities print "[HH:MM:SS] file:line: msg" to stderr (:158-181).
 */
#ifndef MSHADOW_LOGGING_H_
#define MSHADOW_LOGGING_H_

#include <cstdio>
#include <cstdlib>
#include <ctime>
#include <iostream>
#include <sstream>
#include <stdexcept>
#include <string>

#ifndef DMLC_LOG_FATAL_THROW
#define DMLC_LOG_FATAL_THROW 0
#endif

namespace dmlc {

/*! \brief exception thrown by a failed CHECK / LOG(FATAL) when DMLC_LOG_FATAL_THROW == 1 */
struct Error : public std::runtime_error {
  explicit Error(const std::string &s) : std::runtime_error(s) {}
};

namespace logging_detail {
inline void Stamp(std::ostream &os, const char *file, int line) {
  time_t now = time(NULL);
  struct tm tmv;
  localtime_r(&now, &tmv);
  char buf[16];
  snprintf(buf, sizeof(buf), "%02d:%02d:%02d", tmv.tm_hour, tmv.tm_min, tmv.tm_sec);
  os << '[' << buf << "] " << file << ':' << line << ": ";
}
}  // namespace logging_detail

/*! \brief one line written to stderr when the object goes out of scope */
class LogMessage {
 public:
  LogMessage(const char *file, int line) { logging_detail::Stamp(buf_, file, line); }
  ~LogMessage() { std::cerr << buf_.str() << '\n'; }
  std::ostream &stream() { return buf_; }

 private:
  std::ostringstream buf_;
  LogMessage(const LogMessage &);
  void operator=(const LogMessage &);
};

/*! \brief fatal message: abort, or throw dmlc::Error */
class LogMessageFatal {
 public:
  LogMessageFatal(const char *file, int line) { logging_detail::Stamp(buf_, file, line); }
  std::ostream &stream() { return buf_; }
#if DMLC_LOG_FATAL_THROW
  ~LogMessageFatal() noexcept(false) { throw Error(buf_.str()); }
#else
  ~LogMessageFatal() {
    std::cerr << buf_.str() << '\n';
    abort();
  }
#endif

 private:
  std::ostringstream buf_;
  LogMessageFatal(const LogMessageFatal &);
  void operator=(const LogMessageFatal &);
};

/*! \brief swallows the stream expression so that CHECK can be used as a statement */
struct LogMessageVoidify {
  void operator&(std::ostream &) {}
};

}  // namespace dmlc

#define LOG_INFO dmlc::LogMessage(__FILE__, __LINE__)
#define LOG_ERROR LOG_INFO
#define LOG_WARNING LOG_INFO
#define LOG_FATAL dmlc::LogMessageFatal(__FILE__, __LINE__)
#define LOG_QFATAL LOG_FATAL
#define LOG(severity) LOG_##severity.stream()
#define LG LOG_INFO.stream()
#define LOG_IF(severity, condition) \
  !(condition) ? (void)0 : dmlc::LogMessageVoidify() & LOG(severity)

#define CHECK(x) \
  if (!(x)) dmlc::LogMessageFatal(__FILE__, __LINE__).stream() << "Check failed: " #x << ' '
#define CHECK_LT(x, y) CHECK((x) < (y))
#define CHECK_GT(x, y) CHECK((x) > (y))
#define CHECK_LE(x, y) CHECK((x) <= (y))
#define CHECK_GE(x, y) CHECK((x) >= (y))
#define CHECK_EQ(x, y) CHECK((x) == (y))
#define CHECK_NE(x, y) CHECK((x) != (y))
#define CHECK_NOTNULL(x) \
  ((x) == NULL ? LOG(FATAL) << "Check  notnull: " #x << ' ', (x) : (x))

#ifdef NDEBUG
#define DCHECK(x) while (false) CHECK(x)
#define DCHECK_LT(x, y) while (false) CHECK((x) < (y))
#define DCHECK_GT(x, y) while (false) CHECK((x) > (y))
#define DCHECK_LE(x, y) while (false) CHECK((x) <= (y))
#define DCHECK_GE(x, y) while (false) CHECK((x) >= (y))
#define DCHECK_EQ(x, y) while (false) CHECK((x) == (y))
#define DCHECK_NE(x, y) while (false) CHECK((x) != (y))
#else
#define DCHECK(x) CHECK(x)
#define DCHECK_LT(x, y) CHECK((x) < (y))
#define DCHECK_GT(x, y) CHECK((x) > (y))
#define DCHECK_LE(x, y) CHECK((x) <= (y))
#define DCHECK_GE(x, y) CHECK((x) >= (y))
#define DCHECK_EQ(x, y) CHECK((x) == (y))
#define DCHECK_NE(x, y) CHECK((x) != (y))
#endif

#endif  // MSHADOW_LOGGING_H_
