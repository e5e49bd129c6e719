// One-file logger: HT_LOG_{TRACE,DEBUG,INFO,WARN,ERROR} << ...; the level comes
// from the environment variable HETU_INTERNAL_LOG_LEVEL (hetu/common/logging.cc:14
// of the reference), default WARN.
#pragma once

#include <cstdlib>
#include <cstring>
#include <iostream>
#include <sstream>

namespace hetu {
namespace logging {

enum Level { TRACE = 0, DEBUG, INFO, WARN, ERROR, FATAL };

inline Level current_level() {
  static const Level level = [] {
    const char* e = std::getenv("HETU_INTERNAL_LOG_LEVEL");
    if (!e) return WARN;
    static const char* const names[] = {"TRACE", "DEBUG", "INFO", "WARN", "ERROR", "FATAL"};
    for (int i = 0; i < 6; ++i)
      if (strcasecmp(e, names[i]) == 0) return static_cast<Level>(i);
    return WARN;
  }();
  return level;
}

class Line {
 public:
  Line(Level l, const char* tag) : _on(l >= current_level()) {
    if (_on) _ss << "[" << tag << "] ";
  }
  ~Line() {
    if (_on) std::cerr << _ss.str() << std::endl;
  }
  template <typename V>
  Line& operator<<(const V& v) {
    if (_on) _ss << v;
    return *this;
  }

 private:
  bool _on;
  std::ostringstream _ss;
};

} // namespace logging
} // namespace hetu

#define HT_LOG_TRACE ::hetu::logging::Line(::hetu::logging::TRACE, "TRACE")
#define HT_LOG_DEBUG ::hetu::logging::Line(::hetu::logging::DEBUG, "DEBUG")
#define HT_LOG_INFO ::hetu::logging::Line(::hetu::logging::INFO, "INFO")
#define HT_LOG_WARN ::hetu::logging::Line(::hetu::logging::WARN, "WARN")
#define HT_LOG_ERROR ::hetu::logging::Line(::hetu::logging::ERROR, "ERROR")
