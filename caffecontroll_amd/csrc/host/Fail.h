// What the host layer does when a driver call fails or a bridge is built on inconsistent layers.
//
// A C++ caller that drops HIPDriver in next to CPUDriver gets the reference's behaviour
// (src/sched/DeviceDriver.h:48-51: members return void, errors are asserts): the message is
// printed and the process ends.  The C entry points over the bridges (include/cct_bridge.h:
// cct_conv_bridge_*, cct_net_*) cannot let their caller's process die on a HIP error in the
// middle of an iteration; they open an ErrorsAsExceptions scope, under which the same failures
// throw HostError instead, and turn what they catch into a return code plus cct_hip_last_error().
#pragma once
#include <cstdio>
#include <cstdlib>
#include <stdexcept>
#include <string>

namespace cct {

struct HostError : std::runtime_error {
  explicit HostError(const std::string &what) : std::runtime_error(what) {}
};

inline bool &errors_throw() {
  static thread_local bool on = false;
  return on;
}

// Per host thread, nestable; the previous policy returns when the scope ends.
struct ErrorsAsExceptions {
  bool prev;
  ErrorsAsExceptions() : prev(errors_throw()) { errors_throw() = true; }
  ~ErrorsAsExceptions() { errors_throw() = prev; }
  ErrorsAsExceptions(const ErrorsAsExceptions &) = delete;
  ErrorsAsExceptions &operator=(const ErrorsAsExceptions &) = delete;
};

[[noreturn]] inline void host_fail(const std::string &msg) {
  if (errors_throw()) throw HostError(msg);
  std::fprintf(stderr, "%s\n", msg.c_str());
  std::abort();
}

}  // namespace cct
