// Runs one variant of one call under an event timer and keeps the timing log the planner
// reads (reference src/methods/executor.h).
#pragma once
#include <timer_bank.h>
#include <workspace.h>

#include <map>
#include <stdexcept>

namespace rtat {

template <typename Params, typename Key, typename Opts>
class Executor {
 public:
  typedef Params Params_T;
  typedef Key Key_T;
  typedef Opts Opts_T;

  Executor() = default;
  virtual ~Executor() = default;

  // Enqueue `opts`' tree for `params` on stream s, bracketed by events; the timer joins the
  // log of (Key(params), opts) unless that log is full.  The first call warms the kernels up.
  virtual void execute(Params params, Opts opts, Workspace space, Stream s,
                       Device_Timer::Mode sync = Device_Timer::ASYNCHRONOUS) {
    if (!warm) {
      warmup(params, opts, s);
      warm = true;
    }
    Timer_Bank& bank = timer_log[Key(params)][opts];
    if (bank.size() >= log_size_limit && sync == Device_Timer::ASYNCHRONOUS) {
      // The log of this variant is full: nothing would keep the timing, so the call is not
      // bracketed by events at all (they cost several microseconds of stream time each,
      // which is as much as a small problem's kernel).
      internal_execute(params, opts, space, s);
      return;
    }
    Device_Timer timer([&](const Stream& str) { internal_execute(params, opts, space, str); }, s,
                       sync);
    if (bank.size() < log_size_limit) bank.append(timer);
  }

  std::map<Key, std::map<Opts, Timer_Bank>>& get_timings() { return timer_log; }
  std::map<Opts, Timer_Bank>& get_timings(Key key) { return timer_log[key]; }

  // Bytes of scratch the variant's tree needs for this call.
  virtual size_t calculate_workspace(Params params, Opts opts) {
    return opts.form_operation(params)->workspace_req_bytes();
  }

 protected:
  // All device work of one call goes to the stream of params.handle, which the caller keeps
  // equal to `s` (the reference leaves `s` unused, executor.h:47).
  virtual void internal_execute(Params params, Opts opts, Workspace space, Stream) {
    auto operation = opts.form_operation(params);
    if (operation->workspace_req_bytes() > space.size<char>())
      throw std::runtime_error("internal_execute: Insufficient workspace");
    operation->execute(params.handle, Workspace(), space);
  }
  virtual void warmup(Params, Opts, Stream) = 0;

  std::map<Key, std::map<Opts, Timer_Bank>> timer_log;
  const size_t log_size_limit = 100;
  bool warm = false;
};

}  // namespace rtat
