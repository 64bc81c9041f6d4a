// Runs one variant of one call and keeps, per problem key and variant, the log of event
// timings the planner ranks variants by (reference src/methods/executor.h:8-59).
//
// Differences from the reference's executor, none visible in results:
//   * a call whose log is already full is not bracketed by events at all — an event pair
//     costs several microseconds of stream time, as much as a small problem's kernel;
//   * a workspace that is too small raises std::runtime_error (the reference throws a string
//     literal, :49);
//   * the routine executors are one template over a warm-up function instead of one class
//     body per routine.
#pragma once
#include <timer_bank.h>
#include <workspace.h>

#include <map>
#include <stdexcept>

namespace rtat {

template <typename Params, typename Key, typename Opts>
class Executor {
 public:
  using Params_T = Params;
  using Key_T = Key;
  using Opts_T = Opts;
  using Variant_Log = std::map<Opts, Timer_Bank>;

  Executor() = default;
  virtual ~Executor() = default;

  // Enqueue the tree of variant `opts` for `params` on the stream.  While the variant's log
  // has room the work is timed and the timer joins the log; the very first call warms the
  // kernels up before anything is timed.
  virtual void execute(Params params, Opts opts, Workspace space, Stream s,
                       Device_Timer::Mode sync = Device_Timer::ASYNCHRONOUS) {
    if (!warm) {
      warmup(params, opts, s);
      warm = true;
    }
    Timer_Bank& bank = timer_log[Key(params)][opts];
    const bool room = bank.size() < log_size_limit;
    if (!room && sync == Device_Timer::ASYNCHRONOUS) {
      internal_execute(params, opts, space, s);
      return;
    }
    Device_Timer timer([&](const Stream& on) { internal_execute(params, opts, space, on); }, s,
                       sync);
    if (room) bank.append(timer);
  }

  std::map<Key, Variant_Log>& get_timings() { return timer_log; }
  Variant_Log& get_timings(Key key) { return timer_log[key]; }

  // Bytes of scratch the variant's tree needs for this call.
  virtual size_t calculate_workspace(Params params, Opts opts) {
    return opts.form_operation(params)->workspace_req_bytes();
  }

 protected:
  // All device work goes to the stream of params.handle, which the caller keeps equal to the
  // stream argument (unused here, as in the reference, :47).
  virtual void internal_execute(Params params, Opts opts, Workspace space, Stream) {
    auto tree = opts.form_operation(params);
    if (tree->workspace_req_bytes() > space.size<char>())
      throw std::runtime_error("internal_execute: Insufficient workspace");
    tree->execute(params.handle, Workspace(), space);
  }
  virtual void warmup(Params, Opts, Stream) = 0;

  std::map<Key, Variant_Log> timer_log;
  const size_t log_size_limit = 100;
  bool warm = false;
};

// An executor whose warm-up is `Warm(handle)`: the GEMM / SYRK / TRSM executors are aliases
// of this with their routine's warm-up function.
template <typename Params, typename Key, typename Opts, void (*Warm)(gpu::blasHandle_t)>
class Warmed_Executor : public Executor<Params, Key, Opts> {
 protected:
  void warmup(Params params, Opts, Stream) override { Warm(params.handle); }
};

}  // namespace rtat
