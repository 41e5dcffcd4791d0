// Event timers for kernels launched through this library: the classes include/timer.h:6-79 of the
// reference declares (KernelTimer, KernelTimerScoped, Timer) with the same members, given the bodies the
// reference never defines.  Header-only, HIP events on the caller's stream, nothing here blocks until
// synchronize() is called.
//
//   std::vector<std::shared_ptr<KernelTimer>> timers;
//   float ms, gflops;
//   { KernelTimerScoped t(timers, 2 * M * N * K, &ms, &gflops, stream);  launch(...); }
//   for (auto &t : timers) t->synchronize();      // fills ms and gflops, runs the callback once
#pragma once
#include "common.h"

#include <chrono>
#include <memory>
#include <stdexcept>
#include <string>
#include <vector>

typedef void (*TimerCompletionCallback)(float elapsed_time, size_t calc_ops, float *time_ptr, float *gflops_ptr,
                                        void *user_data);

class KernelTimer {
  private:
    size_t calc_ops;
    hipEvent_t start, stop;
    float *time_ptr;
    float *gflops_ptr;
    void *user_data;
    TimerCompletionCallback callback;
    bool callback_executed;
    bool started, stopped;

    static void must(hipError_t e, const char *what) {
        if (e != hipSuccess) throw std::runtime_error(std::string("KernelTimer: ") + what + ": " + hipGetErrorString(e));
    }

  public:
    // calc_ops: operations between start and stop (2*M*N*K for a GEMM); time in ms and the rate in
    // GFLOP/s are written through the two pointers (either may be null) when the timer completes
    KernelTimer(size_t calc_ops, float *time, float *gflops)
        : calc_ops(calc_ops), start(nullptr), stop(nullptr), time_ptr(time), gflops_ptr(gflops), user_data(nullptr),
          callback(nullptr), callback_executed(false), started(false), stopped(false) {
        must(hipEventCreate(&start), "hipEventCreate");
        must(hipEventCreate(&stop), "hipEventCreate");
    }
    KernelTimer(const KernelTimer &) = delete;
    KernelTimer &operator=(const KernelTimer &) = delete;

    void start_timer(hipStream_t stream = 0) {
        must(hipEventRecord(start, stream), "hipEventRecord(start)");
        started = true;
        stopped = callback_executed = false;
    }
    void stop_timer(hipStream_t stream = 0) {
        if (!started) throw std::logic_error("KernelTimer: stop_timer before start_timer");
        must(hipEventRecord(stop, stream), "hipEventRecord(stop)");
        stopped = true;
    }
    void set_callback(TimerCompletionCallback cb, void *data = nullptr) {
        callback = cb;
        user_data = data;
    }

    // Wait for the stop event, publish time and rate, and run the callback (once per start/stop pair)
    void synchronize() {
        if (!stopped) throw std::logic_error("KernelTimer: synchronize before stop_timer");
        must(hipEventSynchronize(stop), "hipEventSynchronize");
        if (callback_executed) return;
        float ms = 0.f;
        must(hipEventElapsedTime(&ms, start, stop), "hipEventElapsedTime");
        execute_callback(ms);
    }

    hipEvent_t get_start_event() const { return start; }
    hipEvent_t get_stop_event() const { return stop; }
    size_t get_calc_ops() const { return calc_ops; }
    float *get_time_ptr() const { return time_ptr; }
    float *get_gflops_ptr() const { return gflops_ptr; }
    void execute_callback(float elapsed_time) {
        const float gflops = elapsed_time > 0.f ? (float)((double)calc_ops / ((double)elapsed_time * 1e6)) : 0.f;
        if (time_ptr) *time_ptr = elapsed_time;
        if (gflops_ptr) *gflops_ptr = gflops;
        if (callback) callback(elapsed_time, calc_ops, time_ptr, gflops_ptr, user_data);
        callback_executed = true;
    }
    void set_callback_executed(bool executed) { callback_executed = executed; }
    bool is_callback_executed() const { return callback_executed; }

    ~KernelTimer() {
        if (start) (void)hipEventDestroy(start);
        if (stop) (void)hipEventDestroy(stop);
    }
};

// Starts a timer on construction and stops it when the scope ends; the timer is kept in `timers` so the
// caller can synchronize() all of them after the launches have been queued.
class KernelTimerScoped {
  private:
    std::shared_ptr<KernelTimer> timer;
    hipStream_t stream;

  public:
    KernelTimerScoped(std::vector<std::shared_ptr<KernelTimer>> &timers, size_t calc_ops, float *time, float *gflops,
                      hipStream_t stream = 0)
        : timer(std::make_shared<KernelTimer>(calc_ops, time, gflops)), stream(stream) {
        timers.push_back(timer);
        timer->start_timer(stream);
    }
    KernelTimerScoped(const KernelTimerScoped &) = delete;
    KernelTimerScoped &operator=(const KernelTimerScoped &) = delete;

    ~KernelTimerScoped() {
        try { timer->stop_timer(stream); } catch (...) {}
    }
};

// Host wall clock in milliseconds
class Timer {
  public:
    Timer() : start_(std::chrono::steady_clock::now()) {}
    double elapsed() const {
        return std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - start_).count();
    }
    void reset() { start_ = std::chrono::steady_clock::now(); }

  private:
    std::chrono::steady_clock::time_point start_;
};
