// Host timers with the reference's two protocols (lib/wtime.h:5-35):
//   wtime(times, action, prep)     mean of per-iteration times; the caller's
//                                  action includes its own synchronisation
//   wtime_new(times, action, end)  times back-to-back launches, end() once
// Both return microseconds per iteration.
#pragma once
#include <chrono>

template <typename Action, typename Prep> double wtime(int times, Action action, Prep prep) {
    using clock = std::chrono::steady_clock;
    double total_us = 0.0;
    for (int i = 0; i < times; i++) {
        prep();
        const auto t0 = clock::now();
        action();
        total_us += std::chrono::duration<double, std::micro>(clock::now() - t0).count();
    }
    return total_us / times;
}

template <typename Action, typename End> double wtime_new(int times, Action action, End end) {
    using clock = std::chrono::steady_clock;
    const auto t0 = clock::now();
    for (int i = 0; i < times; i++) action();
    end();
    return std::chrono::duration<double, std::micro>(clock::now() - t0).count() / times;
}
