#include "timer.hpp"
#include <cstdio>

void Timer::start() { start_time = std::chrono::high_resolution_clock::now(); }

double Timer::elapsed() {
    const auto now = std::chrono::high_resolution_clock::now();
    return (double)std::chrono::duration_cast<std::chrono::microseconds>(now - start_time).count() / 1e6;
}

double Timer::stop(const std::string& label) {
    const double seconds = elapsed();
    std::printf("\033[35m[Timing]\033[0m %s in: %.3f ms\n", label.c_str(), seconds * 1000.0);
    return seconds;
}
