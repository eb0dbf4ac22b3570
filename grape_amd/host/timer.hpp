// Wall-clock timer of the reference's drivers (include/timer.cuh:5-14, src/timer.cu).
#pragma once
#include <chrono>
#include <string>

class Timer {
public:
    void start();
    // prints "[Timing] <label> in: <ms> ms" and returns the elapsed time in SECONDS
    double stop(const std::string& label = "Code block executed");
    double elapsed();

private:
    std::chrono::high_resolution_clock::time_point start_time;
};
