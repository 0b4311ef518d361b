// small::Timer: start() / stop() / elapsed() in nanoseconds (reference include/small/utils/Timer.hpp:53-91, the
// CLOCK_MONOTONIC variant).  Layer calls on this platform are asynchronous, so both start() and stop() first
// wait for the calling thread's stream: the interval then covers exactly the device work issued between them,
// which keeps the reference's "timer around the layer calls" protocol meaningful.
#pragma once

#include <time.h>

#include "../Buffer.hpp"

namespace small
{

class Timer
{
public:
    using TimeType = timespec;

    Timer() : start_time(), stop_time() {}

    TimeType start()
    {
        synchronize();
        clock_gettime(CLOCK_MONOTONIC, &start_time);
        return start_time;
    }

    TimeType stop()
    {
        synchronize();
        clock_gettime(CLOCK_MONOTONIC, &stop_time);
        return stop_time;
    }

    // nanoseconds between the last start() and stop()
    double elapsed() const
    {
        return (double)(stop_time.tv_sec - start_time.tv_sec) * 1.0e9 + (double)(stop_time.tv_nsec - start_time.tv_nsec);
    }

private:
    TimeType start_time, stop_time;
};

} // namespace small
