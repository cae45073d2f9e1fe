// The streaming 16-bit softmax for f16 (see rt_softmax_stream.h).
#include "rt_softmax_stream.h"

int rt_softmax_stream_f16(rt_device* dev, const void* x, const void* mask, uint64_t period, void* y, uint64_t rows, uint32_t cols, bool* done) {
    return launch_stream16<half_t>(dev, x, mask, period, y, rows, cols, done);
}
