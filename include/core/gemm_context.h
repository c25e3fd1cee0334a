// Context argument of the linear operators. The reference passes a cuBLASLt handle
// (include/core/cublas_context.h:16-60); the contractions here are this library's own kernels and
// need no handle, so the class only records the device it was created for.
#pragma once

class GemmContext {
public:
    explicit GemmContext(int device_index = 0) : device_index_(device_index) {}
    [[nodiscard]] int device_index() const noexcept { return device_index_; }

private:
    int device_index_;
};
