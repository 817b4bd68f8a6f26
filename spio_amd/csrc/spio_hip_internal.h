// Helpers shared by the translation units of libspio_hip.so.  Not part of the
// C ABI: these symbols have hidden visibility.
#ifndef SPIO_HIP_INTERNAL_H
#define SPIO_HIP_INTERNAL_H

#define SPIO_HIP_HIDDEN __attribute__((visibility("hidden")))

// Stores `text` as the calling thread's last error and returns `code`.
SPIO_HIP_HIDDEN int spio_hip_set_error(int code, const char* text);

// The geometry and argument-count checks of spio_hip_launch; 0 when they pass.
SPIO_HIP_HIDDEN int spio_hip_check_launch_args(void* function, unsigned gx, unsigned gy, unsigned gz,
                                               unsigned bx, unsigned by, unsigned bz, int num_params);

#endif  // SPIO_HIP_INTERNAL_H
