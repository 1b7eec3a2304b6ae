// What the HIP binding of EDDL's gpu_* seam offers beyond the functions EDDL itself declares
// (include/eddl/hardware/gpu/gpu_tensor.h, gpu_hw.h, nn/gpu_tensor_nn.h).  Nothing in EDDL needs these; they are for
// callers that want to drop the wait after every call, or fix the seed of device-side initialisation.
#ifndef EDDL_HIP_BACKEND_H
#define EDDL_HIP_BACKEND_H

// A C ABI return code of libeddlhip.so -> EDDL's exceptions: a rejected argument becomes msg(text, where)
// (src/utils.cpp:57-67), any other failure std::runtime_error("[HIP ERROR]: ...") in the manner of check_cuda
// (src/hardware/gpu/gpu_tensor.cu:103-112).
void gpu_check(int rc, const char *where);

// Every gpu_* call returns with its work done, as EDDL's CUDA wrappers do (cudaDeviceSynchronize after each
// launch), until gpu_set_synchronous(false): then compute calls return once queued, in order, on the device's
// stream; copies to the host still wait for everything queued before them.
void gpu_set_synchronous(bool on);
bool gpu_get_synchronous();
void gpu_synchronize(int gpu_device);

// Random fills on a device are numbered from a fixed base seed, 1234 as in the CUDA backend's generator
// (src/hardware/gpu/gpu_tensor.cu:179-185); this sets another base and restarts the numbering on every device.
void gpu_set_random_seed(unsigned long long base);

#endif  // EDDL_HIP_BACKEND_H
