// Kernels addressed by string name through eisen_hip_module_load / eisen_hip_get_function /
// eisen_hip_launch: the load-and-launch-by-name boundary of the reference
// (`Graph.functions: HashMap<String, CudaFunction>`, src/graph/mod.rs:60, :162-264).
// Names and argument lists follow the reference kernels they stand in for
// (kernels/ops_f32.cu:101-133, kernels/ops_bf16.cu:4-16) so a host that pushes arguments
// positionally keeps working.  Built with `hipcc --genco` into eisen_kernels.hsaco.
#include "device_utils.cuh"

extern "C" __global__ void fill_f32(float* out, float value, size_t n) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) out[i] = value;
}
extern "C" __global__ void scale_f32(float* data, float factor, size_t n) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) data[i] *= factor;
}
extern "C" __global__ void copy_f32(const float* in, float* out, size_t n) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) out[i] = in[i];
}
extern "C" __global__ void cast_f32_to_bf16(const float* in, bf16_t* out, size_t n) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) out[i] = (bf16_t)in[i];
}
extern "C" __global__ void cast_bf16_to_f32(const bf16_t* in, float* out, size_t n) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) out[i] = (float)in[i];
}
