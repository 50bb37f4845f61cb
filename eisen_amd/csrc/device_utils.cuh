// Internal device helpers: bf16 <-> f32, 128-bit packets, wave64 and block reductions.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef __bf16 bf16_t;
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int kWave = 64;

__device__ __forceinline__ float to_f32(float x) { return x; }
__device__ __forceinline__ float to_f32(bf16_t x) { return (float)x; }
template <typename T> __device__ __forceinline__ T from_f32(float x);
template <> __device__ __forceinline__ float from_f32<float>(float x) { return x; }
template <> __device__ __forceinline__ bf16_t from_f32<bf16_t>(float x) { return (bf16_t)x; }  // RNE (v_cvt_pk_bf16_f32)

// A 16-byte packet of T: 4 floats or 8 bf16.
template <typename T> struct Pack;
template <> struct Pack<float> {
    static constexpr int N = 4;
    float4 raw;
    __device__ __forceinline__ float get(int i) const { return (&raw.x)[i]; }
    __device__ __forceinline__ void set(int i, float v) { (&raw.x)[i] = v; }
};
template <> struct Pack<bf16_t> {
    static constexpr int N = 8;
    bf16x8 raw;
    __device__ __forceinline__ float get(int i) const { return (float)raw[i]; }
    __device__ __forceinline__ void set(int i, float v) { raw[i] = (bf16_t)v; }
};
template <typename T> __device__ __forceinline__ Pack<T> load_pack(const T* p) {
    return *reinterpret_cast<const Pack<T>*>(p);
}
template <typename T> __device__ __forceinline__ void store_pack(T* p, const Pack<T>& v) {
    *reinterpret_cast<Pack<T>*>(p) = v;
}
// The same for data that is touched once (non-temporal: not kept in the caches).
template <typename T> __device__ __forceinline__ Pack<T> load_pack_streaming(const T* p) {
    const f32x4 t = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(p));
    return *reinterpret_cast<const Pack<T>*>(&t);
}
template <typename T> __device__ __forceinline__ void store_pack_streaming(T* p, const Pack<T>& v) {
    __builtin_nontemporal_store(*reinterpret_cast<const f32x4*>(&v), reinterpret_cast<f32x4*>(p));
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}
__device__ __forceinline__ double wave_sum_f64(double v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}

// Block-wide reductions; every thread gets the result.  `smem` holds >= blockDim.x/64 floats.
// The result is the same in every thread and independent of timing (fixed tree).
template <int THREADS> __device__ __forceinline__ float block_sum(float v, float* smem) {
    constexpr int W = THREADS / kWave;
    v = wave_sum(v);
    if (W == 1) return v;
    const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
    __syncthreads();
    if (lane == 0) smem[wid] = v;
    __syncthreads();
    float r = 0.f;
#pragma unroll
    for (int i = 0; i < W; i++) r += smem[i];
    return r;
}
template <int THREADS> __device__ __forceinline__ float block_max(float v, float* smem) {
    constexpr int W = THREADS / kWave;
    v = wave_max(v);
    if (W == 1) return v;
    const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
    __syncthreads();
    if (lane == 0) smem[wid] = v;
    __syncthreads();
    float r = -INFINITY;
#pragma unroll
    for (int i = 0; i < W; i++) r = fmaxf(r, smem[i]);
    return r;
}

// ---- LDS tiles filled by direct-to-LDS loads -------------------------------------------------------
// global_load_lds_dwordx4 writes the 64 lanes' 16-byte chunks to 1 KB of consecutive LDS, so such a tile has
// unpadded rows; bank conflicts are avoided by permuting the chunks of a row instead: chunk cc of row r sits at
// chunk position cc ^ lds_swz<row bytes>(r).  With 64 banks of 4 bytes (a 256-byte bank span) the permutation
// makes both MFMA operand read patterns conflict-free: 16 consecutive rows at one chunk position fall into 16
// different 16-byte slots of the span (16-byte reads of a k-contiguous operand), and 4 consecutive rows x 64
// bytes into 4 different 64-byte slots (the transposing 8-byte reads).
template <int ROW_BYTES>
__device__ __forceinline__ int lds_swz(int row) {
    static_assert(ROW_BYTES == 64 || ROW_BYTES == 128 || ROW_BYTES == 256 || ROW_BYTES == 512, "LDS row length not covered");
    if (ROW_BYTES == 64) return (row >> 2) & 3;                                                          // four rows per bank span
    if (ROW_BYTES == 128) return (((row >> 1) & 1) << 2) | (((row >> 2) & 1) << 1) | ((row >> 3) & 1);  // two rows per bank span
    return ((row & 3) << 2) | ((row >> 2) & 3);                                                          // a row is one or two bank spans
}

// Forward rotary embedding of one interleaved pair by the angle whose (cos, sin) is cs: y0 = x0 c - x1 s, y1 = x0 s + x1 c
// (src/graph/ops/transform.rs:562-566).  The fused multiply-adds are written out so that every kernel that rotates gets
// the same bits, whatever the compiler would contract elsewhere.
__device__ __forceinline__ void rope_rotate_forward(float a, float b, float2 cs, float& y0, float& y1) {
    y0 = __builtin_fmaf(a, cs.x, -(b * cs.y));
    y1 = __builtin_fmaf(a, cs.y, b * cs.x);
}

// Workgroups are handed to the 8 XCDs round-robin by linear id, and each XCD has its own L2.  This
// renumbering gives XCD j the contiguous id range [j*total/8, (j+1)*total/8), in dispatch order, so
// workgroups that are neighbours in the renumbered order (and share operands) also share an L2.
__device__ __forceinline__ int xcd_contiguous_id(int linear, int total) {
    const int per = total / 8;
    return linear < per * 8 ? (linear % 8) * per + linear / 8 : linear;
}
