// Row-wise steps around an fp32 residual stream: layer stacks that keep the running sum of their
// sublayers in 32 bits and hand every projection a copy in the activation type (bf16, or fp32 when
// the whole model runs in 32 bits).
//
//   embed_scaled:        x = table[id] * scale                       (fp32), h = act(x)
//   postnorm_residual:   v = s1*y1 (+ s2*y2); x += v / sqrt(mean(v^2) + eps) * (1 + w); h = act(x)
//                        (the norm sits on the SUBLAYER'S OUTPUT, its weight is stored as an offset
//                        from one)
//   offset_rmsnorm_gather: out = act( x[idx] / sqrt(mean(x[idx]^2) + eps) * (1 + w) )
//   relu_squared:        out = act( max(v, 0)^2 )
//   softcap:             v = cap * tanh(v / cap)
// All arithmetic is fp32 with the library's exact division, square root and tanh.
#include "common.h"

namespace mv {

template <bool F32> struct Act;
template <> struct Act<true> {
    typedef float T;
    static __device__ __forceinline__ float ld(const float* p) { return *p; }
    static __device__ __forceinline__ void st(float* p, float v) { *p = v; }
};
template <> struct Act<false> {
    typedef uint16_t T;
    static __device__ __forceinline__ float ld(const uint16_t* p) { return bf16_bits_to_f32(*p); }
    static __device__ __forceinline__ void st(uint16_t* p, float v) { *p = (uint16_t)f32_to_bf16_bits(v); }
};

template <bool F32>
__global__ __launch_bounds__(256) void embed_scaled_kernel(const void* table_, const int* ids, float* x, int64_t ldx,
                                                           void* h_, int64_t ldh, int n, int vocab, float scale) {
    typedef typename Act<F32>::T T;
    const T* table = (const T*)table_;
    T* h = (T*)h_;
    const int row = blockIdx.x;
    int id = ids[row];
    id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
    for (int c = threadIdx.x; c < n; c += 256) {
        const float v = Act<F32>::ld(table + (int64_t)id * n + c) * scale;
        x[(int64_t)row * ldx + c] = v;
        Act<F32>::st(h + (int64_t)row * ldh + c, v);
    }
}

template <bool F32>
__global__ __launch_bounds__(256) void postnorm_residual_kernel(const float* y1, int64_t ld1, const float* y2,
                                                                int64_t ld2, float s1, float s2, const float* w,
                                                                float eps, float* x, int64_t ldx, void* h_,
                                                                int64_t ldh, int n) {
    typedef typename Act<F32>::T T;
    __shared__ float red[4];
    T* h = (T*)h_;
    const int row = blockIdx.x;
    const float* a = y1 + (int64_t)row * ld1;
    const float* b = y2 ? y2 + (int64_t)row * ld2 : nullptr;
    float ss = 0.f;
    for (int c = threadIdx.x; c < n; c += 256) {
        const float v = b ? s1 * a[c] + s2 * b[c] : s1 * a[c];
        ss += v * v;
    }
    ss = block_sum(ss, red);
    const float inv = 1.0f / sqrtf(ss / (float)n + eps);
    for (int c = threadIdx.x; c < n; c += 256) {
        const float v = b ? s1 * a[c] + s2 * b[c] : s1 * a[c];
        const float s = x[(int64_t)row * ldx + c] + (v * inv) * (1.0f + w[c]);
        x[(int64_t)row * ldx + c] = s;
        Act<F32>::st(h + (int64_t)row * ldh + c, s);
    }
}

template <bool F32>
__global__ __launch_bounds__(256) void offset_rmsnorm_gather_kernel(const float* x, int64_t ldx, const int* idx,
                                                                    const float* w, float eps, void* out_,
                                                                    int64_t ldo, int n) {
    typedef typename Act<F32>::T T;
    __shared__ float red[4];
    T* out = (T*)out_;
    const int row = blockIdx.x;
    const float* a = x + (int64_t)(idx ? idx[row] : row) * ldx;
    float ss = 0.f;
    for (int c = threadIdx.x; c < n; c += 256) ss += a[c] * a[c];
    ss = block_sum(ss, red);
    const float inv = 1.0f / sqrtf(ss / (float)n + eps);
    for (int c = threadIdx.x; c < n; c += 256) Act<F32>::st(out + (int64_t)row * ldo + c, (a[c] * inv) * (1.0f + w[c]));
}

template <bool F32>
__global__ __launch_bounds__(256) void relu_squared_kernel(const float* in, int64_t ldi, void* out_, int64_t ldo,
                                                           int n) {
    typedef typename Act<F32>::T T;
    T* out = (T*)out_;
    const int row = blockIdx.x;
    const int c = blockIdx.y * 256 + threadIdx.x;
    if (c >= n) return;
    const float v = fmaxf(in[(int64_t)row * ldi + c], 0.f);
    Act<F32>::st(out + (int64_t)row * ldo + c, v * v);
}

__global__ __launch_bounds__(256) void softcap_kernel(float* v, int64_t count, float cap) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < count) v[i] = cap * tanhf(v[i] / cap);
}

}  // namespace mv

extern "C" {

int mv_embed_scaled(const void* table, const int32_t* ids, float* x, int64_t ldx, void* h, int64_t ldh, int rows,
                    int n, int vocab, float scale, int f32, mv_stream_t stream) {
    using namespace mv;
    if (rows < 0 || n <= 0 || vocab <= 0) return MV_ERR_INVALID_ARG;
    if (rows == 0) return MV_OK;
    if (!table || !ids || !x || !h || ldx < n || ldh < n) return MV_ERR_INVALID_ARG;
    hipStream_t s = (hipStream_t)stream;
    if (f32) hipLaunchKernelGGL(embed_scaled_kernel<true>, dim3(rows), dim3(256), 0, s, table, ids, x, ldx, h, ldh, n, vocab, scale);
    else hipLaunchKernelGGL(embed_scaled_kernel<false>, dim3(rows), dim3(256), 0, s, table, ids, x, ldx, h, ldh, n, vocab, scale);
    return check_launch();
}

int mv_postnorm_residual(const float* y1, int64_t ld1, const float* y2, int64_t ld2, float s1, float s2,
                         const float* w, float eps, float* x, int64_t ldx, void* h, int64_t ldh, int rows, int n,
                         int f32, mv_stream_t stream) {
    using namespace mv;
    if (rows < 0 || n <= 0) return MV_ERR_INVALID_ARG;
    if (rows == 0) return MV_OK;
    if (!y1 || !w || !x || !h || ld1 < n || (y2 && ld2 < n) || ldx < n || ldh < n) return MV_ERR_INVALID_ARG;
    hipStream_t s = (hipStream_t)stream;
    if (f32) hipLaunchKernelGGL(postnorm_residual_kernel<true>, dim3(rows), dim3(256), 0, s, y1, ld1, y2, ld2, s1, s2, w, eps, x, ldx, h, ldh, n);
    else hipLaunchKernelGGL(postnorm_residual_kernel<false>, dim3(rows), dim3(256), 0, s, y1, ld1, y2, ld2, s1, s2, w, eps, x, ldx, h, ldh, n);
    return check_launch();
}

int mv_offset_rmsnorm_gather(const float* x, int64_t ldx, const int32_t* idx, const float* w, float eps, void* out,
                             int64_t ldo, int rows, int n, int f32, mv_stream_t stream) {
    using namespace mv;
    if (rows < 0 || n <= 0) return MV_ERR_INVALID_ARG;
    if (rows == 0) return MV_OK;
    if (!x || !w || !out || ldx < n || ldo < n) return MV_ERR_INVALID_ARG;
    hipStream_t s = (hipStream_t)stream;
    if (f32) hipLaunchKernelGGL(offset_rmsnorm_gather_kernel<true>, dim3(rows), dim3(256), 0, s, x, ldx, idx, w, eps, out, ldo, n);
    else hipLaunchKernelGGL(offset_rmsnorm_gather_kernel<false>, dim3(rows), dim3(256), 0, s, x, ldx, idx, w, eps, out, ldo, n);
    return check_launch();
}

int mv_relu_squared(const float* in, int64_t ldi, void* out, int64_t ldo, int rows, int n, int f32,
                    mv_stream_t stream) {
    using namespace mv;
    if (rows < 0 || n <= 0) return MV_ERR_INVALID_ARG;
    if (rows == 0) return MV_OK;
    if (!in || !out || ldi < n || ldo < n) return MV_ERR_INVALID_ARG;
    hipStream_t s = (hipStream_t)stream;
    const dim3 grid(rows, (n + 255) / 256);
    if (f32) hipLaunchKernelGGL(relu_squared_kernel<true>, grid, dim3(256), 0, s, in, ldi, out, ldo, n);
    else hipLaunchKernelGGL(relu_squared_kernel<false>, grid, dim3(256), 0, s, in, ldi, out, ldo, n);
    return check_launch();
}

int mv_softcap(float* v, int64_t count, float cap, mv_stream_t stream) {
    using namespace mv;
    if (count < 0 || !(cap > 0.f)) return MV_ERR_INVALID_ARG;
    if (count == 0) return MV_OK;
    if (!v) return MV_ERR_INVALID_ARG;
    hipLaunchKernelGGL(softcap_kernel, dim3((unsigned)((count + 255) / 256)), dim3(256), 0, (hipStream_t)stream, v, count, cap);
    return check_launch();
}

}  // extern "C"
