// y[M,N] (fp32) = x[M,K] . W[N,K]^T for ANY M, N, K, row-major operands as a checkpoint stores them.
//
// The wave-tile projections (wgemm.hip, gemm_prefill.hip) want N % 16 == 0, K % 32 / 64 == 0 and a
// relaid-out weight image; layer stacks whose widths are whatever their configuration says (an
// input projection of 2*inner + 2*groups*state + heads rows, an inner width of heads * vdim) use
// this kernel for the shapes those cannot take.  Two forms:
//   bf16 operands: 64 x 64 output tile per workgroup of 4 waves, k in steps of 32 through LDS,
//                  v_mfma_f32_16x16x32_bf16, edges zero-filled in LDS;
//   fp32 operands: the same tile with fused multiply-adds (no reduced-precision matrix mode).
// Every output is the sum over k in ascending order of 32-wide (bf16) or 16-wide (fp32) steps,
// whatever M is: a row's result does not depend on which other rows share the launch.
#include "common.h"
#include <type_traits>

namespace mv {

typedef __attribute__((ext_vector_type(8))) __bf16 la_bf16x8_t;

// Rows in segments: with `seg` the launch's z-th product owns output rows seg[z] .. seg[z+1] (tokens sorted by
// the expert they go to) and reads, for output row i, operand row src[i] / src_div (src == NULL: row i).
struct RowSegments {
    const int* seg;
    const int* src;
    int src_div;
};

constexpr int kFewRows = 32;   // up to this many output rows a product takes the form without tiles
constexpr int kLaBM = 64, kLaBN = 64, kLaBK = 32, kLaPad = 40;  // LDS row = 40 bf16 = 80 bytes

__device__ __forceinline__ uint4 la_load8(const uint16_t* base, int64_t ld, int row, int nrows, int col, int k,
                                          bool vec) {
    if (row >= nrows || col >= k) return make_uint4(0, 0, 0, 0);
    const uint16_t* p = base + (int64_t)row * ld + col;
    if (vec && col + 8 <= k) return ld16(p);
    uint16_t e[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) e[i] = (col + i < k) ? p[i] : (uint16_t)0;
    return make_uint4(e[0] | ((uint32_t)e[1] << 16), e[2] | ((uint32_t)e[3] << 16), e[4] | ((uint32_t)e[5] << 16),
                      e[6] | ((uint32_t)e[7] << 16));
}

__global__ __launch_bounds__(256) void linear_any_bf16_kernel(
    const uint16_t* __restrict__ x, int64_t ldx, const uint16_t* __restrict__ w, int64_t ldw,
    float* __restrict__ y, int64_t ldy, int M, int N, int K, int vec_x, int vec_w, int64_t zx, int64_t zw,
    int64_t zy, RowSegments sg) {
    x += blockIdx.z * zx;   // blockIdx.z: one of several products that share a launch (per-head weights)
    w += blockIdx.z * zw;
    y += blockIdx.z * zy;
    __shared__ __attribute__((aligned(16))) uint16_t xs[kLaBM][kLaPad];
    __shared__ __attribute__((aligned(16))) uint16_t ws[kLaBN][kLaPad];
    const int m0 = blockIdx.y * kLaBM, n0 = blockIdx.x * kLaBN;
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, r = lane & 15, q = lane >> 4;
    const int lrow = tid >> 2, lcol = (tid & 3) * 8;
    int64_t y0 = 0;
    if (sg.seg) {   // blockIdx.z owns output rows seg[z] .. seg[z+1]
        y0 = sg.seg[blockIdx.z];
        M = sg.seg[blockIdx.z + 1] - (int)y0;
        if (m0 >= M) return;
        y += y0 * ldy;
    }
    // this thread's operand row: the output row itself, or the row the segment's list names for it
    {
        const int mr = m0 + lrow;
        const int64_t xrow = mr < M ? (sg.src ? sg.src[y0 + mr] / sg.src_div : y0 + mr) : 0;
        x += xrow * ldx - (int64_t)(m0 + lrow) * ldx;
    }
    f32x4_t acc[4] = {{0, 0, 0, 0}, {0, 0, 0, 0}, {0, 0, 0, 0}, {0, 0, 0, 0}};
    uint4 xr = la_load8(x, ldx, m0 + lrow, M, lcol, K, vec_x);
    uint4 wr = la_load8(w, ldw, n0 + lrow, N, lcol, K, vec_w);
    for (int k0 = 0; k0 < K; k0 += kLaBK) {
        __syncthreads();
        st16(&xs[lrow][lcol], xr);
        st16(&ws[lrow][lcol], wr);
        __syncthreads();
        if (k0 + kLaBK < K) {
            xr = la_load8(x, ldx, m0 + lrow, M, k0 + kLaBK + lcol, K, vec_x);
            wr = la_load8(w, ldw, n0 + lrow, N, k0 + kLaBK + lcol, K, vec_w);
        }
        // first operand: 16 weight rows of this wave; second: 16 activation rows per m-tile
        const la_bf16x8_t wf = __builtin_bit_cast(la_bf16x8_t, ld16(&ws[wave * 16 + r][q * 8]));
#pragma unroll
        for (int mt = 0; mt < 4; ++mt) {
            const la_bf16x8_t xf = __builtin_bit_cast(la_bf16x8_t, ld16(&xs[mt * 16 + r][q * 8]));
            acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf, xf, acc[mt], 0, 0, 0);
        }
    }
    // acc[mt][j] = C[n = n0 + 16 wave + 4 q + j][m = m0 + 16 mt + r]
#pragma unroll
    for (int mt = 0; mt < 4; ++mt) {
        const int m = m0 + mt * 16 + r;
        if (m >= M) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + wave * 16 + q * 4 + j;
            if (n < N) y[(int64_t)m * ldy + n] = acc[mt][j];
        }
    }
}

// The same product on a 128 x 128 tile for launches with many rows: four waves as 2 x 2, each 64 x 64 (sixteen
// accumulator tiles), so that a k-step of 32 costs a wave eight LDS reads for sixteen matrix instructions
// instead of five for four.  Same order of the sums over k as the 64 x 64 form: the results are equal bit for bit.
constexpr int kLbBM = 128, kLbBN = 128, kLbBK = 64, kLbPad = 72;   // LDS row = 72 bf16 = 144 bytes

__global__ __launch_bounds__(256) void linear_any_bf16_big_kernel(
    const uint16_t* __restrict__ x, int64_t ldx, const uint16_t* __restrict__ w, int64_t ldw,
    float* __restrict__ y, int64_t ldy, int M, int N, int K, int vec_x, int vec_w, int64_t zx, int64_t zw,
    int64_t zy, RowSegments sg) {
    x += blockIdx.z * zx;
    w += blockIdx.z * zw;
    y += blockIdx.z * zy;
    __shared__ __attribute__((aligned(16))) uint16_t xs[kLbBM][kLbPad];
    __shared__ __attribute__((aligned(16))) uint16_t ws[kLbBN][kLbPad];
    const int m0 = blockIdx.y * kLbBM, n0 = blockIdx.x * kLbBN;
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, r = lane & 15, q = lane >> 4;
    const int wm = wave >> 1, wn = wave & 1;
    const int lrow = tid >> 3, lcol = (tid & 7) * 8;   // a thread stages rows lrow + 32 u, eight values at lcol
    int64_t y0 = 0;
    if (sg.seg) {
        y0 = sg.seg[blockIdx.z];
        M = sg.seg[blockIdx.z + 1] - (int)y0;
        if (m0 >= M) return;
        y += y0 * ldy;
    }
    const uint16_t* xp[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        const int mr = m0 + lrow + 32 * u;
        const int64_t xrow = mr < M ? (sg.src ? sg.src[y0 + mr] / sg.src_div : y0 + mr) : 0;
        xp[u] = x + xrow * ldx;
    }
    f32x4_t acc[4][4];
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
        for (int b = 0; b < 4; ++b) acc[a][b] = f32x4_t{0, 0, 0, 0};
    uint4 xr[4], wr[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        xr[u] = la_load8(xp[u], ldx, 0, m0 + lrow + 32 * u < M ? 1 : 0, lcol, K, vec_x);
        wr[u] = la_load8(w, ldw, n0 + lrow + 32 * u, N, lcol, K, vec_w);
    }
    for (int k0 = 0; k0 < K; k0 += kLbBK) {
        __syncthreads();
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            st16(&xs[lrow + 32 * u][lcol], xr[u]);
            st16(&ws[lrow + 32 * u][lcol], wr[u]);
        }
        __syncthreads();
        if (k0 + kLbBK < K) {
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                xr[u] = la_load8(xp[u], ldx, 0, m0 + lrow + 32 * u < M ? 1 : 0, k0 + kLbBK + lcol, K, vec_x);
                wr[u] = la_load8(w, ldw, n0 + lrow + 32 * u, N, k0 + kLbBK + lcol, K, vec_w);
            }
        }
#pragma unroll
        for (int ks = 0; ks < kLbBK; ks += 32) {   // two steps of 32, in ascending k as the narrow tile takes them
            la_bf16x8_t wf[4], xf[4];
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                wf[t] = __builtin_bit_cast(la_bf16x8_t, ld16(&ws[wn * 64 + t * 16 + r][ks + q * 8]));
                xf[t] = __builtin_bit_cast(la_bf16x8_t, ld16(&xs[wm * 64 + t * 16 + r][ks + q * 8]));
            }
#pragma unroll
            for (int nt = 0; nt < 4; ++nt)
#pragma unroll
                for (int mt = 0; mt < 4; ++mt)
                    acc[nt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[nt], xf[mt], acc[nt][mt], 0, 0, 0);
        }
    }
    // acc[nt][mt][j] = C[n = n0 + 64 wn + 16 nt + 4 q + j][m = m0 + 64 wm + 16 mt + r]
#pragma unroll
    for (int mt = 0; mt < 4; ++mt) {
        const int m = m0 + wm * 64 + mt * 16 + r;
        if (m >= M) continue;
#pragma unroll
        for (int nt = 0; nt < 4; ++nt) {
            const int n = n0 + wn * 64 + nt * 16 + q * 4;
            float* dst = y + (int64_t)m * ldy + n;
            if (n + 3 < N && (reinterpret_cast<uintptr_t>(dst) & 15) == 0) {
                *reinterpret_cast<float4*>(dst) = make_float4(acc[nt][mt][0], acc[nt][mt][1], acc[nt][mt][2], acc[nt][mt][3]);
            } else {
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    if (n + j < N) dst[j] = acc[nt][mt][j];
            }
        }
    }
}

constexpr int kLfBK = 16;

__global__ __launch_bounds__(256) void linear_any_f32_kernel(
    const float* __restrict__ x, int64_t ldx, const float* __restrict__ w, int64_t ldw,
    float* __restrict__ y, int64_t ldy, int M, int N, int K, int64_t zx, int64_t zw, int64_t zy, RowSegments sg) {
    x += blockIdx.z * zx;
    w += blockIdx.z * zw;
    y += blockIdx.z * zy;
    __shared__ float xs[kLfBK][kLaBM + 4];
    __shared__ float ws[kLfBK][kLaBN + 4];
    const int m0 = blockIdx.y * kLaBM, n0 = blockIdx.x * kLaBN;
    const int tid = threadIdx.x, tx = tid & 15, ty = tid >> 4;
    const int lrow = tid >> 2, lcol = (tid & 3) * 4;
    int64_t y0 = 0;
    if (sg.seg) {
        y0 = sg.seg[blockIdx.z];
        M = sg.seg[blockIdx.z + 1] - (int)y0;
        if (m0 >= M) return;
        y += y0 * ldy;
    }
    {
        const int mr = m0 + lrow;
        const int64_t xrow = mr < M ? (sg.src ? sg.src[y0 + mr] / sg.src_div : y0 + mr) : 0;
        x += xrow * ldx - (int64_t)(m0 + lrow) * ldx;
    }
    float acc[4][4] = {};
    for (int k0 = 0; k0 < K; k0 += kLfBK) {
        __syncthreads();
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int kk = k0 + lcol + i;
            xs[lcol + i][lrow] = (m0 + lrow < M && kk < K) ? x[(int64_t)(m0 + lrow) * ldx + kk] : 0.f;
            ws[lcol + i][lrow] = (n0 + lrow < N && kk < K) ? w[(int64_t)(n0 + lrow) * ldw + kk] : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < kLfBK; ++kk) {
            float a[4], b[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                a[i] = xs[kk][ty * 4 + i];
                b[i] = ws[kk][tx * 4 + i];
            }
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
        }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = m0 + ty * 4 + i;
        if (m >= M) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + tx * 4 + j;
            if (n < N) y[(int64_t)m * ldy + n] = acc[i][j];
        }
    }
}

// Few output rows (decoding): a wave forms four neighbouring outputs of ONE row from 16-byte loads of the operand
// row and of four weight rows, no LDS, no barrier; grid = (column groups of 16, rows, products).  With segments
// the row's weight is found from the segment table.  Needs K % 8 == 0 (bf16) / K % 4 == 0 (fp32) and aligned rows.
template <bool F32>
__global__ __launch_bounds__(256) void linear_fewrows_kernel(const void* __restrict__ x_, int64_t ldx,
                                                             const void* __restrict__ w_, int64_t ldw,
                                                             float* __restrict__ y, int64_t ldy, int N, int K,
                                                             int64_t zx, int64_t zw, int64_t zy, RowSegments sg,
                                                             int segments) {
    typedef typename std::conditional<F32, float, uint16_t>::type T_;
    const T_* x = (const T_*)x_;
    const T_* w = (const T_*)w_;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    int64_t row = blockIdx.y, xrow = row;
    if (sg.seg) {
        if (row >= sg.seg[segments]) return;
        int lo = 0, hi = segments;              // the segment that holds the row
        while (hi - lo > 1) {
            const int mid = (lo + hi) >> 1;
            if (sg.seg[mid] <= row) lo = mid; else hi = mid;
        }
        w += (int64_t)lo * zw;
        xrow = sg.src ? sg.src[row] / sg.src_div : row;
    } else {
        x += blockIdx.z * zx;
        w += blockIdx.z * zw;
        y += blockIdx.z * zy;
    }
    const int n0 = (blockIdx.x * 4 + wave) * 4;
    if (n0 >= N) return;
    const T_* xr = x + xrow * ldx;
    const T_* wr[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) wr[j] = w + (int64_t)(n0 + j < N ? n0 + j : n0) * ldw;
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    constexpr int PER = F32 ? 4 : 8;
    for (int k = lane * PER; k < K; k += 64 * PER) {
        const uint4 xv = ld16(xr + k);
        uint4 wv[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) wv[j] = ld16_nt(wr[j] + k);
        if (F32) {
            const float xf[4] = {__uint_as_float(xv.x), __uint_as_float(xv.y), __uint_as_float(xv.z), __uint_as_float(xv.w)};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float wf[4] = {__uint_as_float(wv[j].x), __uint_as_float(wv[j].y), __uint_as_float(wv[j].z),
                                     __uint_as_float(wv[j].w)};
#pragma unroll
                for (int e = 0; e < 4; ++e) acc[j] = fmaf(xf[e], wf[e], acc[j]);
            }
        } else {
            const uint32_t xp[4] = {xv.x, xv.y, xv.z, xv.w};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint32_t wp[4] = {wv[j].x, wv[j].y, wv[j].z, wv[j].w};
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    acc[j] = fmaf(bf16_lo(xp[e]), bf16_lo(wp[e]), acc[j]);
                    acc[j] = fmaf(bf16_hi(xp[e]), bf16_hi(wp[e]), acc[j]);
                }
            }
        }
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const float tot = wave_sum(acc[j]);
        if (lane == 0 && n0 + j < N) y[row * ldy + n0 + j] = tot;
    }
}

}  // namespace mv

static int launch_linear_any(const void* x, int64_t ldx, const void* w, int64_t ldw, float* y, int64_t ldy, int m, int n,
                             int k, int f32, int batch, int64_t zx, int64_t zw, int64_t zy, mv_stream_t stream,
                             mv::RowSegments sg = mv::RowSegments{nullptr, nullptr, 1}, int few_rows = 0,
                             bool big_tiles = false) {
    using namespace mv;
    const dim3 grid((n + kLaBN - 1) / kLaBN, (m + kLaBM - 1) / kLaBM, batch);
    if (grid.y > 65535 || batch > 65535) return MV_ERR_UNSUPPORTED;
    hipStream_t s = (hipStream_t)stream;
    if (few_rows > 0) {
        const int per = f32 ? 4 : 8;
        const bool fits = k % per == 0 && ldx % per == 0 && ldw % per == 0 && zx % per == 0 && zw % per == 0 &&
                          aligned16(x) && aligned16(w);
        if (fits) {
            const dim3 g((n + 15) / 16, few_rows, sg.seg ? 1 : batch);
            if (f32) hipLaunchKernelGGL(linear_fewrows_kernel<true>, g, dim3(256), 0, s, x, ldx, w, ldw, y, ldy, n, k, zx, zw, zy, sg, batch);
            else hipLaunchKernelGGL(linear_fewrows_kernel<false>, g, dim3(256), 0, s, x, ldx, w, ldw, y, ldy, n, k, zx, zw, zy, sg, batch);
            return check_launch();
        }
    }
    if (f32) {
        hipLaunchKernelGGL(linear_any_f32_kernel, grid, dim3(256), 0, s, (const float*)x, ldx, (const float*)w, ldw,
                           y, ldy, m, n, k, zx, zw, zy, sg);
    } else {
        const int vx = aligned16(x) && ldx % 8 == 0 && zx % 8 == 0, vw = aligned16(w) && ldw % 8 == 0 && zw % 8 == 0;
        if (big_tiles && n >= kLbBN) {
            const dim3 big((n + kLbBN - 1) / kLbBN, (m + kLbBM - 1) / kLbBM, batch);
            hipLaunchKernelGGL(linear_any_bf16_big_kernel, big, dim3(256), 0, s, (const uint16_t*)x, ldx,
                               (const uint16_t*)w, ldw, y, ldy, m, n, k, vx, vw, zx, zw, zy, sg);
            return check_launch();
        }
        hipLaunchKernelGGL(linear_any_bf16_kernel, grid, dim3(256), 0, s, (const uint16_t*)x, ldx, (const uint16_t*)w,
                           ldw, y, ldy, m, n, k, vx, vw, zx, zw, zy, sg);
    }
    return check_launch();
}

extern "C" int mv_linear_any(const void* x, int64_t ldx, const void* w, int64_t ldw, float* y, int64_t ldy,
                             int m, int n, int k, int f32, mv_stream_t stream) {
    if (m < 0 || n <= 0 || k <= 0) return MV_ERR_INVALID_ARG;
    if (m == 0) return MV_OK;
    if (!x || !w || !y || ldx < k || ldw < k || ldy < n) return MV_ERR_INVALID_ARG;
    return launch_linear_any(x, ldx, w, ldw, y, ldy, m, n, k, f32, 1, 0, 0, 0, stream,
                             mv::RowSegments{nullptr, nullptr, 1}, 0, m >= 256);
}

// `heads` products in one launch: y[:, h*zy + ..n] = x[:, h*zx + ..k] . W_h^T with W_h = w + h*zw ([n,k], row stride ldw)
extern "C" int mv_linear_heads(const void* x, int64_t ldx, int64_t zx, const void* w, int64_t ldw, int64_t zw, float* y,
                               int64_t ldy, int64_t zy, int m, int n, int k, int heads, int f32, mv_stream_t stream) {
    if (m < 0 || n <= 0 || k <= 0 || heads <= 0 || zx < 0 || zw < 0 || zy < 0) return MV_ERR_INVALID_ARG;
    if (m == 0) return MV_OK;
    if (!x || !w || !y || ldx < (heads - 1) * zx + k || ldw < k || ldy < (heads - 1) * zy + n) return MV_ERR_INVALID_ARG;
    return launch_linear_any(x, ldx, w, ldw, y, ldy, m, n, k, f32, heads, zx, zw, zy, stream,
                             mv::RowSegments{nullptr, nullptr, 1}, m <= mv::kFewRows ? m : 0, m >= 256);
}

// Products by segment: output rows seg[e] .. seg[e+1] (e < segments) use weight w + e*zw; `max_rows` bounds the
// rows of any one segment (the launch has that many row tiles per segment, the ones past a segment's end leave
// at once).  src: operand row of output row i is src[i] / src_div (NULL: i).  total_rows = seg[segments] as the host
// knows it (the rows of `y`): few of them take the form without tiles.
extern "C" int mv_linear_segments(const void* x, int64_t ldx, const void* w, int64_t ldw, int64_t zw, float* y,
                                  int64_t ldy, const int32_t* seg, const int32_t* src, int src_div, int segments,
                                  int max_rows, int total_rows, int n, int k, int f32, mv_stream_t stream) {
    if (max_rows < 0 || n <= 0 || k <= 0 || segments <= 0 || src_div <= 0 || zw < 0) return MV_ERR_INVALID_ARG;
    if (max_rows == 0) return MV_OK;
    if (!x || !w || !y || !seg || ldx < k || ldw < k || ldy < n) return MV_ERR_INVALID_ARG;
    return launch_linear_any(x, ldx, w, ldw, y, ldy, max_rows, n, k, f32, segments, 0, zw, 0, stream,
                             mv::RowSegments{seg, src, src_div}, total_rows <= mv::kFewRows ? total_rows : 0,
                             total_rows / segments >= 96);
}
