// The element-wise and shape operations of the reference's backend interface on device memory, fp32:
//   Add / Sub / Mul / Div with NumPy-style broadcasting  (tensor.Backend, internal/tensor/backend.go:14-17;
//     CPU form internal/backend/cpu/backend.go:32-134; shape rule internal/tensor/shape.go:83-118)
//   Transpose by an axis permutation                      (internal/backend/cpu/backend.go:164-209)
//   Conv2D, MaxPool2D                                     (internal/backend/cpu/conv2d.go, maxpool2d.go)
// The element-wise and shape operations are bound by HBM traffic: every operand element is read once and every result written once.
// Each result is one IEEE fp32 operation (the division correctly rounded), so results equal the CPU's bit
// for bit.
#include "dev_common.h"
#include "kernels.h"

namespace born {

typedef float t_f32x4 __attribute__((ext_vector_type(4)));

template <int OP>
__device__ __forceinline__ float tensor_apply(float x, float y) {
    return OP == 0 ? x + y : OP == 1 ? x - y : OP == 2 ? x * y : x / y;
}

constexpr int TOPS_BLOCK = 256;

// Same shape, both operands contiguous: 128-bit accesses, one pass.
template <int OP>
__global__ __launch_bounds__(TOPS_BLOCK) void binary_flat_kernel(const float *a, const float *b, float *out, long long n,
                                                                  int vec) {
    const long long gid = (long long)blockIdx.x * TOPS_BLOCK + threadIdx.x;
    const long long stride = (long long)gridDim.x * TOPS_BLOCK;
    if (vec) {
        const long long n4 = n >> 2;
        for (long long i = gid; i < n4; i += stride) {
            const t_f32x4 x = __builtin_nontemporal_load(reinterpret_cast<const t_f32x4 *>(a) + i);
            const t_f32x4 y = __builtin_nontemporal_load(reinterpret_cast<const t_f32x4 *>(b) + i);
            t_f32x4 r;
#pragma unroll
            for (int c = 0; c < 4; c++) r[c] = tensor_apply<OP>(x[c], y[c]);
            __builtin_nontemporal_store(r, reinterpret_cast<t_f32x4 *>(out) + i);
        }
        for (long long i = (n4 << 2) + gid; i < n; i += stride) out[i] = tensor_apply<OP>(a[i], b[i]);
    } else {
        for (long long i = gid; i < n; i += stride) out[i] = tensor_apply<OP>(a[i], b[i]);
    }
}

// out[r, c] = a[r * ars + c * acs] op b[r * brs + c * bcs] over a [rows, cols] result, every stride 0 or the
// contiguous one: a matrix with a row vector (the bias of a linear layer), a column vector, or a scalar.
// A workgroup takes a strip of 1024 columns of one row, so a broadcast operand stays in cache or in a register.
template <int OP>
__global__ __launch_bounds__(TOPS_BLOCK) void binary_rowcol_kernel(const float *a, const float *b, float *out, long long rows,
                                                                    long long cols, long long ars, long long acs,
                                                                    long long brs, long long bcs) {
    const long long strips = (cols + 4 * TOPS_BLOCK - 1) / (4 * TOPS_BLOCK);
    const long long total = rows * strips;
    for (long long w = blockIdx.x; w < total; w += gridDim.x) {
        const long long r = w / strips, c0 = (w % strips) * (4 * TOPS_BLOCK);
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const long long c = c0 + u * TOPS_BLOCK + threadIdx.x;
            if (c < cols) out[r * cols + c] = tensor_apply<OP>(a[r * ars + c * acs], b[r * brs + c * bcs]);
        }
    }
}

// The same for rows whose length is a multiple of 4 with 16-byte aligned operands and column strides of 0 or 1:
// 128-bit accesses along the row; an operand broadcast along the row is one scalar per row.
template <int OP>
__global__ __launch_bounds__(TOPS_BLOCK) void binary_rowcol_vec_kernel(const float *a, const float *b, float *out,
                                                                        long long rows, long long cols4, long long ars,
                                                                        int a_along, long long brs, int b_along) {
    const long long total = rows * cols4;
    const long long stride = (long long)gridDim.x * TOPS_BLOCK;
    for (long long i = (long long)blockIdx.x * TOPS_BLOCK + threadIdx.x; i < total; i += stride) {
        const long long r = i / cols4, c4 = i - r * cols4;
        t_f32x4 x, y, v;
        if (a_along) {
            x = __builtin_nontemporal_load(reinterpret_cast<const t_f32x4 *>(a + r * ars) + c4);
        } else {
            const float sx = a[r * ars];
            x = t_f32x4{sx, sx, sx, sx};
        }
        if (b_along) {
            y = __builtin_nontemporal_load(reinterpret_cast<const t_f32x4 *>(b + r * brs) + c4);
        } else {
            const float sy = b[r * brs];
            y = t_f32x4{sy, sy, sy, sy};
        }
#pragma unroll
        for (int c = 0; c < 4; c++) v[c] = tensor_apply<OP>(x[c], y[c]);
        __builtin_nontemporal_store(v, reinterpret_cast<t_f32x4 *>(out + r * cols4 * 4) + c4);
    }
}

// Any broadcast of up to TENSOR_MAX_DIMS dimensions: one result element per thread and step, operand offsets
// from the result's multi-index (a broadcast dimension has stride 0).
template <int OP>
__global__ __launch_bounds__(TOPS_BLOCK) void binary_general_kernel(TensorIndexArgs t, const float *a, const float *b,
                                                                     float *out) {
    const long long stride = (long long)gridDim.x * TOPS_BLOCK;
    for (long long i = (long long)blockIdx.x * TOPS_BLOCK + threadIdx.x; i < t.n; i += stride) {
        long long rem = i, oa = 0, ob = 0;
#pragma unroll 1
        for (int d = t.nd - 1; d >= 0; d--) {
            const long long q = rem / t.shape[d], idx = rem - q * t.shape[d];
            rem = q;
            oa += idx * t.sa[d];
            ob += idx * t.sb[d];
        }
        out[i] = tensor_apply<OP>(a[oa], b[ob]);
    }
}

// out[b, c, r] = in[b, r, c]: 64 x 64 tiles through LDS (pitch 65), reads and writes both contiguous.
constexpr int TR_TILE = 64;
__global__ __launch_bounds__(TOPS_BLOCK) void transpose_tiled_kernel(const float *in, float *out, long long batch,
                                                                      long long R, long long C) {
    __shared__ float tile[TR_TILE][TR_TILE + 1];
    const long long tr = (R + TR_TILE - 1) / TR_TILE, tc = (C + TR_TILE - 1) / TR_TILE;
    const long long total = batch * tr * tc;
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;          // 64 x 4 threads
    for (long long w = blockIdx.x; w < total; w += gridDim.x) {
        const long long bb = w / (tr * tc), rem = w % (tr * tc);
        const long long r0 = (rem / tc) * TR_TILE, c0 = (rem % tc) * TR_TILE;
        const float *src = in + bb * R * C;
        float *dst = out + bb * R * C;
#pragma unroll
        for (int k = 0; k < TR_TILE; k += 4) {
            const long long r = r0 + ty + k, c = c0 + tx;
            if (r < R && c < C) tile[ty + k][tx] = src[r * C + c];
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < TR_TILE; k += 4) {
            const long long c = c0 + ty + k, r = r0 + tx;
            if (r < R && c < C) dst[c * R + r] = tile[tx][ty + k];
        }
        __syncthreads();
    }
}

// The same with 128-bit global accesses on both sides (R and C multiples of 4, 16-byte aligned): a quarter of
// the memory instructions.  Lane (q, l) = (thread / 16, thread % 16) reads columns 4 l .. 4 l + 3 of rows
// q, q + 16, .. of the tile and later writes rows 4 l .. 4 l + 3 of the transposed tile's rows q, q + 16, ..
__global__ __launch_bounds__(TOPS_BLOCK) void transpose_tiled_vec_kernel(const float *in, float *out, long long batch,
                                                                          long long R, long long C) {
    __shared__ float tile[TR_TILE][TR_TILE + 1];
    const long long tr = (R + TR_TILE - 1) / TR_TILE, tc = (C + TR_TILE - 1) / TR_TILE;
    const long long total = batch * tr * tc;
    const int l = threadIdx.x & 15, q = threadIdx.x >> 4;            // 16 x 16 threads
    for (long long w = blockIdx.x; w < total; w += gridDim.x) {
        const long long bb = w / (tr * tc), rem = w % (tr * tc);
        const long long r0 = (rem / tc) * TR_TILE, c0 = (rem % tc) * TR_TILE;
        const float *src = in + bb * R * C;
        float *dst = out + bb * R * C;
        t_f32x4 v[4];
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const long long r = r0 + q + 16 * k, c = c0 + 4 * l;
            if (r < R && c < C) v[k] = __builtin_nontemporal_load(reinterpret_cast<const t_f32x4 *>(src + r * C + c));
        }
#pragma unroll
        for (int k = 0; k < 4; k++)
#pragma unroll
            for (int e = 0; e < 4; e++) tile[q + 16 * k][4 * l + e] = v[k][e];
        __syncthreads();
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const long long c = c0 + q + 16 * k, r = r0 + 4 * l;
            if (c < C && r < R) {
                t_f32x4 o;
#pragma unroll
                for (int e = 0; e < 4; e++) o[e] = tile[4 * l + e][q + 16 * k];
                __builtin_nontemporal_store(o, reinterpret_cast<t_f32x4 *>(dst + c * R + r));
            }
        }
        __syncthreads();
    }
}

// Any permutation: one result element per thread and step, the source offset from the result's multi-index
// through the permuted source strides (t.sa).
__global__ __launch_bounds__(TOPS_BLOCK) void transpose_general_kernel(TensorIndexArgs t, const float *in, float *out) {
    const long long stride = (long long)gridDim.x * TOPS_BLOCK;
    for (long long i = (long long)blockIdx.x * TOPS_BLOCK + threadIdx.x; i < t.n; i += stride) {
        long long rem = i, oa = 0;
#pragma unroll 1
        for (int d = t.nd - 1; d >= 0; d--) {
            const long long q = rem / t.shape[d], idx = rem - q * t.shape[d];
            rem = q;
            oa += idx * t.sa[d];
        }
        out[i] = in[oa];
    }
}

// Conv2D (internal/backend/cpu/conv2d.go:35-203): input [N, C, H, W], kernel [CO, C, KH, KW], zero padding;
// out[n, co, oh, ow] = sum over (c, kh, kw), in that order, of kernel * input, one fp32 accumulator per output,
// product and sum each rounded (the reference's im2col + row-by-row dot product adds the terms in exactly this
// order, the padded positions as a multiplication by 0), so results equal the CPU's bit for bit.
// conv2d_kernel: one output per thread; neighbouring threads read neighbouring input columns and share the kernel values
// through the caches.  conv2d_group_kernel (below), which the launcher prefers: a workgroup takes 256 consecutive
// positions (n, oh, ow) and CONV_COG output channels, so the kernel values are the same for every thread - scalar
// loads, one per channel and product - and an input value is loaded once for CONV_COG products; every output still
// has its own accumulator and the same order of terms.
__global__ __launch_bounds__(TOPS_BLOCK) void conv2d_kernel(const float *in, const float *ker, float *out, int N, int C,
                                                            int H, int W, int CO, int KH, int KW, int HO, int WO, int stride,
                                                            int padding) {
    const long long total = (long long)N * CO * HO * WO;
    const long long step = (long long)gridDim.x * TOPS_BLOCK;
    for (long long i = (long long)blockIdx.x * TOPS_BLOCK + threadIdx.x; i < total; i += step) {
        const int ow = (int)(i % WO), oh = (int)((i / WO) % HO), co = (int)((i / ((long long)WO * HO)) % CO);
        const int n = (int)(i / ((long long)WO * HO * CO));
        const int h0 = oh * stride - padding, w0 = ow * stride - padding;
        const float *kp = ker + (long long)co * C * KH * KW;
        float sum = 0.0f;
        for (int c = 0; c < C; c++) {
            const float *ip = in + ((long long)n * C + c) * H * W;
            for (int kh = 0; kh < KH; kh++) {
                const int h = h0 + kh;
                for (int kw = 0; kw < KW; kw++) {
                    const int w = w0 + kw;
                    const float x = (h >= 0 && h < H && w >= 0 && w < W) ? ip[(long long)h * W + w] : 0.0f;
                    sum += kp[(c * KH + kh) * KW + kw] * x;
                }
            }
        }
        out[i] = sum;
    }
}

// MaxPool2D (internal/backend/cpu/maxpool2d.go:26-113): windows of kernel x kernel, no padding; the running
// maximum starts at -1e38 and is replaced by values that compare greater, as in the reference (so a NaN never
// wins and nothing below -1e38 is returned).
__global__ __launch_bounds__(TOPS_BLOCK) void maxpool2d_kernel(const float *in, float *out, long long planes, int H, int W,
                                                               int HO, int WO, int ksize, int stride) {
    const long long total = planes * HO * WO;
    const long long step = (long long)gridDim.x * TOPS_BLOCK;
    for (long long i = (long long)blockIdx.x * TOPS_BLOCK + threadIdx.x; i < total; i += step) {
        const int ow = (int)(i % WO), oh = (int)((i / WO) % HO);
        const long long plane = i / ((long long)WO * HO);
        const float *ip = in + plane * H * W + (long long)(oh * stride) * W + ow * stride;
        float best = -1e38f;
        for (int kh = 0; kh < ksize; kh++)
            for (int kw = 0; kw < ksize; kw++) {
                const float v = ip[(long long)kh * W + kw];
                if (v > best) best = v;
            }
        out[i] = best;
    }
}

hipError_t launch_conv2d(const float *in, const float *ker, float *out, int N, int C, int H, int W, int CO, int KH, int KW,
                         int HO, int WO, int stride, int padding, hipStream_t st);
hipError_t launch_maxpool2d(const float *in, float *out, long long planes, int H, int W, int HO, int WO, int ksize, int stride,
                            hipStream_t st);

static unsigned tensor_grid(long long work_items) {
    const long long want = (work_items + TOPS_BLOCK - 1) / TOPS_BLOCK;
    const long long cap = 256 * 32;                                  // a few waves of workgroups per CU, grid-stride beyond
    return (unsigned)(want < 1 ? 1 : want > cap ? cap : want);
}

template <int OP>
static void launch_binary_op(const TensorIndexArgs &t, const float *a, const float *b, float *out, hipStream_t st) {
    // which form: t.sa / t.sb are element strides per (already collapsed) result dimension
    bool flat = true;
    long long run = 1;
    for (int d = t.nd - 1; d >= 0; d--) {
        if (t.shape[d] != 1 && (t.sa[d] != run || t.sb[d] != run)) flat = false;
        run *= t.shape[d];
    }
    if (flat) {
        const int vec = (((uintptr_t)a | (uintptr_t)b | (uintptr_t)out) & 15) == 0;
        hipLaunchKernelGGL(binary_flat_kernel<OP>, dim3(tensor_grid((t.n + 3) / 4)), dim3(TOPS_BLOCK), 0, st, a, b, out, t.n, vec);
    } else if (t.nd <= 2) {
        const long long rows = t.nd == 2 ? t.shape[0] : 1, cols = t.shape[t.nd - 1];
        const long long ars = t.nd == 2 ? t.sa[0] : 0, brs = t.nd == 2 ? t.sb[0] : 0;
        const long long acs = t.sa[t.nd - 1], bcs = t.sb[t.nd - 1];
        const bool vec = (cols & 3) == 0 && (acs == 0 || acs == 1) && (bcs == 0 || bcs == 1) && ((uintptr_t)out & 15) == 0 &&
                         (acs == 0 || ((((uintptr_t)a) & 15) == 0 && (ars & 3) == 0)) &&
                         (bcs == 0 || ((((uintptr_t)b) & 15) == 0 && (brs & 3) == 0));
        if (vec) {
            hipLaunchKernelGGL(binary_rowcol_vec_kernel<OP>, dim3(tensor_grid(rows * (cols >> 2))), dim3(TOPS_BLOCK), 0, st, a, b,
                               out, rows, cols >> 2, ars, (int)acs, brs, (int)bcs);
            return;
        }
        const long long strips = (cols + 4 * TOPS_BLOCK - 1) / (4 * TOPS_BLOCK);
        const long long items = rows * strips;
        hipLaunchKernelGGL(binary_rowcol_kernel<OP>, dim3((unsigned)(items > 65536 ? 65536 : items)), dim3(TOPS_BLOCK), 0, st,
                           a, b, out, rows, cols, ars, t.sa[t.nd - 1], brs, t.sb[t.nd - 1]);
    } else {
        hipLaunchKernelGGL(binary_general_kernel<OP>, dim3(tensor_grid(t.n)), dim3(TOPS_BLOCK), 0, st, t, a, b, out);
    }
}

hipError_t launch_tensor_binary(int op, const TensorIndexArgs &t, const float *a, const float *b, float *out, hipStream_t st) {
    switch (op) {
        case 0: launch_binary_op<0>(t, a, b, out, st); break;
        case 1: launch_binary_op<1>(t, a, b, out, st); break;
        case 2: launch_binary_op<2>(t, a, b, out, st); break;
        case 3: launch_binary_op<3>(t, a, b, out, st); break;
        default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

hipError_t launch_tensor_transpose(const TensorIndexArgs &t, const float *in, float *out, hipStream_t st) {
    // after collapsing: [batch, R, C] -> [batch, C, R] (or [R, C] -> [C, R]) goes through LDS tiles
    const bool swap_last_two =
        (t.nd == 2 && t.sa[0] == 1 && t.sa[1] == t.shape[0]) ||
        (t.nd == 3 && t.sa[1] == 1 && t.sa[2] == t.shape[1] && t.sa[0] == t.shape[1] * t.shape[2]);
    if (swap_last_two) {
        const long long batch = t.nd == 3 ? t.shape[0] : 1;
        const long long C = t.shape[t.nd - 2], R = t.shape[t.nd - 1];   // result is [.., C, R], source [.., R, C]
        const long long tiles = batch * ((R + TR_TILE - 1) / TR_TILE) * ((C + TR_TILE - 1) / TR_TILE);
        const dim3 gr((unsigned)(tiles > 262144 ? 262144 : tiles)), bl(TOPS_BLOCK);
        if ((R & 3) == 0 && (C & 3) == 0 && ((((uintptr_t)in) | ((uintptr_t)out)) & 15) == 0)
            hipLaunchKernelGGL(transpose_tiled_vec_kernel, gr, bl, 0, st, in, out, batch, R, C);
        else
            hipLaunchKernelGGL(transpose_tiled_kernel, gr, bl, 0, st, in, out, batch, R, C);
    } else {
        hipLaunchKernelGGL(transpose_general_kernel, dim3(tensor_grid(t.n)), dim3(TOPS_BLOCK), 0, st, t, in, out);
    }
    return hipGetLastError();
}

// KWT: the kernel's width when it is 1, 3, 5 or 7 (the row of products is unrolled, its loads in flight together), else 0.
// SQUARE: the kernel's height is KWT too, and a whole channel's patch is unrolled.
// CONV_COG: output channels per thread (4; 2 or 1 where the launch would otherwise leave the SIMDs a wave or two each).
template <int KWT, bool SQUARE, int CONV_COG>
__global__ __launch_bounds__(TOPS_BLOCK) void conv2d_group_kernel(const float *__restrict__ in, const float *__restrict__ ker,
                                                                  float *__restrict__ out, int N, int C, int H, int W, int CO, int KH,
                                                                  int KW, int HO, int WO, int stride, int padding) {
    const long long P = (long long)N * HO * WO;                      // positions
    const long long p = (long long)blockIdx.x * TOPS_BLOCK + threadIdx.x;
    const int co0 = (int)blockIdx.y * CONV_COG;                      // uniform: the kernel values come through scalar loads
    const bool live = p < P;
    const long long pc = live ? p : 0;
    const int ow = (int)(pc % WO), oh = (int)((pc / WO) % HO), n = (int)(pc / ((long long)WO * HO));
    const int h0 = oh * stride - padding, w0 = ow * stride - padding;
    const long long ksz = (long long)C * KH * KW;
    const float *kp[CONV_COG];
#pragma unroll
    for (int g = 0; g < CONV_COG; g++) kp[g] = ker + (long long)min(co0 + g, CO - 1) * ksz;   // (a channel past the last: computed, not stored)
    float sum[CONV_COG];
#pragma unroll
    for (int g = 0; g < CONV_COG; g++) sum[g] = 0.0f;
    const float *ip = in + (long long)n * C * H * W;
    int kidx = 0;
    for (int c = 0; c < C; c++, ip += (long long)H * W) {
        if (SQUARE) {
            float x[KWT > 0 ? KWT * KWT : 1];
#pragma unroll
            for (int kh = 0; kh < KWT; kh++) {
                const int h = h0 + kh;
                const bool hin = h >= 0 && h < H;
                const float *rowp = ip + (long long)(hin ? h : 0) * W;
#pragma unroll
                for (int kw = 0; kw < KWT; kw++) {
                    const int w = w0 + kw;
                    x[kh * KWT + kw] = (hin && w >= 0 && w < W) ? rowp[w] : 0.0f;
                }
            }
#pragma unroll
            for (int t = 0; t < KWT * KWT; t++)
#pragma unroll
                for (int g = 0; g < CONV_COG; g++) sum[g] += kp[g][kidx + t] * x[t];
            kidx += KWT * KWT;
            continue;
        }
        for (int kh = 0; kh < KH; kh++) {
            const int h = h0 + kh;
            const bool hin = h >= 0 && h < H;
            const float *rowp = ip + (long long)(hin ? h : 0) * W;
            if (KWT > 0) {
                float x[KWT > 0 ? KWT : 1];
#pragma unroll
                for (int kw = 0; kw < KWT; kw++) {
                    const int w = w0 + kw;
                    x[kw] = (hin && w >= 0 && w < W) ? rowp[w] : 0.0f;
                }
#pragma unroll
                for (int kw = 0; kw < KWT; kw++)
#pragma unroll
                    for (int g = 0; g < CONV_COG; g++) sum[g] += kp[g][kidx + kw] * x[kw];
                kidx += KWT;
            } else {
                for (int kw = 0; kw < KW; kw++, kidx++) {
                    const int w = w0 + kw;
                    const bool win = hin && w >= 0 && w < W;
                    const float x = win ? rowp[w] : 0.0f;
#pragma unroll
                    for (int g = 0; g < CONV_COG; g++) sum[g] += kp[g][kidx] * x;
                }
            }
        }
    }
    if (live) {
#pragma unroll
        for (int g = 0; g < CONV_COG; g++)
            if (co0 + g < CO) out[(((long long)n * CO + co0 + g) * HO + oh) * WO + ow] = sum[g];
    }
}

template <int KWT, bool SQUARE>
static void launch_conv2d_group(int cog, dim3 block, long long blocks, int CO, hipStream_t st, const float *in, const float *ker, float *out, int N,
                                int C, int H, int W, int KH, int KW, int HO, int WO, int stride, int padding) {
    const dim3 grid((unsigned)blocks, (unsigned)((CO + cog - 1) / cog));
    if (cog == 4) hipLaunchKernelGGL((conv2d_group_kernel<KWT, SQUARE, 4>), grid, block, 0, st, in, ker, out, N, C, H, W, CO, KH, KW, HO, WO, stride, padding);
    else if (cog == 2) hipLaunchKernelGGL((conv2d_group_kernel<KWT, SQUARE, 2>), grid, block, 0, st, in, ker, out, N, C, H, W, CO, KH, KW, HO, WO, stride, padding);
    else hipLaunchKernelGGL((conv2d_group_kernel<KWT, SQUARE, 1>), grid, block, 0, st, in, ker, out, N, C, H, W, CO, KH, KW, HO, WO, stride, padding);
}

hipError_t launch_conv2d(const float *in, const float *ker, float *out, int N, int C, int H, int W, int CO, int KH, int KW,
                         int HO, int WO, int stride, int padding, hipStream_t st) {
    const long long P = (long long)N * HO * WO, blocks = (P + TOPS_BLOCK - 1) / TOPS_BLOCK;
    // four output channels per thread share every input load; fewer where that would leave fewer than eight waves to a CU
    // (2048 on the device) to hide the loads behind
    const long long waves1 = blocks * (TOPS_BLOCK / 64) * CO;
    const int cog = waves1 >= 4 * 2048 ? 4 : waves1 >= 2 * 2048 ? 2 : 1;
    if (blocks <= 0x7FFFFFFFll && (CO + cog - 1) / cog <= 65535) {
        const dim3 block(TOPS_BLOCK);
        if (KW == 3 && KH == 3) launch_conv2d_group<3, true>(cog, block, blocks, CO, st, in, ker, out, N, C, H, W, KH, KW, HO, WO, stride, padding);
        else if (KW == 5 && KH == 5) launch_conv2d_group<5, true>(cog, block, blocks, CO, st, in, ker, out, N, C, H, W, KH, KW, HO, WO, stride, padding);
        else if (KW == 1) launch_conv2d_group<1, false>(cog, block, blocks, CO, st, in, ker, out, N, C, H, W, KH, KW, HO, WO, stride, padding);
        else if (KW == 3) launch_conv2d_group<3, false>(cog, block, blocks, CO, st, in, ker, out, N, C, H, W, KH, KW, HO, WO, stride, padding);
        else if (KW == 5) launch_conv2d_group<5, false>(cog, block, blocks, CO, st, in, ker, out, N, C, H, W, KH, KW, HO, WO, stride, padding);
        else if (KW == 7) launch_conv2d_group<7, false>(cog, block, blocks, CO, st, in, ker, out, N, C, H, W, KH, KW, HO, WO, stride, padding);
        else launch_conv2d_group<0, false>(cog, block, blocks, CO, st, in, ker, out, N, C, H, W, KH, KW, HO, WO, stride, padding);
        return hipGetLastError();
    }
    hipLaunchKernelGGL(conv2d_kernel, dim3(tensor_grid((long long)N * CO * HO * WO)), dim3(TOPS_BLOCK), 0, st, in, ker, out, N, C, H,
                       W, CO, KH, KW, HO, WO, stride, padding);
    return hipGetLastError();
}
hipError_t launch_maxpool2d(const float *in, float *out, long long planes, int H, int W, int HO, int WO, int ksize, int stride,
                            hipStream_t st) {
    hipLaunchKernelGGL(maxpool2d_kernel, dim3(tensor_grid(planes * HO * WO)), dim3(TOPS_BLOCK), 0, st, in, out, planes, H, W, HO, WO,
                       ksize, stride);
    return hipGetLastError();
}

}  // namespace born
