// Codebook-lookup operators: every weight is a BITS-wide index into a small
// table of centroids shared by the whole matrix.  One kernel covers the
// reference's operators of this family; they differ only in how a packed row is
// addressed and in which activation row meets which weight row:
//
//   kernel::quant4_gemm   src/kernel/kernel_quant4.cpp:18-47
//       out[m*N+n] = sum_k cb[nib((m*N+n), k)] * act[n*K+k]; the packed row of the
//       pair (m,n) starts at byte ((m*N+n)*K)/2, nibble k is the low half of byte
//       k/2 for even k.  One packed row PER OUTPUT, activation row chosen by n.
//   kernel::quant8_gemm   src/kernel/kernel_quant8.cpp:14-32
//       out[m*N+n] = sum_k cb[idx[n*K+k]] * act[m*K+k].
//   prod::gemv_quant4_tiled/_batch, gemv_quant8_tiled/_batch, gemv_quant_tiled/_batch
//       src/kernel/kernel_production.cpp:68-117, 334-353 (the scalar loops are the
//       semantics): Y[n*M+m] = scale * sum_k cb[idx(m,k)] * X[n*K+k], rows of
//       ceil(K*BITS/8) bytes; the 2-bit form maps codes 0,1,2,3 to -1,0,+1,+1.
//
// One wavefront owns one packed row and up to BT activation rows at a time.
// Lanes take 16-byte chunks of the row (128/BITS weights) with 128-bit loads when
// the row starts are 16-byte aligned, single elements otherwise.  The table sits
// in LDS; tables of at most 16 entries are replicated per lane so that a lookup
// never meets a bank conflict.  Partial sums meet through a DPP/shuffle
// reduction.  The traffic is the index bytes, read once per BT activation rows.

#include "tfq_internal.hpp"

#include <vector>

namespace tfq {

namespace {

constexpr int kWaves = 4;  // wavefronts (packed rows) per workgroup

struct LutArgs {
    const uint8_t* W;
    const float* X;
    float* Y;
    int64_t R;        // packed rows
    int64_t stride2;  // twice the byte distance between row starts (row r starts at (r*stride2)/2)
    int64_t xmod;     // activation row of packed row r is (r % xmod) + b
    int K, B;
    float scale;
};

template <int ENTRIES>
struct Table {
    float c[ENTRIES];
};

template <int BITS>
__device__ __forceinline__ float lookup(const float* tab, uint32_t idx, int lane) {
    if constexpr (BITS <= 4) return tab[idx * 64 + lane];
    else return tab[idx];
}

template <int BITS, int BT, bool VEC>
__global__ __launch_bounds__(kWaves * 64) void lut_rows_kernel(LutArgs a, Table<(1 << BITS)> cb) {
    constexpr int ENTRIES = 1 << BITS;
    constexpr int PER16 = 128 / BITS;  // weights in a 16-byte chunk
    constexpr uint32_t MASK = ENTRIES - 1;
    __shared__ float tab[BITS <= 4 ? ENTRIES * 64 : ENTRIES];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if constexpr (BITS <= 4) {
        for (int i = threadIdx.x; i < ENTRIES * 64; i += kWaves * 64) tab[i] = cb.c[i >> 6];
    } else {
        for (int i = threadIdx.x; i < ENTRIES; i += kWaves * 64) tab[i] = cb.c[i];
    }
    __syncthreads();
    const int64_t r = (int64_t)blockIdx.x * kWaves + wave;
    if (r >= a.R) return;
    const uint8_t* row = a.W + ((r * a.stride2) >> 1);
    const int64_t xrow0 = r % a.xmod;
    for (int b0 = 0; b0 < a.B; b0 += BT) {
        float acc[BT];
#pragma unroll
        for (int t = 0; t < BT; ++t) acc[t] = 0.0f;
        const float* xb[BT];
#pragma unroll
        for (int t = 0; t < BT; ++t) xb[t] = a.X + (xrow0 + (b0 + t < a.B ? b0 + t : b0)) * (int64_t)a.K;
        int kdone = 0;
        if constexpr (VEC) {
            const int chunks = a.K / PER16;
            for (int c = lane; c < chunks; c += 64) {
                const uint4 v = reinterpret_cast<const uint4*>(row)[c];
                const uint32_t wds[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
                for (int e4 = 0; e4 < PER16; e4 += 4) {
                    float w[4];
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const int bit = (e4 + j) * BITS;
                        w[j] = lookup<BITS>(tab, (wds[bit >> 5] >> (bit & 31)) & MASK, lane);
                    }
#pragma unroll
                    for (int t = 0; t < BT; ++t) {
                        const float4 x = reinterpret_cast<const float4*>(xb[t] + (int64_t)c * PER16)[e4 >> 2];
                        acc[t] = fmaf(w[0], x.x, acc[t]);
                        acc[t] = fmaf(w[1], x.y, acc[t]);
                        acc[t] = fmaf(w[2], x.z, acc[t]);
                        acc[t] = fmaf(w[3], x.w, acc[t]);
                    }
                }
            }
            kdone = chunks * PER16;
        }
        for (int k = kdone + lane; k < a.K; k += 64) {
            const int bit = k * BITS;
            const float w = lookup<BITS>(tab, ((uint32_t)row[bit >> 3] >> (bit & 7)) & MASK, lane);
#pragma unroll
            for (int t = 0; t < BT; ++t) acc[t] = fmaf(w, xb[t][k], acc[t]);
        }
#pragma unroll
        for (int t = 0; t < BT; ++t) {
            float s = acc[t];
#pragma unroll
            for (int m = 32; m >= 1; m >>= 1) s += __shfl_xor(s, m, 64);
            if (lane == 0 && b0 + t < a.B) a.Y[(int64_t)(b0 + t) * a.R + r] = s * a.scale;
        }
    }
}

// Packed-row lookup operators whose index width does not divide a register: 3, 6 and 12 bits
// (kernel::q3_gemm, q6_gemm, q12_gemm: src/kernel/kernel_q3.cpp:27-72, kernel_q6.cpp:28-68,
// kernel_q12.cpp:30-71), and the 24-bit float rows of kernel::q24_gemm (kernel_q24.cpp:28-68).
// All share quant4_gemm's convention: out[m*N+n] uses packed row (m*N+n), of ceil(K*BITS/8)
// bytes, against activation row n; indices are an LSB-first bit stream.  One wavefront per
// packed row; a lane takes 8 consecutive weights, which are exactly BITS bytes.
// BITS == 24: no table, a weight is the top 24 bits of a binary32, stored big-endian.
template <int BITS>
__global__ __launch_bounds__(kWaves * 64) void lutn_rows_kernel(const uint8_t* __restrict__ W, const float* __restrict__ tab_g,
                                                               const float* __restrict__ X, float* __restrict__ Y,
                                                               int64_t R, int N, int K) {
    extern __shared__ float tab[];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if constexpr (BITS != 24) {
        for (int i = threadIdx.x; i < (1 << BITS); i += kWaves * 64) tab[i] = tab_g[i];
        __syncthreads();
    }
    const int64_t r = (int64_t)blockIdx.x * kWaves + wave;
    if (r >= R) return;
    const int64_t row_bytes = ((int64_t)K * BITS + 7) / 8;
    const uint8_t* row = W + r * row_bytes;
    const float* x = X + (r % N) * (int64_t)K;
    float acc = 0.0f;
    for (int k0 = lane * 8; k0 < K; k0 += 64 * 8) {
        const uint8_t* p = row + (int64_t)k0 * BITS / 8;  // 8 weights start on a byte boundary
        const int cnt = K - k0 < 8 ? K - k0 : 8;
        const int64_t avail = row_bytes - (int64_t)k0 * BITS / 8;
        uint32_t w[BITS / 4 + 1] = {};
#pragma unroll
        for (int b = 0; b < BITS; ++b)
            if (b < avail) w[b >> 2] |= (uint32_t)p[b] << (8 * (b & 3));
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            if (j >= cnt) break;
            float v;
            if constexpr (BITS == 24) {
                const uint32_t b0 = (w[(3 * j) >> 2] >> (8 * ((3 * j) & 3))) & 0xFFu;
                const uint32_t b1 = (w[(3 * j + 1) >> 2] >> (8 * ((3 * j + 1) & 3))) & 0xFFu;
                const uint32_t b2 = (w[(3 * j + 2) >> 2] >> (8 * ((3 * j + 2) & 3))) & 0xFFu;
                v = __uint_as_float((b0 << 24) | (b1 << 16) | (b2 << 8));
            } else {
                const int pos = j * BITS, i = pos >> 5, sh = pos & 31;
                uint32_t idx = w[i] >> sh;
                if (sh + BITS > 32) idx |= w[i + 1] << (32 - sh);
                v = tab[idx & ((1u << BITS) - 1u)];
            }
            acc = fmaf(v, x[k0 + j], acc);
        }
    }
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) acc += __shfl_xor(acc, m, 64);
    if (lane == 0) Y[r] = acc;
}

// q24_encode / q24_decode (src/kernel/kernel_q24.cpp:28-45, 152-193): top 24 bits of the binary32, big-endian
__global__ void fp24_encode_kernel(const float* __restrict__ w, uint8_t* __restrict__ packed, int64_t count) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= count) return;
    const uint32_t u = __float_as_uint(w[i]);
    packed[3 * i] = (uint8_t)(u >> 24);
    packed[3 * i + 1] = (uint8_t)(u >> 16);
    packed[3 * i + 2] = (uint8_t)(u >> 8);
}

__global__ void fp24_decode_kernel(const uint8_t* __restrict__ packed, float* __restrict__ w, int64_t count) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= count) return;
    w[i] = __uint_as_float(((uint32_t)packed[3 * i] << 24) | ((uint32_t)packed[3 * i + 1] << 16) | ((uint32_t)packed[3 * i + 2] << 8));
}

template <int BITS, int BT>
void launch_bt(const LutArgs& a, const Table<(1 << BITS)>& cb, bool vec, hipStream_t s) {
    const dim3 grid((unsigned)((a.R + kWaves - 1) / kWaves)), block(kWaves * 64);
    if (vec) hipLaunchKernelGGL((lut_rows_kernel<BITS, BT, true>), grid, block, 0, s, a, cb);
    else hipLaunchKernelGGL((lut_rows_kernel<BITS, BT, false>), grid, block, 0, s, a, cb);
}

template <int BITS>
int run_lut(const LutArgs& a, const Table<(1 << BITS)>& cb, hipStream_t s) {
    if (a.R <= 0 || a.B <= 0) return TFQ_OK;
    if ((a.R + kWaves - 1) / kWaves > 0x7FFFFFFF) return fail(TFQ_ERR_SHAPE, "lookup matmul: too many packed rows for one launch");
    // 128-bit loads need 16-byte aligned row starts and activation rows.
    const bool vec = (uintptr_t)a.W % 16 == 0 && a.stride2 % 32 == 0 && (uintptr_t)a.X % 16 == 0 && a.K % 4 == 0 &&
                     a.K >= 128 / BITS;
    if (a.B >= 4) launch_bt<BITS, 4>(a, cb, vec, s);
    else if (a.B >= 2) launch_bt<BITS, 2>(a, cb, vec, s);
    else launch_bt<BITS, 1>(a, cb, vec, s);
    return hip_fail(hipGetLastError(), "lookup matmul launch");
}

// binary16 bits -> float on the host (detail::fp16_to_float, include/quant/detail/fp16.h:18-34)
float half_to_float_host(uint16_t h) {
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t ex = (h >> 10) & 0x1Fu, man = h & 0x3FFu, u;
    if (ex == 0) {
        if (man == 0) {
            u = sign;
        } else {
            int e = 113;
            while (!(man & 0x400u)) { man <<= 1; --e; }
            u = sign | ((uint32_t)e << 23) | ((man & 0x3FFu) << 13);
        }
    } else if (ex == 31) {
        u = sign | 0x7F800000u | (man << 13);
    } else {
        u = sign | ((ex + 112u) << 23) | (man << 13);
    }
    float f;
    __builtin_memcpy(&f, &u, 4);
    return f;
}

}  // namespace

// codebook: 8 or 64 floats (3, 6 bits), 4096 binary16 (12 bits), none (24 bits); device scratch for the table
int launch_lutn_gemm(int bits, const uint8_t* packed, const void* codebook, const float* act, float* out, int M, int N,
                     int K, hipStream_t s) {
    const int64_t R = (int64_t)M * N;
    if ((R + kWaves - 1) / kWaves > 0x7FFFFFFF) return fail(TFQ_ERR_SHAPE, "lookup matmul: too many packed rows for one launch");
    const dim3 grid((unsigned)((R + kWaves - 1) / kWaves)), block(kWaves * 64);
    if (bits == 24) {
        hipLaunchKernelGGL(lutn_rows_kernel<24>, grid, block, 0, s, packed, (const float*)nullptr, act, out, R, N, K);
        return hip_fail(hipGetLastError(), "lookup matmul launch");
    }
    const int entries = 1 << bits;
    std::vector<float> host(entries);
    for (int i = 0; i < entries; ++i)
        host[i] = bits == 12 ? half_to_float_host(static_cast<const uint16_t*>(codebook)[i]) : static_cast<const float*>(codebook)[i];
    float* tab = nullptr;
    TFQ_HIP(hipMalloc(&tab, entries * sizeof(float)));
    int rc = hip_fail(hipMemcpyAsync(tab, host.data(), entries * sizeof(float), hipMemcpyHostToDevice, s), "table upload");
    if (!rc) rc = hip_fail(hipStreamSynchronize(s), "table upload");  // `host` goes out of scope below
    if (!rc) {
        const size_t lds = entries * sizeof(float);
        if (bits == 3) hipLaunchKernelGGL(lutn_rows_kernel<3>, grid, block, lds, s, packed, tab, act, out, R, N, K);
        else if (bits == 6) hipLaunchKernelGGL(lutn_rows_kernel<6>, grid, block, lds, s, packed, tab, act, out, R, N, K);
        else hipLaunchKernelGGL(lutn_rows_kernel<12>, grid, block, lds, s, packed, tab, act, out, R, N, K);
        rc = hip_fail(hipGetLastError(), "lookup matmul launch");
        if (!rc) rc = hip_fail(hipStreamSynchronize(s), "lookup matmul");  // the table is freed below
    }
    (void)hipFree(tab);
    return rc;
}

int launch_fp24_convert(bool encode, const void* src, void* dst, int64_t count, hipStream_t s) {
    if (count <= 0) return TFQ_OK;
    const int64_t grid = (count + 255) / 256;
    if (grid > 0x7FFFFFFF) return fail(TFQ_ERR_SHAPE, "fp24: too many elements for one launch");
    if (encode) hipLaunchKernelGGL(fp24_encode_kernel, dim3((unsigned)grid), dim3(256), 0, s, (const float*)src, (uint8_t*)dst, count);
    else hipLaunchKernelGGL(fp24_decode_kernel, dim3((unsigned)grid), dim3(256), 0, s, (const uint8_t*)src, (float*)dst, count);
    return hip_fail(hipGetLastError(), "fp24 launch");
}

int launch_lut4_gemm(const uint8_t* packed, const uint16_t* cb16, const float* act, float* out, int M, int N, int K,
                     hipStream_t s) {
    Table<16> t;
    for (int i = 0; i < 16; ++i) t.c[i] = half_to_float_host(cb16[i]);
    LutArgs a{packed, act, out, (int64_t)M * N, (int64_t)K, (int64_t)N, K, 1, 1.0f};
    return run_lut<4>(a, t, s);
}

int launch_lut8_gemm(const uint8_t* idx, const float* cb, const float* act, float* out, int M, int N, int K,
                     hipStream_t s) {
    Table<256> t;
    for (int i = 0; i < 256; ++i) t.c[i] = cb[i];
    LutArgs a{idx, act, out, (int64_t)N, 2 * (int64_t)K, 1, K, M, 1.0f};
    return run_lut<8>(a, t, s);
}

int launch_lut_gemv_batch(int bits, const uint8_t* packed, const void* cb, float scale, const float* X, float* Y,
                          int M, int Nb, int K, hipStream_t s) {
    const int64_t row_bytes = ((int64_t)K * bits + 7) / 8;
    LutArgs a{packed, X, Y, (int64_t)M, 2 * row_bytes, 1, K, Nb, scale};
    if (bits == 2) {
        Table<4> t{{-1.0f, 0.0f, 1.0f, 1.0f}};
        return run_lut<2>(a, t, s);
    }
    if (bits == 4) {
        Table<16> t;
        for (int i = 0; i < 16; ++i) t.c[i] = half_to_float_host(static_cast<const uint16_t*>(cb)[i]);
        return run_lut<4>(a, t, s);
    }
    Table<256> t;
    for (int i = 0; i < 256; ++i) t.c[i] = static_cast<const float*>(cb)[i];
    return run_lut<8>(a, t, s);
}

}  // namespace tfq
