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
