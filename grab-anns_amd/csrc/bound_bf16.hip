// Bounds for the symmetric pass of the kNN build, estimated on the bf16 matrix pipe.
//
// The symmetric pass (topk_gemm.hip) keeps, for every row, the keys at or below a per-row bound, and redoes the
// rows whose bound admitted fewer than kk keys: the bound decides how much work the pass does, never what it
// returns.  So the bound may be an estimate.  Here every row is set against an evenly spaced sample of the rows
// with squared distances computed from bf16 copies (centred on the sample's mean first, which no distance
// notices and which keeps bf16's eight bits for the part of a coordinate that differs between rows), sixteen
// times the rate of the fp32 matrix instructions; the fp32 pass over the same sample took a tenth of the build.
//
// The rank-th smallest estimate of a row would need a selection over all the sample columns.  Instead every
// accumulator position keeps the minimum of the columns it sees - 128 classes of columns (column index mod 128),
// 128 minima a row, a multiply-add and a minimum per distance - and the q-th smallest of the 128 minima stands in:
// q columns of q different classes lie at or below it, and with q well below 128 few of a row's nearest
// columns share a class, so it is the estimate of rank about q + q^2/256.
#include <algorithm>
#include <cmath>

#include "device_utils.hpp"
#include "topk_gemm.hpp"

namespace grab {

using namespace dev;

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 v8bf16;
typedef __attribute__((ext_vector_type(16))) float v16f;

constexpr uint32_t kDimP = 128;      // dimensions of the bf16 copies (zero beyond the row's end)
constexpr uint32_t kRows = 128;      // rows of a workgroup
constexpr uint32_t kCols = 128;      // sample columns of a step
constexpr uint32_t kPitch = 272;     // bytes of a column in LDS: 256 of data, 16 so that 16-byte reads of 8 consecutive columns cover all banks

// round to nearest, ties to even; the inputs are finite
__device__ __forceinline__ uint32_t bf16_bits(float x) {
    const uint32_t u = __float_as_uint(x);
    return (u + 0x7FFFu + ((u >> 16) & 1u)) >> 16;
}
__device__ __forceinline__ float bf16_value(uint32_t bits) { return __uint_as_float(bits << 16); }

// mean[k] = average of coordinate k over the sample rows (row i * n / count of the data), zero for k >= dim
__global__ void __launch_bounds__(256) sample_mean_kernel(const float* __restrict__ data, uint64_t n, uint32_t count, uint32_t dim,
                                                          float* __restrict__ mean) {
    __shared__ float part[256];
    const uint32_t k = blockIdx.x;  // one workgroup per coordinate
    float s = 0.0f;
    for (uint32_t i = threadIdx.x; i < count; i += 256) s += data[(size_t)((uint64_t)i * n / count) * dim + k];
    part[threadIdx.x] = s;
    __syncthreads();
    for (int w = 128; w > 0; w >>= 1) {
        if ((int)threadIdx.x < w) part[threadIdx.x] += part[threadIdx.x + w];
        __syncthreads();
    }
    if (threadIdx.x == 0) mean[k] = part[0] / (float)count;
}

// row i * n / count of the data (every row when count = n), centred, as bf16 in rows of 128 (zeros beyond dim), with the
// squared norm of what was stored; 16 lanes a row.  The loads are unconditional (clamped index) and the select
// comes after: a load under a condition would be a branch and a wait per element.
// SPLIT: a row of the output is 272 values - the 128 bf16 values as before (the high halves), then the 128 low halves,
// bf16 of what the high half left of the centred coordinate (high + low carry 16 of its 24 bits) - and `norm_full`
// receives the squared norm of the centred fp32 row itself.  The last 16 values carry h = -|row|^2 / 2 as three bf16
// pieces (all 24 bits) for a 16-wide k-step of its own: as a column (1, 1, 1, h0, h1, h2, 0, 0), as a row
// (h0, h1, h2, 1, 1, 1, 0, 0), so that row . column of the extended vectors is a.b - |a|^2/2 - |b|^2/2, minus half
// the squared distance, straight out of the matrix instructions.
template <bool SPLIT>
__global__ void __launch_bounds__(256) rows_bf16_kernel(const float* __restrict__ data, uint64_t n, uint32_t count, uint32_t dim,
                                                        const float* __restrict__ mean, uint16_t* __restrict__ out,
                                                        float* __restrict__ norm, float* __restrict__ norm_full) {
    const uint32_t g = (blockIdx.x * 256 + threadIdx.x) >> 4, j = threadIdx.x & 15;
    const bool live = g < count;
    const uint32_t gi = min(g, count - 1u);
    const float* row = data + (size_t)(count == n ? (uint64_t)gi : (uint64_t)gi * n / count) * dim;
    float x[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        const uint32_t k = min(8u * j + (uint32_t)e, dim - 1u);
        x[e] = row[k] - mean[k];
    }
    float sq = 0.0f, sq_full = 0.0f;
    uint32_t w[4], wl[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        uint32_t pair = 0, pair_lo = 0;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const bool in = 8u * j + 2u * e + h < dim;
            const uint32_t b = in ? bf16_bits(x[2 * e + h]) : 0u;
            const float v = bf16_value(b);
            sq = __builtin_fmaf(v, v, sq);
            pair |= b << (16 * h);
            if (SPLIT) {
                const float xf = in ? x[2 * e + h] : 0.0f;
                sq_full = __builtin_fmaf(xf, xf, sq_full);
                pair_lo |= (in ? bf16_bits(xf - v) : 0u) << (16 * h);  // the difference is exact in fp32
            }
        }
        w[e] = pair;
        wl[e] = pair_lo;
    }
    constexpr uint32_t kOut = SPLIT ? 2 * kDimP + 16 : kDimP;
    if (live) *reinterpret_cast<uint4*>(out + (size_t)g * kOut + 8u * j) = make_uint4(w[0], w[1], w[2], w[3]);
    if (SPLIT && live) *reinterpret_cast<uint4*>(out + (size_t)g * kOut + kDimP + 8u * j) = make_uint4(wl[0], wl[1], wl[2], wl[3]);
#pragma unroll
    for (int m = 1; m < 16; m <<= 1) {
        sq += __shfl_xor(sq, m, 64);
        if (SPLIT) sq_full += __shfl_xor(sq_full, m, 64);
    }
    if (live && j == 0) norm[g] = sq;
    if (SPLIT && live && j == 0) {
        norm_full[g] = sq_full;
        const float h = -0.5f * sq_full;
        const uint32_t h0 = bf16_bits(h);
        const float r1 = h - bf16_value(h0);  // exact, as the next one
        const uint32_t h1 = bf16_bits(r1);
        const uint32_t h2 = bf16_bits(r1 - bf16_value(h1));
        const uint32_t one = 0x3F80u;
        *reinterpret_cast<uint4*>(out + (size_t)g * kOut + 2 * kDimP) = make_uint4(one | (one << 16), one | (h0 << 16), h1 | (h2 << 16), 0u);
        *reinterpret_cast<uint4*>(out + (size_t)g * kOut + 2 * kDimP + 8) = make_uint4(h0 | (h1 << 16), h2 | (one << 16), one | (one << 16), 0u);
    }
}

// Workgroup = 8 waves (two per SIMD, so that one's minima run beside the other's matrix instructions and waits), 128
// rows against all sample columns, 128 columns a step.  Wave (wr, wc) owns rows wr*32..+31 and, of every step, columns
// wc*64..+63: 2 blocks of 32 x 32.  A row block's operands stay in registers for the whole sweep (lane (l32, half) holds,
// for k-step s, the 8 values k = 16 s + 8 half .. + 7 of row l32; the columns use the same split of k, so every product
// is formed once).  The columns of a step are staged in LDS, the next step's in flight meanwhile.  Accumulator register
// v of lane (l32, half): row (v & 3) + 8 (v >> 2) + 4 half, column l32.
constexpr uint32_t kSweepWaves = 8;
__global__ void __launch_bounds__(64 * kSweepWaves, 1) bound_sweep_kernel(const uint16_t* __restrict__ A, uint32_t pitchA, uint32_t M,
                                                                        const uint16_t* __restrict__ B, const float* __restrict__ normB,
                                                                        uint32_t S, float* __restrict__ minima) {
    __shared__ __align__(16) uint8_t s_b[2][kCols * kPitch];
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, wr = wave >> 1, wc = wave & 1;
    const uint32_t l32 = lane & 31, half = lane >> 5;
    const uint32_t row0 = blockIdx.x * kRows;

    v8bf16 afr[8];
    {
        const uint16_t* x = A + (size_t)min(row0 + wr * 32 + l32, M - 1u) * pitchA + 8u * half;
#pragma unroll
        for (int s = 0; s < 8; ++s) afr[s] = __builtin_bit_cast(v8bf16, *reinterpret_cast<const uint4*>(x + 16 * s));
    }

    float mins[2][16];
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) mins[j][v] = __builtin_inff();

    // a step's columns: 128 x 16 pieces of 16 bytes, 4 pieces a thread, a column's pieces by consecutive threads
    const uint32_t steps = (S + kCols - 1) / kCols;
    uint4 st0, st1, st2, st3;
    auto piece_of = [&](uint32_t u) { return tid + 64u * kSweepWaves * u; };
    auto load_piece = [&](uint32_t step, uint32_t piece) {
        const uint32_t col = step * kCols + (piece >> 4);
        return *reinterpret_cast<const uint4*>(B + (size_t)min(col, S - 1u) * kDimP + 8u * (piece & 15u));
    };
    auto store_piece = [&](uint32_t buf, uint32_t piece, uint4 v) {
        *reinterpret_cast<uint4*>(&s_b[buf][(piece >> 4) * kPitch + 16u * (piece & 15u)]) = v;
    };
#define fetch(step_)                            \
    do {                                        \
        st0 = load_piece(step_, piece_of(0));   \
        st1 = load_piece(step_, piece_of(1));   \
        st2 = load_piece(step_, piece_of(2));   \
        st3 = load_piece(step_, piece_of(3));   \
    } while (0)
#define park(buf_)                              \
    do {                                        \
        store_piece(buf_, piece_of(0), st0);    \
        store_piece(buf_, piece_of(1), st1);    \
        store_piece(buf_, piece_of(2), st2);    \
        store_piece(buf_, piece_of(3), st3);    \
    } while (0)
    fetch(0);
    park(0);
    __syncthreads();
    for (uint32_t step = 0; step < steps; ++step) {
        const uint32_t buf = step & 1u;
        const uint32_t next = min(step + 1, steps - 1u);  // the last step fetches its own columns once more, into the buffer nobody reads
        v16f acc[2];
        const v16f zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        // the next step's columns travel while this step's matrix instructions run, and are parked in the other buffer,
        // which nobody reads (the barrier below closed the step before)
        fetch(next);
        float nb[2];
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const uint32_t col = step * kCols + wc * 64 + j * 32 + l32;
            nb[j] = col < S ? normB[col] : __builtin_inff();  // columns past the sample's end never hold a minimum
        }
#pragma unroll
        for (int s = 0; s < 8; ++s) {
            v8bf16 bfr[2];
#pragma unroll
            for (int j = 0; j < 2; ++j)
                bfr[j] = __builtin_bit_cast(v8bf16, *reinterpret_cast<const uint4*>(&s_b[buf][(wc * 64 + j * 32 + l32) * kPitch + 32u * s + 16u * half]));
#pragma unroll
            for (int j = 0; j < 2; ++j) acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(afr[s], bfr[j], s == 0 ? zero : acc[j], 0, 0, 0);
        }
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) mins[j][v] = fminf(mins[j][v], __builtin_fmaf(-2.0f, acc[j][v], nb[j]));
        park(buf ^ 1u);
        __syncthreads();  // the present step is closed before its buffer is written again, the next one's columns are all there
    }
#undef fetch
#undef park
    // minima[row][class]: class = column index mod 128
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const uint32_t row = row0 + wr * 32 + (v & 3) + 8 * (v >> 2) + 4 * half;
            if (row < M) minima[(size_t)row * kCols + wc * 64 + j * 32 + l32] = mins[j][v];
        }
}

// bound[row] = |row|^2 + the q-th smallest of the row's 128 minima (of |column|^2 - 2 row.column), not below zero; a wave a row
__global__ void __launch_bounds__(256) bound_select_kernel(const float* __restrict__ minima, const float* __restrict__ normA,
                                                           uint32_t M, uint32_t q, float* __restrict__ bound) {
    __shared__ __align__(16) float s_v[4][kCols];
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t row = blockIdx.x * 4 + wave;
    if (row >= M) return;  // whole waves; no barrier below
    const float a = minima[(size_t)row * kCols + lane], b = minima[(size_t)row * kCols + 64 + lane];
    s_v[wave][lane] = a;
    s_v[wave][64 + lane] = b;
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    // place of a value = values that are smaller, or equal at a lower index
    uint32_t ra = 0, rb = 0;
    const float4* v4 = reinterpret_cast<const float4*>(s_v[wave]);
#pragma unroll 4
    for (uint32_t c = 0; c < kCols / 4; ++c) {
        const float4 v = v4[c];
        const float e[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (uint32_t u = 0; u < 4; ++u) {
            const uint32_t at = 4 * c + u;
            ra += (e[u] < a || (e[u] == a && at < lane)) ? 1u : 0u;
            rb += (e[u] < b || (e[u] == b && at < 64 + lane)) ? 1u : 0u;
        }
    }
    const float na = normA[row];
    if (ra == q - 1) bound[row] = fmaxf(a + na, 0.0f);
    if (rb == q - 1) bound[row] = fmaxf(b + na, 0.0f);
}

}  // namespace

// classes of sample columns that keep a minimum each, and with it the largest rank this estimate stands in for
uint32_t bf16_bound_classes() { return kCols; }

// Bounds of the rows of `data` (n x dim fp32, dim <= 128, L2) for the symmetric pass: for every row an estimate of
// its distance to about the rank-th nearest of `n_sample` evenly spaced rows.  `workspace` holds
// bf16_bound_workspace_bytes(n, n_sample) bytes.  Everything is queued on `stream`; nothing is awaited.
size_t bf16_bound_workspace_bytes(size_t n, uint32_t n_sample) {
    return 512 + (size_t)n_sample * kDimP * 2 + (size_t)n_sample * 4 + n * 8 + (n + kSplitPadRows) * (size_t)(2 * kDimP + 16) * 2 + n * (size_t)kCols * 4 + 1024;
}

int bf16_bounds_async(const float* data, uint32_t n, uint32_t dim, uint32_t n_sample, uint32_t rank, void* workspace, float* bound,
                      hipStream_t stream, const uint16_t** split_rows, const float** centred_norms) {
    GRAB_REQUIRE(data && workspace && bound, "null pointer");
    GRAB_REQUIRE(dim >= 1 && dim <= kDimP && n >= 1 && n_sample >= 1 && n_sample <= n, "internal: bf16 bounds for %u x %u rows, %u sample rows", n, dim, n_sample);
    // the q-th smallest of the class minima is the estimate of rank about q + q^2 / 256: the q whose expected rank is `rank`
    uint32_t q = 1;
    while (q < kCols / 2 && (double)kCols * (1.0 - std::pow(1.0 - 1.0 / kCols, (double)rank)) > (double)q + 0.5) ++q;
    char* ws = static_cast<char*>(workspace);
    float* mean = reinterpret_cast<float*>(ws);
    ws += 512;
    uint16_t* sample = reinterpret_cast<uint16_t*>(ws);
    ws += (size_t)n_sample * kDimP * 2;
    float* sample_norm = reinterpret_cast<float*>(ws);
    ws += (size_t)n_sample * 4;
    float* row_norm = reinterpret_cast<float*>(ws);
    ws += (size_t)n * 4;
    float* row_norm_full = reinterpret_cast<float*>(ws);
    ws += (size_t)n * 4;
    ws = reinterpret_cast<char*>((reinterpret_cast<uintptr_t>(ws) + 255) & ~(uintptr_t)255);
    uint16_t* rows = reinterpret_cast<uint16_t*>(ws);
    ws += (size_t)(n + kSplitPadRows) * (2 * kDimP + 16) * 2;
    float* minima = reinterpret_cast<float*>((reinterpret_cast<uintptr_t>(ws) + 255) & ~(uintptr_t)255);
    GRAB_HIP(hipMemsetAsync(mean, 0, 512, stream));
    // rows of zeros behind the last one: the symmetric pass reads whole column tiles
    GRAB_HIP(hipMemsetAsync(rows + (size_t)n * (2 * kDimP + 16), 0, (size_t)kSplitPadRows * (2 * kDimP + 16) * 2, stream));
    hipLaunchKernelGGL(sample_mean_kernel, dim3(dim), dim3(256), 0, stream, data, (uint64_t)n, n_sample, dim, mean);
    hipLaunchKernelGGL(rows_bf16_kernel<false>, dim3((uint32_t)(((size_t)n_sample * 16 + 255) / 256)), dim3(256), 0, stream, data, (uint64_t)n,
                       n_sample, dim, mean, sample, sample_norm, (float*)nullptr);
    hipLaunchKernelGGL(rows_bf16_kernel<true>, dim3((uint32_t)(((size_t)n * 16 + 255) / 256)), dim3(256), 0, stream, data, (uint64_t)n, n, dim, mean,
                       rows, row_norm, row_norm_full);
    hipLaunchKernelGGL(bound_sweep_kernel, dim3((n + kRows - 1) / kRows), dim3(64 * kSweepWaves), 0, stream, rows, 2 * kDimP + 16, n, sample, sample_norm, n_sample,
                       minima);
    hipLaunchKernelGGL(bound_select_kernel, dim3((n + 3) / 4), dim3(256), 0, stream, minima, row_norm, n, q, bound);
    GRAB_HIP(hipGetLastError());
    if (split_rows) *split_rows = rows;
    if (centred_norms) *centred_norms = row_norm_full;
    return GRAB_OK;
}

}  // namespace grab
