// Producer + per-token quantiser in one pass over the activation.
//
// Inside the DiT block the input of a quantised linear is produced by a row-local operation:
//   * LayerNorm (fp32 statistics) followed by a per-column multiply-add -- the adaLN modulation
//     norm(x) * (1 + scale) + shift in front of the self-attention and FFN projections, or the
//     LayerNorm's own weight / bias in front of the cross-attention projections;
//   * GELU (tanh form) between the two FFN linears.
// Run eagerly, the producer writes a bf16 [M, K] tensor that the quantiser reads back; under the
// reference's torch.compile (dax/adapters/wan/functional.py:33-36) Inductor fuses the quantiser's
// row reduction (dax/quant/nn/dynamic/functional.py:124-129) into the producing kernel.  These
// kernels are that fusion written out: one wavefront owns a row, keeps it in VGPRs, applies the
// producer in fp32, rounds to bf16 exactly where the unfused graph would (the value the reference
// quantises is the bf16 tensor), and then runs the same abs-max / scale / leaf-quantiser code as
// quant_rows.hip.  The bf16 tensor itself is only written when the caller asks for it.
//
// HBM traffic: 2 B read + 1 B written per element (+ 2 B when the bf16 result is wanted), against
// 2 + 2 + 2 + 1 for producer and quantiser run separately.  The GELU form is VALU-bound on gfx950
// (one v_exp_f32 and one v_rcp_f32 per element), not HBM-bound.
#include <type_traits>

#include "quant_rows.h"

namespace daxq {

enum { PRE_LN = 1, PRE_GELU = 2 };

// v_dot2_f32_bf16 d, a, b, c: both products of the bf16 pairs a and b, exact, added to the fp32 value c.  The compiler
// only selects the form whose destination is the addend (v_dot2c), which costs x - mean a copy per element, so the
// instruction is written out -- with its hazards: a different VALU instruction needs three wait states behind a DOT
// instruction before it reads the result and four before it overwrites it, and the compiler keeps those only for
// instructions it can see (the consumer of a single-instruction asm statement was once scheduled directly behind it
// and read the register's old value).  Hence whole chunks per statement, closed by four wait states, and results that
// no input register may share.
// Row sums of a chunk: sum += x, sq += x * x over its eight values (a DOT reading the previous DOT's result as its
// addend needs no wait; dot_sums_done() closes the chain before anything else reads the sums).
__device__ __forceinline__ void dot_sums(const uint4& v, float& sum, float& sq) {
    asm("v_dot2_f32_bf16 %0, %2, %6, %0\n\tv_dot2_f32_bf16 %1, %2, %2, %1\n\t"
        "v_dot2_f32_bf16 %0, %3, %6, %0\n\tv_dot2_f32_bf16 %1, %3, %3, %1\n\t"
        "v_dot2_f32_bf16 %0, %4, %6, %0\n\tv_dot2_f32_bf16 %1, %4, %4, %1\n\t"
        "v_dot2_f32_bf16 %0, %5, %6, %0\n\tv_dot2_f32_bf16 %1, %5, %5, %1"
        : "+v"(sum), "+v"(sq)
        : "v"(v.x), "v"(v.y), "v"(v.z), "v"(v.w), "v"(0x3f803f80u));
}
__device__ __forceinline__ void dot_sums_done(float& sum, float& sq) { asm volatile("s_nop 3" : "+v"(sum), "+v"(sq)); }
// f[e] = x[e] + c for the eight values of a chunk: the pair times (1, 0) or (0, 1) plus c, one instruction per element.
// (A non-finite neighbour turns the element into NaN through its zero product; the callers' rows are NaN throughout
// then anyway, their mean being non-finite.)
__device__ __forceinline__ void dot_add8(const uint4& v, float c, float (&f)[8]) {
    asm("v_dot2_f32_bf16 %0, %8, %12, %14\n\tv_dot2_f32_bf16 %1, %8, %13, %14\n\t"
        "v_dot2_f32_bf16 %2, %9, %12, %14\n\tv_dot2_f32_bf16 %3, %9, %13, %14\n\t"
        "v_dot2_f32_bf16 %4, %10, %12, %14\n\tv_dot2_f32_bf16 %5, %10, %13, %14\n\t"
        "v_dot2_f32_bf16 %6, %11, %12, %14\n\tv_dot2_f32_bf16 %7, %11, %13, %14\n\t"
        "s_nop 3"
        : "=&v"(f[0]), "=&v"(f[1]), "=&v"(f[2]), "=&v"(f[3]), "=&v"(f[4]), "=&v"(f[5]), "=&v"(f[6]), "=&v"(f[7])
        : "v"(v.x), "v"(v.y), "v"(v.z), "v"(v.w), "v"(0x00003f80u), "v"(0x3f800000u), "v"(c));
}

__device__ __forceinline__ void unpack8(const uint4& v, float (&f)[8]) {
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int h = 0; h < 4; ++h) {
        f[2 * h] = __uint_as_float(w[h] << 16);
        f[2 * h + 1] = __uint_as_float(w[h] & 0xffff0000u);
    }
}

__device__ __forceinline__ uint4 pack8(const float (&f)[8]) {
    return make_uint4(pack_bf16_rne(f[0], f[1]), pack_bf16_rne(f[2], f[3]), pack_bf16_rne(f[4], f[5]),
                      pack_bf16_rne(f[6], f[7]));
}

// The row stays packed (bf16 pairs) between the passes over it.  Without this the compiler keeps the unpacked
// fp32 copies of one pass alive for the next one, three times the registers, and the kernel loses half of its
// wavefronts per SIMD.
template <int N>
__device__ __forceinline__ void forget_values(uint4 (&v)[N]) {
#pragma unroll
    for (int i = 0; i < N; ++i) asm volatile("" : "+v"(v[i].x), "+v"(v[i].y), "+v"(v[i].z), "+v"(v[i].w));
}

// gelu(x, approximate="tanh") = 0.5 x (1 + tanh(u)), u = sqrt(2/pi) (x + 0.044715 x^3), evaluated as
// x / (1 + exp(-2u)): the same function without the cancellation in 1 + tanh(u) for negative x.
__device__ __forceinline__ float gelu_tanh_f32(float x) {
    // exp(-2u) = exp2(x * (c1 + c2 x^2)) with c1 = -2 log2(e) sqrt(2/pi), c2 = 0.044715 c1: three operations in
    // front of the v_exp_f32 instead of six
    constexpr float kC1 = -2.0f * 1.4426950408889634f * 0.7978845608028654f, kC2 = kC1 * 0.044715f;
    const float t = x * __builtin_fmaf(x * x, kC2, kC1);
    const float e = __builtin_amdgcn_exp2f(t);   // exp(-2u); +inf for very negative x
    return x * __builtin_amdgcn_rcpf(1.0f + e);  // x * 0 = -0 there, as the limit
}

// One wavefront per row, 4 rows per workgroup pass, grid-stride over row quads.
// PRE_LN: y = bf16( ((x - mean) * rstd) * mul[g][c] + add[g][c] ), g = row / rows_per_group; the two
//         vectors of the workgroup's current group are staged in LDS (mul / add may be null: 1 / 0).
// PRE_GELU: y = bf16( gelu_tanh(x) ).
// Requires k % 8 == 0, 16-byte aligned rows of x (and y), 8-byte aligned rows of q, kfill/8 <= NCH*64.
// The quantise-only LayerNorm form for rows of up to 12 x 64 chunks holds two rows (the current and the requested
// next one); rows of whole 512-element columns take ln_rows_exact below instead.
template <int NCH, int FMT, int PRE, bool WRITE_Y>
__global__ __launch_bounds__(256, (PRE == PRE_LN && NCH <= 12 && !WRITE_Y) ? 2 : 1) void fused_rows_wave(
    const uint16_t* __restrict__ x, int64_t m, int k, int64_t ld_x, const float* __restrict__ mul,
    const float* __restrict__ add, int64_t rows_per_group, float eps, uint16_t* __restrict__ y, int64_t ld_y,
    uint8_t* __restrict__ q, int64_t ld_q, int kfill, float* __restrict__ scale, float qmax) {
    // PRE_LN: mul then add, each in the order the lanes read them: per 64 chunks of 8 elements, the first halves of
    // the 64 chunks, then the second halves, so that one 16-byte read per lane covers 1 KB without a gap (the plain
    // order makes the lanes read 16 bytes every 32 and half of the banks collide)
    extern __shared__ __attribute__((aligned(16))) float s_vec[];
    const int kpad = ((k + 511) >> 9) << 9;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int nch = k >> 3;
    const int npad = kfill >> 3;  // columns [k, kfill) are written as zeros
    int64_t staged = -1;
    // The resident LayerNorm form requests the wavefront's next row before it works on the current one.
    constexpr bool AHEAD = PRE == PRE_LN && NCH <= 12;
    auto load_row = [&](int64_t r, uint4 (&dst)[NCH]) {
        const uint4* xr = reinterpret_cast<const uint4*>(x + r * ld_x);
#pragma unroll
        for (int i = 0; i < NCH; ++i) {
            const int c = i * 64 + lane;
            dst[i] = c < nch ? load_stream_16(xr + c) : make_uint4(0, 0, 0, 0);
        }
    };
    uint4 v[NCH], nv[AHEAD ? NCH : 1];
    if constexpr (AHEAD) {
        if ((int64_t)blockIdx.x * 4 + wave < m) load_row((int64_t)blockIdx.x * 4 + wave, v);
    }

    for (int64_t row0 = (int64_t)blockIdx.x * 4; row0 < m; row0 += (int64_t)gridDim.x * 4) {
        const int64_t row = row0 + wave;
        if constexpr (PRE == PRE_LN) {
            // the group of the quad's first row is staged; a wave whose row lies in another group
            // (a quad that straddles a boundary) reads the vectors from memory instead
            const int64_t g0 = row0 / rows_per_group;
            if (g0 != staged) {
                __syncthreads();  // everyone is done with the previous group's vectors
                for (int e = threadIdx.x; e < k; e += 256) {
                    const int c = e >> 3;
                    const int pos = (((((c >> 6) << 1) + ((e >> 2) & 1)) * 64 + (c & 63)) << 2) | (e & 3);
                    s_vec[pos] = mul ? mul[g0 * k + e] : 1.0f;
                    s_vec[kpad + pos] = add ? add[g0 * k + e] : 0.0f;
                }
                staged = g0;
                __syncthreads();
            }
        }
        if (row >= m) continue;

        if constexpr (AHEAD) {
            const int64_t next = row + (int64_t)gridDim.x * 4;
            if (next < m) load_row(next, nv);
        } else {
            load_row(row, v);
        }

        if constexpr (PRE == PRE_LN) {
            // Mean and biased variance in fp32.  Both row sums come straight from the packed bf16 pairs: v_dot2_f32_bf16
            // multiplies two pairs exactly and adds the products to an fp32 accumulator, so sum(x) = dot(x, 1) and
            // sum(x^2) = dot(x, x) cost one instruction per pair each, where unpacking, subtracting the mean and
            // squaring cost five per element.  var = E[x^2] - mean^2 loses bits when the mean is large against the
            // spread (the two terms cancel), so that form is kept only while mean^2 <= 7 var (the error of the sums,
            // at most 40 roundings per lane, is then amplified eightfold at worst: 2e-5 of var, 1e-5 of rstd, a 400th
            // of a bf16 step); any other row -- large offset, constant, non-finite -- takes the second pass over the
            // registers with the mean subtracted first.  The choice is uniform over the wavefront.
            float sum = 0.0f, sq = 0.0f;
#pragma unroll
            for (int i = 0; i < NCH; ++i) dot_sums(v[i], sum, sq);  // padding chunks are zero and add nothing
            dot_sums_done(sum, sq);
            float mean = wave_sum_f32(sum) / (float)k;
            float var = wave_sum_f32(sq) / (float)k - mean * mean;
            if (!(mean * mean <= 7.0f * var)) {
                // The deviations from the first mean also give what that mean is off by: a plain fp32 sum of K values
                // near 1000 is uncertain by a few units, i.e. the mean by 1e-3, which is a large part of an output
                // that lies close to zero.  mean += sum(d) / K, var = sum(d^2) / K - (sum(d) / K)^2.
                float sd = 0.0f, ssq = 0.0f;
#pragma unroll
                for (int i = 0; i < NCH; ++i) {
                    if (i * 64 + lane < nch) {
                        float f[8];
                        unpack8(v[i], f);
#pragma unroll
                        for (int e = 0; e < 8; ++e) {
                            const float d = f[e] - mean;
                            sd += d;
                            ssq += d * d;
                        }
                    }
                }
                const float dm = wave_sum_f32(sd) / (float)k;
                var = wave_sum_f32(ssq) / (float)k - dm * dm;
                mean += dm;
            }
            forget_values(v);
            const float rstd = 1.0f / sqrtf(var + eps);  // IEEE sqrt and division
            const int64_t g = row / rows_per_group;
            // The two forms of the pass are separate loops, chosen once per row.  With the choice inside the loop the
            // registers of the two vectors are written by global loads on one path and by LDS reads on the other, and
            // the compiler then waits for every load in flight -- the requested next row among them -- before each
            // chunk's LDS reads.
            auto modulate = [&](auto IN_LDS) __attribute__((always_inline)) {
#pragma unroll
                for (int i = 0; i < NCH; ++i) {
                    const int c = i * 64 + lane;
                    if (c < nch) {
                        float f[8], a[8], b[8];
                        dot_add8(v[i], -mean, f);  // x - mean
                        if constexpr (decltype(IN_LDS)::value) {
                            const float* sv = s_vec + (i * 128 + lane) * 4;
                            const float4 a0 = *reinterpret_cast<const float4*>(sv);
                            const float4 a1 = *reinterpret_cast<const float4*>(sv + 256);
                            const float4 b0 = *reinterpret_cast<const float4*>(sv + kpad);
                            const float4 b1 = *reinterpret_cast<const float4*>(sv + kpad + 256);
                            a[0] = a0.x, a[1] = a0.y, a[2] = a0.z, a[3] = a0.w, a[4] = a1.x, a[5] = a1.y, a[6] = a1.z, a[7] = a1.w;
                            b[0] = b0.x, b[1] = b0.y, b[2] = b0.z, b[3] = b0.w, b[4] = b1.x, b[5] = b1.y, b[6] = b1.z, b[7] = b1.w;
                        } else {
#pragma unroll
                            for (int e = 0; e < 8; ++e) {
                                a[e] = mul ? mul[g * k + c * 8 + e] : 1.0f;
                                b[e] = add ? add[g * k + c * 8 + e] : 0.0f;
                            }
                        }
#pragma unroll
                        for (int e = 0; e < 8; ++e) {
                            // the normalised value rounded to fp32, then one fused multiply-add with the two vectors
                            const float xh = __fmul_rn(f[e], rstd);
                            f[e] = __builtin_fmaf(xh, a[e], b[e]);
                        }
                        v[i] = pack8(f);
                    }
                }
            };
            if (g == staged) modulate(std::true_type{});
            else modulate(std::false_type{});
        } else {
#pragma unroll
            for (int i = 0; i < NCH; ++i) {
                if (i * 64 + lane < nch) {
                    float f[8];
                    unpack8(v[i], f);
#pragma unroll
                    for (int e = 0; e < 8; ++e) f[e] = gelu_tanh_f32(f[e]);
                    v[i] = pack8(f);
                }
            }
        }

        if constexpr (WRITE_Y) {
            uint4* yr = reinterpret_cast<uint4*>(y + row * ld_y);
#pragma unroll
            for (int i = 0; i < NCH; ++i) {
                const int c = i * 64 + lane;
                if (c < nch) yr[c] = v[i];
            }
        }

        // ---- from here on: the per-token quantiser of quant_rows.hip on the bf16 values
        uint32_t mx = 0;
#pragma unroll
        for (int i = 0; i < NCH; ++i) mx = chunk_absmax(mx, v[i]);
        uint32_t amax = (mx & 0xffffu) > (mx >> 16) ? (mx & 0xffffu) : (mx >> 16);
        amax = wave_max_u32(amax);
        const float s = scale_from_amax_bits<true>(amax, qmax);
        if (lane == 0) scale[row] = s;
        const float inv = 1.0f / s;
        uint2* qr = reinterpret_cast<uint2*>(q + row * ld_q);
#pragma unroll
        for (int i = 0; i < NCH; ++i) {
            const int c = i * 64 + lane;
            if (c < nch) {
                store_stream_8(qr + c, quant_chunk<FMT, false, DAXQ_BF16, false>(v[i], s, inv));  // own scale at the format's maximum: no clamp
            } else if (c < npad) {
                store_stream_8(qr + c, make_uint2(0, 0));
            }
        }
        if constexpr (AHEAD) {
#pragma unroll
            for (int i = 0; i < NCH; ++i) v[i] = nv[i];
        }
    }
}

// The LayerNorm form for rows of exactly NCOL x 512 elements (every lane owns NCOL whole chunks), quantised bytes only,
// groups of a multiple of four rows (the four rows of a workgroup pass share the staged vectors): the shapes the DiT
// blocks have.  Against fused_rows_wave it has no lane predicates and no path that reads the vectors from memory, the row
// number is a scalar (row base in SGPRs, one lane offset for all chunks), and the current and the requested row swap
// roles from one pass to the next instead of being copied.  Same arithmetic, same bits.
template <int NCOL, int FMT>
__global__ __launch_bounds__(256, NCOL <= 10 ? 3 : 2) void ln_rows_exact(const uint16_t* __restrict__ x, int64_t m, int64_t ld_x,
                                                                          const float* __restrict__ mul, const float* __restrict__ add,
                                                                          int64_t rows_per_group, float eps, uint8_t* __restrict__ q,
                                                                          int64_t ld_q, float* __restrict__ scale, float qmax) {
    constexpr int K = NCOL * 512;
    extern __shared__ __attribute__((aligned(16))) float s_vec[];  // mul, then add, in the lanes' read order (as above)
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int64_t stride = (int64_t)gridDim.x * 4;
    int64_t staged = -1;
    auto load_row = [&](int64_t r, uint4 (&dst)[NCOL]) __attribute__((always_inline)) {
        const uint4* xr = reinterpret_cast<const uint4*>(x + r * ld_x) + lane;
#pragma unroll
        for (int i = 0; i < NCOL; ++i) dst[i] = load_stream_16(xr + i * 64);
    };
    // one pass: stage the vectors of the quad's group if they changed, request the row of the next pass, work on `cur`
    auto pass = [&](int64_t row0, uint4 (&cur)[NCOL], uint4 (&nxt)[NCOL]) __attribute__((always_inline)) {
        const int64_t g0 = row0 / rows_per_group;
        if (g0 != staged) {
            __syncthreads();  // everyone is done with the previous group's vectors
            for (int e = threadIdx.x; e < K; e += 256) {
                const int c = e >> 3;
                const int pos = (((((c >> 6) << 1) + ((e >> 2) & 1)) * 64 + (c & 63)) << 2) | (e & 3);
                s_vec[pos] = mul ? mul[g0 * K + e] : 1.0f;
                s_vec[K + pos] = add ? add[g0 * K + e] : 0.0f;
            }
            staged = g0;
            __syncthreads();
        }
        const int64_t row = row0 + wave;
        // always requested, beyond the last row that row again: a load under a condition makes the registers of `nxt` a
        // merge of two values, which the compiler resolves with copies right behind the loads, i.e. by waiting for them
        load_row(row + stride < m ? row + stride : m - 1, nxt);
        if (row >= m) return;

        float sum = 0.0f, sq = 0.0f;  // see fused_rows_wave for the statistics
#pragma unroll
        for (int i = 0; i < NCOL; ++i) dot_sums(cur[i], sum, sq);
        dot_sums_done(sum, sq);
        float mean = wave_sum_f32(sum) / (float)K;
        float var = wave_sum_f32(sq) / (float)K - mean * mean;
        if (!(mean * mean <= 7.0f * var)) {
            float sd = 0.0f, ssq = 0.0f;
#pragma unroll
            for (int i = 0; i < NCOL; ++i) {
                float f[8];
                unpack8(cur[i], f);
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const float d = f[e] - mean;
                    sd += d;
                    ssq += d * d;
                }
            }
            const float dm = wave_sum_f32(sd) / (float)K;
            var = wave_sum_f32(ssq) / (float)K - dm * dm;
            mean += dm;
        }
        forget_values(cur);
        const float rstd = 1.0f / sqrtf(var + eps);  // IEEE sqrt and division
        const float nm = -mean;
#pragma unroll
        for (int i = 0; i < NCOL; ++i) {
            float f[8];
            dot_add8(cur[i], nm, f);  // x - mean
            const float* sv = s_vec + (i * 128 + lane) * 4;
            const float4 a0 = *reinterpret_cast<const float4*>(sv);
            const float4 a1 = *reinterpret_cast<const float4*>(sv + 256);
            const float4 b0 = *reinterpret_cast<const float4*>(sv + K);
            const float4 b1 = *reinterpret_cast<const float4*>(sv + K + 256);
            const float a[8] = {a0.x, a0.y, a0.z, a0.w, a1.x, a1.y, a1.z, a1.w};
            const float b[8] = {b0.x, b0.y, b0.z, b0.w, b1.x, b1.y, b1.z, b1.w};
#pragma unroll
            for (int e = 0; e < 8; ++e) f[e] = __builtin_fmaf(__fmul_rn(f[e], rstd), a[e], b[e]);
            cur[i] = pack8(f);
        }
        uint32_t mx = 0;
#pragma unroll
        for (int i = 0; i < NCOL; ++i) mx = chunk_absmax(mx, cur[i]);
        uint32_t amax = (mx & 0xffffu) > (mx >> 16) ? (mx & 0xffffu) : (mx >> 16);
        amax = wave_max_u32(amax);
        const float s = scale_from_amax_bits<true>(amax, qmax);
        if (lane == 0) scale[row] = s;
        const float inv = 1.0f / s;
        uint2* qr = reinterpret_cast<uint2*>(q + row * ld_q) + lane;
#pragma unroll
        for (int i = 0; i < NCOL; ++i) store_stream_8(qr + i * 64, quant_chunk<FMT, false, DAXQ_BF16, false>(cur[i], s, inv));
    };
    uint4 ra[NCOL], rb[NCOL];
    int64_t row0 = (int64_t)blockIdx.x * 4;
    load_row(row0 + wave < m ? row0 + wave : m - 1, ra);
    while (row0 < m) {
        pass(row0, ra, rb);
        row0 += stride;
        if (row0 >= m) break;
        pass(row0, rb, ra);
        row0 += stride;
    }
}

// The GELU form for rows of exactly NCOL x 512 elements, quantised bytes only: no lane predicates (the general kernel
// keeps one execution mask per chunk alive, 28 of them, which the compiler spills from scalar registers into vector lanes:
// some 300 v_writelane / v_readlane per row on a kernel that is bound by VALU issue) and a scalar row number.  Same
// arithmetic, same bits.  One row per wavefront, four per workgroup.
template <int NCOL, int FMT>
__global__ __launch_bounds__(256) void gelu_rows_exact(const uint16_t* __restrict__ x, int64_t m, int64_t ld_x, uint8_t* __restrict__ q,
                                                       int64_t ld_q, float* __restrict__ scale, float qmax) {
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int64_t row = (int64_t)blockIdx.x * 4 + wave;
    if (row >= m) return;
    uint4 v[NCOL];
    const uint4* xr = reinterpret_cast<const uint4*>(x + row * ld_x) + lane;
#pragma unroll
    for (int i = 0; i < NCOL; ++i) v[i] = load_stream_16(xr + i * 64);
#pragma unroll
    for (int i = 0; i < NCOL; ++i) {
        float f[8];
        unpack8(v[i], f);
#pragma unroll
        for (int e = 0; e < 8; ++e) f[e] = gelu_tanh_f32(f[e]);
        v[i] = pack8(f);
    }
    uint32_t mx = 0;
#pragma unroll
    for (int i = 0; i < NCOL; ++i) mx = chunk_absmax(mx, v[i]);
    uint32_t amax = (mx & 0xffffu) > (mx >> 16) ? (mx & 0xffffu) : (mx >> 16);
    amax = wave_max_u32(amax);
    const float s = scale_from_amax_bits<true>(amax, qmax);
    if (lane == 0) scale[row] = s;
    const float inv = 1.0f / s;
    uint2* qr = reinterpret_cast<uint2*>(q + row * ld_q) + lane;
#pragma unroll
    for (int i = 0; i < NCOL; ++i) store_stream_8(qr + i * 64, quant_chunk<FMT, false, DAXQ_BF16, false>(v[i], s, inv));
}

template <int NCOL, int FMT>
static int launch_ln_exact(const char* what, const uint16_t* x, int64_t m, int64_t ld_x, const float* mul, const float* add,
                           int64_t rows_per_group, float eps, uint8_t* q, int64_t ld_q, float* scale, float qmax, int cus,
                           hipStream_t st) {
    constexpr size_t lds = (size_t)NCOL * 512 * 8;
    static int per_cu = 0;  // asked once per instantiation; a race between two threads stores the same value twice
    if (per_cu <= 0) {
        int v = 0;
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&v, ln_rows_exact<NCOL, FMT>, 256, lds) != hipSuccess || v <= 0)
            return fail(DAXQ_ERR_LAUNCH, "%s: occupancy query failed", what);
        per_cu = v;
    }
    const int64_t quads = (m + 3) / 4, want = (int64_t)cus * per_cu;
    hipLaunchKernelGGL((ln_rows_exact<NCOL, FMT>), dim3((unsigned)(quads < want ? quads : want)), dim3(256), lds, st, x, m, ld_x, mul,
                       add, rows_per_group, eps, q, ld_q, scale, qmax);
    return check_launch(what);
}

template <int FMT, int PRE>
static int launch_fused_rows(const char* what, const void* x, int64_t m, int64_t k, int64_t ld_x, const float* mul,
                             const float* add, int64_t rows_per_group, float eps, void* y, int64_t ld_y, void* q,
                             int64_t ld_q, float* scale, float qmax, hipStream_t st) {
    if (m < 0 || k <= 0 || ld_x < k || ld_q < k || (y && ld_y < k))
        return fail(DAXQ_ERR_ARG, "%s: bad shape m=%lld k=%lld ld_x=%lld ld_q=%lld", what, (long long)m, (long long)k,
                    (long long)ld_x, (long long)ld_q);
    if (PRE == PRE_LN && (rows_per_group <= 0 || !(eps >= 0.0f))) return fail(DAXQ_ERR_ARG, "%s: rows_per_group and eps must be positive", what);
    if (m == 0) return DAXQ_OK;
    if (!x || !q || !scale) return fail(DAXQ_ERR_ARG, "%s: null pointer", what);
    const int64_t kfill = fill_width(k, ld_q);
    // the row has to fit the registers of one wavefront and move in 16-byte pieces
    const bool ok = (k % 8 == 0) && (ld_x % 8 == 0) && (ld_q % 8 == 0) && (!y || ld_y % 8 == 0) && (((uintptr_t)x & 15) == 0) &&
                    (((uintptr_t)y & 15) == 0) && (((uintptr_t)q & 7) == 0) && (((uintptr_t)scale & 3) == 0) &&
                    (((uintptr_t)mul & 3) == 0) && (((uintptr_t)add & 3) == 0) && (kfill / 8 <= 28 * 64) &&
                    (PRE != PRE_LN || k <= 8192);
    if (!ok)
        return fail(DAXQ_ERR_ALIGN, "%s: needs k %% 8 == 0, k <= 14336 (8192 with LayerNorm), 16-byte aligned rows of x / y and 8-byte aligned rows of q", what);
    const uint16_t* xp = static_cast<const uint16_t*>(x);
    uint16_t* yp = static_cast<uint16_t*>(y);
    uint8_t* qp = static_cast<uint8_t*>(q);
    const int nchunks = (int)((kfill / 8 + 63) / 64);
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
        return fail(DAXQ_ERR_LAUNCH, "%s: cannot read the CU count", what);
    if constexpr (PRE == PRE_LN) {
        // whole 512-element columns, groups of whole row quads, bytes only: the kernel without predicates
        if (!yp && k % 512 == 0 && kfill == k && rows_per_group % 4 == 0) {
            switch (k / 512) {
#define DAXQ_LN_EXACT(N) \
    case N: return launch_ln_exact<N, FMT>(what, xp, m, ld_x, mul, add, rows_per_group, eps, qp, ld_q, scale, qmax, cus, st);
                DAXQ_LN_EXACT(3)
                DAXQ_LN_EXACT(4)
                DAXQ_LN_EXACT(6)
                DAXQ_LN_EXACT(8)
                DAXQ_LN_EXACT(10)
                DAXQ_LN_EXACT(12)
                DAXQ_LN_EXACT(16)
#undef DAXQ_LN_EXACT
                default: break;
            }
        }
    }
    if constexpr (PRE == PRE_GELU) {
        if (!yp && k % 512 == 0 && kfill == k) {
            const dim3 grid((unsigned)((m + 3) / 4));
            switch (k / 512) {
#define DAXQ_GELU_EXACT(N)                                                                                                        \
    case N:                                                                                                                       \
        hipLaunchKernelGGL((gelu_rows_exact<N, FMT>), grid, dim3(256), 0, st, xp, m, ld_x, qp, ld_q, scale, qmax);                 \
        return check_launch(what);
                DAXQ_GELU_EXACT(12)
                DAXQ_GELU_EXACT(16)
                DAXQ_GELU_EXACT(24)
                DAXQ_GELU_EXACT(27)
#undef DAXQ_GELU_EXACT
                default: break;
            }
        }
    }
    // PRE_LN keeps its workgroups resident -- exactly as many as fit a CU (measured: 0.340 ms with the exact
    // number against 0.355 / 0.49 ms with twice / half as many) -- so that the staged vectors are reused over
    // many rows; the GELU form has nothing to reuse and takes one quad of rows per workgroup
    const int64_t quads = (m + 3) / 4;
    const size_t lds = PRE == PRE_LN ? (size_t)((k + 511) / 512) * 512 * 8 : 0;  // two vectors, padded to whole 64-chunk groups
    const dim3 block(256);
#define DAXQ_F_CASE(N)                                                                                                   \
    if (nchunks <= N) {                                                                                                  \
        int64_t want = quads;                                                                                            \
        if (PRE == PRE_LN) {                                                                                             \
            /* asked once per kernel and LDS size (k); a race between two threads stores the same value twice */         \
            static int cached_per_cu[2] = {0, 0};                                                                        \
            static int64_t cached_k[2] = {0, 0};                                                                         \
            const int slot = yp ? 1 : 0;                                                                                 \
            if (cached_per_cu[slot] <= 0 || cached_k[slot] != k) {                                                       \
                int per_cu = 0;                                                                                          \
                hipError_t oe = yp ? hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, fused_rows_wave<N, FMT, PRE, true>, 256, lds) \
                                   : hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, fused_rows_wave<N, FMT, PRE, false>, 256, lds); \
                if (oe != hipSuccess || per_cu <= 0) return fail(DAXQ_ERR_LAUNCH, "%s: occupancy query failed", what);   \
                cached_k[slot] = k;                                                                                      \
                cached_per_cu[slot] = per_cu;                                                                            \
            }                                                                                                            \
            want = (int64_t)cus * cached_per_cu[slot];                                                                   \
        }                                                                                                                \
        const dim3 grid((unsigned)(quads < want ? quads : want));                                                        \
        if (yp)                                                                                                          \
            hipLaunchKernelGGL((fused_rows_wave<N, FMT, PRE, true>), grid, block, lds, st, xp, m, (int)k, ld_x, mul, add, \
                               rows_per_group, eps, yp, ld_y, qp, ld_q, (int)kfill, scale, qmax);                                    \
        else                                                                                                             \
            hipLaunchKernelGGL((fused_rows_wave<N, FMT, PRE, false>), grid, block, lds, st, xp, m, (int)k, ld_x, mul, add, \
                               rows_per_group, eps, yp, ld_y, qp, ld_q, (int)kfill, scale, qmax);                                    \
        return check_launch(what);                                                                                       \
    }
    DAXQ_F_CASE(4)
    DAXQ_F_CASE(12)
    DAXQ_F_CASE(20)
    DAXQ_F_CASE(28)
#undef DAXQ_F_CASE
    return fail(DAXQ_ERR_ARG, "%s: row too long", what);
}

}  // namespace daxq

extern "C" {

#define DAXQ_LN_ENTRY(NAME, FMT, QT, QMAX)                                                                                \
    int NAME(const void* x, int64_t m, int64_t k, int64_t ld_x, const float* mul, const float* add, int64_t rows_per_group, \
             float eps, void* y, int64_t ld_y, QT* q, int64_t ld_q, float* scale, daxq_stream_t stream) {                  \
        return daxq::launch_fused_rows<FMT, daxq::PRE_LN>(#NAME, x, m, k, ld_x, mul, add, rows_per_group, eps, y, ld_y, q,  \
                                                          ld_q, scale, QMAX, (hipStream_t)stream);                         \
    }
DAXQ_LN_ENTRY(daxq_layernorm_act_quant_i8, 0, int8_t, 127.0f)
DAXQ_LN_ENTRY(daxq_layernorm_act_quant_e4m3, 1, uint8_t, 448.0f)
DAXQ_LN_ENTRY(daxq_layernorm_act_quant_e5m2, 2, uint8_t, 57344.0f)
#undef DAXQ_LN_ENTRY

#define DAXQ_GELU_ENTRY(NAME, FMT, QT, QMAX)                                                                           \
    int NAME(const void* x, int64_t m, int64_t k, int64_t ld_x, void* y, int64_t ld_y, QT* q, int64_t ld_q, float* scale, \
             daxq_stream_t stream) {                                                                                   \
        return daxq::launch_fused_rows<FMT, daxq::PRE_GELU>(#NAME, x, m, k, ld_x, nullptr, nullptr, 1, 0.0f, y, ld_y, q,  \
                                                            ld_q, scale, QMAX, (hipStream_t)stream);                    \
    }
DAXQ_GELU_ENTRY(daxq_gelu_tanh_act_quant_i8, 0, int8_t, 127.0f)
DAXQ_GELU_ENTRY(daxq_gelu_tanh_act_quant_e4m3, 1, uint8_t, 448.0f)
DAXQ_GELU_ENTRY(daxq_gelu_tanh_act_quant_e5m2, 2, uint8_t, 57344.0f)
#undef DAXQ_GELU_ENTRY

}  // extern "C"
