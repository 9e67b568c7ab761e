// latent_ops.hip: the small fp32 row kernels of decoders built on ops/latent.py (scalar-gain RMS norm, embedding
// gather + norm, sigmoid-gated normed residual add, squared ReLU, causal tap convolution with carried tails, the
// two latent norms + paged append, per-head output gate + head-major -> token-major pack).
//
// All statistics, gates and the residual are fp32; 16-bit (bf16) appears only on outputs that feed a GEMM and in
// the cached latent. Launchers are `extern "C" int mxl_*(..., hipStream_t)`, return the launch's hipError_t, never
// allocate or synchronise (safe under stream capture) and check the shapes their grids assume.
#include "../mx_common.h"

namespace {

constexpr int NT = 256;

MX_DEV float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}

// sum over the NT threads of a block, returned to every thread
MX_DEV float block_sum(float v, float* red) {
    v = wave_sum(v);
    const int w = threadIdx.x >> 6;
    __syncthreads();
    if ((threadIdx.x & 63) == 0) red[w] = v;
    __syncthreads();
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < NT / 64; ++i) s += red[i];
    return s;
}

MX_DEV float sigmoidf_(float v) { return 1.f / (1.f + __expf(-v)); }

template <bool B16>
MX_DEV float ld_elem(const void* p, long i) {
    if constexpr (B16) return bf16_to_f32(((const bf16_t*)p)[i]);
    else return ((const float*)p)[i];
}
template <bool B16>
MX_DEV void st_elem(void* p, long i, float v) {
    if constexpr (B16) ((bf16_t*)p)[i] = f32_to_bf16(v);
    else ((float*)p)[i] = v;
}

constexpr int RC = 16;  // rows of up to NT * RC numbers are read once and kept in registers

template <bool B16>
__global__ __launch_bounds__(NT) void embed_norm_kernel(const void* table, int V, const int* tokens, const float* g,
                                                        float eps, float* out, int ldo, int C) {
    __shared__ float red[NT / 64];
    const int t = blockIdx.x;
    int tok = tokens[t];
    if (tok < 0 || tok >= V) tok = 0;
    const long base = (long)tok * C;
    const bool cached = C <= NT * RC;
    float keep[RC];
    float ss = 0.f;
    if (cached) {
#pragma unroll
        for (int k = 0; k < RC; ++k) {  // clamped addresses: straight-line loads, all in flight together
            const int c = threadIdx.x + k * NT;
            const float v = ld_elem<B16>(table, base + min(c, C - 1));
            keep[k] = c < C ? v : 0.f;
            ss += keep[k] * keep[k];
        }
    } else {
        for (int c = threadIdx.x; c < C; c += NT) {
            const float v = ld_elem<B16>(table, base + c);
            ss += v * v;
        }
    }
    ss = block_sum(ss, red);
    const float sc = g[0] / sqrtf(ss / (float)C + eps);
    if (cached) {
#pragma unroll
        for (int k = 0; k < RC; ++k) {
            const int c = threadIdx.x + k * NT;
            if (c < C) out[(long)t * ldo + c] = keep[k] * sc;
        }
        return;
    }
    for (int c = threadIdx.x; c < C; c += NT) out[(long)t * ldo + c] = ld_elem<B16>(table, base + c) * sc;
}

__global__ __launch_bounds__(NT) void scalar_norm_kernel(const float* x, int ldx, const int* rows, const float* g,
                                                         float eps, float* o32, int ld32, bf16_t* o16, int ld16,
                                                         int C) {
    __shared__ float red[NT / 64];
    const int i = blockIdx.x;
    const float* xr = x + (long)(rows ? rows[i] : i) * ldx;
    const bool cached = C <= NT * RC;
    float keep[RC];
    float ss = 0.f;
    if (cached) {
#pragma unroll
        for (int k = 0; k < RC; ++k) {  // clamped addresses: straight-line loads, all in flight together
            const int c = threadIdx.x + k * NT;
            const float v = xr[min(c, C - 1)];
            keep[k] = c < C ? v : 0.f;
            ss += keep[k] * keep[k];
        }
    } else {
        for (int c = threadIdx.x; c < C; c += NT) {
            const float v = xr[c];
            ss += v * v;
        }
    }
    ss = block_sum(ss, red);
    const float sc = g[0] / sqrtf(ss / (float)C + eps);
    if (cached) {
#pragma unroll
        for (int k = 0; k < RC; ++k) {
            const int c = threadIdx.x + k * NT;
            if (c < C) {
                const float v = keep[k] * sc;
                if (o32) o32[(long)i * ld32 + c] = v;
                if (o16) o16[(long)i * ld16 + c] = f32_to_bf16(v);
            }
        }
        return;
    }
    for (int c = threadIdx.x; c < C; c += NT) {
        const float v = xr[c] * sc;
        if (o32) o32[(long)i * ld32 + c] = v;
        if (o16) o16[(long)i * ld16 + c] = f32_to_bf16(v);
    }
}

// x += g * unit_rms(z), z = y * sigmoid(gate_pre + gate_bias); then, when gn is given, the NEXT norm of the updated
// row in the same pass: n = gn * unit_rms(x) written as fp32 and / or bf16 (the row is still in registers)
__global__ __launch_bounds__(NT) void gated_norm_add_kernel(float* x, int ldx, const float* y, int ldy,
                                                            const float* gp, int ldg, const float* gb, const float* g,
                                                            float eps, int C, const float* gn, float* n32, int ldn32,
                                                            bf16_t* n16, int ldn16) {
    __shared__ float red[NT / 64];
    __shared__ float red2[NT / 64];
    const int i = blockIdx.x;
    const float* yr = y + (long)i * ldy;
    const float* gr = gp + (long)i * ldg;
    const bool cached = C <= NT * RC;
    float keep[RC], xin[RC];
    float ss = 0.f;
    if (cached) {
        // every load of the row (the residual too) is issued before the statistics: one memory round trip
        float yv[RC], gv[RC];
#pragma unroll
        for (int k = 0; k < RC; ++k) {  // clamped addresses: straight-line loads, all in flight together
            const int c = min(threadIdx.x + k * NT, C - 1);
            xin[k] = x[(long)i * ldx + c];
            yv[k] = yr[c];
            gv[k] = gr[c] + (gb ? gb[c] : 0.f);
        }
#pragma unroll
        for (int k = 0; k < RC; ++k) {
            const int c = threadIdx.x + k * NT;
            keep[k] = c < C ? yv[k] * sigmoidf_(gv[k]) : 0.f;
            ss += keep[k] * keep[k];
        }
    } else {
        for (int c = threadIdx.x; c < C; c += NT) {
            const float z = yr[c] * sigmoidf_(gr[c] + (gb ? gb[c] : 0.f));
            ss += z * z;
        }
    }
    ss = block_sum(ss, red);
    const float sc = g[0] / sqrtf(ss / (float)C + eps);
    float s2 = 0.f;
    if (cached) {
#pragma unroll
        for (int k = 0; k < RC; ++k) {
            const int c = threadIdx.x + k * NT;
            xin[k] = c < C ? xin[k] + keep[k] * sc : 0.f;
            if (c < C) x[(long)i * ldx + c] = xin[k];
            s2 += xin[k] * xin[k];
        }
    } else {
        for (int c = threadIdx.x; c < C; c += NT) {
            const float v = x[(long)i * ldx + c] + yr[c] * sigmoidf_(gr[c] + (gb ? gb[c] : 0.f)) * sc;
            x[(long)i * ldx + c] = v;
            s2 += v * v;
        }
    }
    if (gn == nullptr) return;
    s2 = block_sum(s2, red2);
    const float sn = gn[0] / sqrtf(s2 / (float)C + eps);
    if (cached) {
#pragma unroll
        for (int k = 0; k < RC; ++k) {
            const int c = threadIdx.x + k * NT;
            if (c < C) {
                const float v = xin[k] * sn;
                if (n32) n32[(long)i * ldn32 + c] = v;
                if (n16) n16[(long)i * ldn16 + c] = f32_to_bf16(v);
            }
        }
        return;
    }
    for (int c = threadIdx.x; c < C; c += NT) {  // the thread re-reads what it wrote itself
        const float v = x[(long)i * ldx + c] * sn;
        if (n32) n32[(long)i * ldn32 + c] = v;
        if (n16) n16[(long)i * ldn16 + c] = f32_to_bf16(v);
    }
}

template <bool B16>
__global__ __launch_bounds__(NT) void relu2_kernel(const float* u, int ldu, void* out, int ldo, int F) {
    const int i = blockIdx.y;
    for (int c = blockIdx.x * NT + threadIdx.x; c < F; c += gridDim.x * NT) {
        const float v = fmaxf(u[(long)i * ldu + c], 0.f);
        st_elem<B16>(out, (long)i * ldo + c, v * v);
    }
}

constexpr int CONV_ROWS = 64;  // rows of one sequence per block; >= taps - 1, so only row tile 0 reads the old tail

// grid (channel tiles, sequences, row tiles). A thread owns one channel. Only the block of row tile 0 reads the
// sequence's old tail, and after its outputs it writes the new one (ascending, in place: entry i is written after
// entry i + n was read), so no other block races with the update.
template <bool B16>
__global__ __launch_bounds__(NT) void tap_conv_kernel(const float* h, int ldh, const float* w, int taps, float* tails,
                                                      const int* state, const int* positions, int n_dec,
                                                      const int* pf_cu, void* out, int ldo, int C) {
    const int c = blockIdx.x * NT + threadIdx.x;
    const int s = blockIdx.y;
    int row0, n;
    if (s < n_dec) {
        row0 = s;
        n = 1;
    } else {
        const int k = s - n_dec;
        row0 = n_dec + pf_cu[k];
        n = pf_cu[k + 1] - pf_cu[k];
    }
    const int t0 = blockIdx.z * CONV_ROWS;
    if (t0 >= n || c >= C) return;
    const int slot = state[s];
    const int nt = taps - 1;
    const bool fresh = positions[row0] == 0 || slot < 0;
    float* tail = tails + ((long)(slot < 0 ? 0 : slot) * (nt > 0 ? nt : 1)) * C + c;  // entry i at tail[i * C]
    float wr[16];
#pragma unroll
    for (int j = 0; j < 16; ++j) wr[j] = j < taps ? w[(long)c * taps + j] : 0.f;
    const int t1 = min(n, t0 + CONV_ROWS);
    for (int t = t0; t < t1; ++t) {
        const float cur = h[(long)(row0 + t) * ldh + c];
        float acc = cur;
#pragma unroll
        for (int j = 0; j < 16; ++j) {
            if (j < taps) {
                const int tau = t - nt + j;  // input index within the chunk; < 0: carried from earlier steps
                float v;
                if (tau >= 0) v = h[(long)(row0 + tau) * ldh + c];
                else v = fresh ? 0.f : tail[(long)(nt + tau) * C];
                acc += wr[j] * v;
            }
        }
        st_elem<B16>(out, (long)(row0 + t) * ldo + c, acc);
    }
    if (t0 == 0 && slot >= 0) {
        for (int i = 0; i < nt; ++i) {
            const int tau = n - nt + i;
            float v;
            if (tau >= 0) v = h[(long)(row0 + tau) * ldh + c];
            else v = fresh ? 0.f : tail[(long)(nt + tau) * C];
            tail[(long)i * C] = v;
        }
    }
}

// grid (T, 2): y = 0 the query latent (-> cq), y = 1 the key/value latent (-> paged pool at the row's slot)
template <bool Q16, bool C16>
__global__ __launch_bounds__(NT) void latent_norm_append_kernel(const float* y, int ldy, int q_rank, int rank,
                                                                const float* wq, const float* wkv, float eps, void* cq,
                                                                int ldcq, void* cache, const int* slots) {
    __shared__ float red[NT / 64];
    const int t = blockIdx.x;
    const bool kv = blockIdx.y == 1;
    const int n = kv ? rank : q_rank;
    const float* yr = y + (long)t * ldy + (kv ? q_rank : 0);
    long dst = 0;
    if (kv) {
        const int sl = slots[t];
        if (sl < 0) return;
        dst = (long)sl * rank;
    }
    float ss = 0.f;
    for (int c = threadIdx.x; c < n; c += NT) {
        const float v = yr[c];
        ss += v * v;
    }
    ss = block_sum(ss, red);
    const float sc = 1.f / sqrtf(ss / (float)n + eps);
    const float* wv = kv ? wkv : wq;
    for (int c = threadIdx.x; c < n; c += NT) {
        const float v = yr[c] * sc * wv[c];
        if (kv) st_elem<C16>(cache, dst + c, v);
        else st_elem<Q16>(cq, (long)t * ldcq + c, v);
    }
}

template <bool B16>
__global__ __launch_bounds__(NT) void head_gate_pack_kernel(const float* ov, const float* gp, int ldg, void* out,
                                                            int ldo, int H, int T, int dv) {
    const int t = blockIdx.x;
    const int n = H * dv;
    for (int i = threadIdx.x; i < n; i += NT) {
        const int hh = i / dv, e = i - hh * dv;
        const float v = ov[((long)hh * T + t) * dv + e] * sigmoidf_(gp[(long)t * ldg + hh]);
        st_elem<B16>(out, (long)t * ldo + i, v);
    }
}

}  // namespace

#define MXL_CHECK(cond) \
    if (!(cond)) return (int)hipErrorInvalidValue

extern "C" int mxl_embed_norm(const void* table, int is16, int V, const int* tokens, const float* g, float eps,
                              float* out, int ldo, int T, int C, hipStream_t st) {
    if (T <= 0) return 0;
    MXL_CHECK(table && tokens && g && out && C > 0 && V > 0 && ldo >= C);
    if (is16) embed_norm_kernel<true><<<T, NT, 0, st>>>(table, V, tokens, g, eps, out, ldo, C);
    else embed_norm_kernel<false><<<T, NT, 0, st>>>(table, V, tokens, g, eps, out, ldo, C);
    return (int)hipGetLastError();
}

extern "C" int mxl_scalar_norm(const float* x, int ldx, const int* rows, const float* g, float eps, float* o32,
                               int ld32, bf16_t* o16, int ld16, int M, int C, hipStream_t st) {
    if (M <= 0) return 0;
    MXL_CHECK(x && g && C > 0 && ldx >= C && (o32 || o16) && (!o32 || ld32 >= C) && (!o16 || ld16 >= C));
    scalar_norm_kernel<<<M, NT, 0, st>>>(x, ldx, rows, g, eps, o32, ld32, o16, ld16, C);
    return (int)hipGetLastError();
}

extern "C" int mxl_gated_norm_add(float* x, int ldx, const float* y, int ldy, const float* gp, int ldg, const float* gb,
                                  const float* g, float eps, int M, int C, const float* gn, float* n32, int ldn32,
                                  bf16_t* n16, int ldn16, hipStream_t st) {
    if (M <= 0) return 0;
    MXL_CHECK(x && y && gp && g && C > 0 && ldx >= C && ldy >= C && ldg >= C);
    MXL_CHECK(!gn || ((n32 || n16) && (!n32 || ldn32 >= C) && (!n16 || ldn16 >= C)));
    gated_norm_add_kernel<<<M, NT, 0, st>>>(x, ldx, y, ldy, gp, ldg, gb, g, eps, C, gn, n32, ldn32, n16, ldn16);
    return (int)hipGetLastError();
}

extern "C" int mxl_relu2(const float* u, int ldu, void* out, int ldo, int is16, int M, int F, hipStream_t st) {
    if (M <= 0 || F <= 0) return 0;
    MXL_CHECK(u && out && ldu >= F && ldo >= F && M <= 65535);  // rows ride on grid.y
    dim3 grid(min((F + NT - 1) / NT, 64), M);
    if (is16) relu2_kernel<true><<<grid, NT, 0, st>>>(u, ldu, out, ldo, F);
    else relu2_kernel<false><<<grid, NT, 0, st>>>(u, ldu, out, ldo, F);
    return (int)hipGetLastError();
}

extern "C" int mxl_tap_conv(const float* h, int ldh, const float* w, int taps, float* tails, const int* state,
                            const int* positions, int n_dec, const int* pf_cu, int n_pf, void* out, int ldo, int is16,
                            int T, int C, hipStream_t st) {
    const int S = n_dec + n_pf;
    if (S <= 0 || T <= 0) return 0;
    MXL_CHECK(h && w && tails && state && positions && out && taps >= 1 && taps <= 16 && C > 0 && ldh >= C &&
              ldo >= C && (n_pf == 0 || pf_cu) && n_dec <= T && S <= 65535);
    const int longest = n_pf ? T - n_dec : 1;
    dim3 grid((C + NT - 1) / NT, S, (max(longest, 1) + CONV_ROWS - 1) / CONV_ROWS);
    MXL_CHECK(grid.z <= 65535);
    if (is16) tap_conv_kernel<true><<<grid, NT, 0, st>>>(h, ldh, w, taps, tails, state, positions, n_dec, pf_cu, out, ldo, C);
    else tap_conv_kernel<false><<<grid, NT, 0, st>>>(h, ldh, w, taps, tails, state, positions, n_dec, pf_cu, out, ldo, C);
    return (int)hipGetLastError();
}

extern "C" int mxl_latent_norm_append(const float* y, int ldy, int q_rank, int rank, const float* wq, const float* wkv,
                                      float eps, void* cq, int ldcq, int cq16, void* cache, int cache16,
                                      const int* slots, int T, hipStream_t st) {
    if (T <= 0) return 0;
    MXL_CHECK(y && wq && wkv && cq && cache && slots && q_rank > 0 && rank > 0 && ldy >= q_rank + rank &&
              ldcq >= q_rank);
    dim3 grid(T, 2);
    if (cq16 && cache16)
        latent_norm_append_kernel<true, true><<<grid, NT, 0, st>>>(y, ldy, q_rank, rank, wq, wkv, eps, cq, ldcq, cache, slots);
    else if (!cq16 && !cache16)
        latent_norm_append_kernel<false, false><<<grid, NT, 0, st>>>(y, ldy, q_rank, rank, wq, wkv, eps, cq, ldcq, cache, slots);
    else if (cq16)
        latent_norm_append_kernel<true, false><<<grid, NT, 0, st>>>(y, ldy, q_rank, rank, wq, wkv, eps, cq, ldcq, cache, slots);
    else
        latent_norm_append_kernel<false, true><<<grid, NT, 0, st>>>(y, ldy, q_rank, rank, wq, wkv, eps, cq, ldcq, cache, slots);
    return (int)hipGetLastError();
}

extern "C" int mxl_head_gate_pack(const float* ov, const float* gp, int ldg, void* out, int ldo, int is16, int H, int T,
                                  int dv, hipStream_t st) {
    if (T <= 0) return 0;
    MXL_CHECK(ov && gp && out && H > 0 && dv > 0 && ldg >= H && ldo >= H * dv);
    if (is16) head_gate_pack_kernel<true><<<T, NT, 0, st>>>(ov, gp, ldg, out, ldo, H, T, dv);
    else head_gate_pack_kernel<false><<<T, NT, 0, st>>>(ov, gp, ldg, out, ldo, H, T, dv);
    return (int)hipGetLastError();
}
