// hybrid_scan.hip: the linear recurrence of gated-delta-rule and state-space (duality form) layers (ops/hybrid.py
// state_scan). Per sequence and head, over the step's rows in order:
//     S <- a_t S;   u = c_t (v_t - S^T k_t)  [delta]   or   u = c_t v_t;   S <- S + k_t u^T;   o_t = S^T q_t (+ D v_t)
// S is [N, P] fp32. Its P columns never mix, so a column belongs to LPC neighbouring lanes that each keep NPL of its
// N numbers in registers for the whole chunk; the two dot products of a step are finished with LPC-wide shuffles. k_t
// and q_t are the same for every column of a head: the block stages them in LDS (double buffered, one barrier per
// token). The state is read from the sequence's slot unless the chunk starts at position 0, and written back after
// the chunk's last row: a decode row is a chunk of one, a prompt chunk walks its rows inside one launch.
#include "../mx_common.h"

namespace {

// grid (column blocks, H, sequences); block = cols * LPC threads (a multiple of 64)
template <int NPL, int LPC, bool DELTA>
__global__ __launch_bounds__(256) void state_scan_kernel(const float* k, int ldk, const float* q, int ldq,
                                                         const float* v, int ldv, const float* decay, const float* coef,
                                                         const float* skip, float* state, const int* seq_state,
                                                         const int* positions, int n_dec, const int* pf_cu, float* out,
                                                         int ldo, int H, int G, int N, int P) {
    constexpr int NP = NPL * LPC;  // padded N
    __shared__ float kq[2][2][NP];
    const int cols = blockDim.x / LPC;
    const int col = blockIdx.x * cols + threadIdx.x / LPC;
    const int part = threadIdx.x % LPC;
    const int h = blockIdx.y, s = blockIdx.z;
    int row0, n;
    if (s < n_dec) {
        row0 = s;
        n = 1;
    } else {
        const int i = s - n_dec;
        row0 = n_dec + pf_cu[i];
        n = pf_cu[i + 1] - pf_cu[i];
    }
    if (n <= 0) return;
    const int slot = seq_state[s];
    const bool fresh = positions[row0] == 0 || slot < 0;
    const bool live = col < P;
    const int g = h / (H / G);
    float* sp = state + (((long)(slot < 0 ? 0 : slot) * H + h) * N + part * NPL) * P + col;
    float S[NPL];
#pragma unroll
    for (int j = 0; j < NPL; ++j) S[j] = (!fresh && live && part * NPL + j < N) ? sp[(long)j * P] : 0.f;
    const float* kp = k + (long)g * N;
    const float* qp = q + (long)g * N;
    const float sk = skip ? skip[h] : 0.f;
    for (int i = threadIdx.x; i < 2 * NP; i += blockDim.x) {
        const int w = i / NP, e = i % NP;
        kq[0][w][e] = e < N ? (w ? qp[(long)row0 * ldq + e] : kp[(long)row0 * ldk + e]) : 0.f;
    }
    for (int t = 0; t < n; ++t) {
        const int row = row0 + t, b = t & 1;
        __syncthreads();
        if (t + 1 < n) {
            for (int i = threadIdx.x; i < 2 * NP; i += blockDim.x) {
                const int w = i / NP, e = i % NP;
                kq[b ^ 1][w][e] = e < N ? (w ? qp[(long)(row + 1) * ldq + e] : kp[(long)(row + 1) * ldk + e]) : 0.f;
            }
        }
        const float a = decay[(long)row * H + h], c = coef[(long)row * H + h];
        const float vv = live ? v[(long)row * ldv + (long)h * P + col] : 0.f;
        const float* kb = &kq[b][0][part * NPL];
        const float* qb = &kq[b][1][part * NPL];
        float u;
        if constexpr (DELTA) {
            float d = 0.f;
#pragma unroll
            for (int j = 0; j < NPL; ++j) {
                S[j] *= a;
                d += S[j] * kb[j];
            }
            d = group_sum<LPC>(d);
            u = c * (vv - d);
        } else {
#pragma unroll
            for (int j = 0; j < NPL; ++j) S[j] *= a;
            u = c * vv;
        }
        float o = 0.f;
#pragma unroll
        for (int j = 0; j < NPL; ++j) {
            S[j] += kb[j] * u;
            o += S[j] * qb[j];
        }
        o = group_sum<LPC>(o);
        if (live && part == 0) out[(long)row * ldo + (long)h * P + col] = o + sk * vv;
    }
    if (slot >= 0 && live) {
#pragma unroll
        for (int j = 0; j < NPL; ++j)
            if (part * NPL + j < N) sp[(long)j * P] = S[j];
    }
}

}  // namespace

#define MXH_CHECK(cond) \
    if (!(cond)) return (int)hipErrorInvalidValue

extern "C" int mxh_state_scan(const float* k, int ldk, const float* q, int ldq, const float* v, int ldv,
                              const float* decay, const float* coef, const float* skip, float* state,
                              const int* seq_state, const int* positions, int n_dec, const int* pf_cu, int n_pf,
                              float* out, int ldo, int H, int G, int N, int P, int delta, hipStream_t st) {
    const int n_seqs = n_dec + n_pf;
    if (n_seqs <= 0) return 0;
    MXH_CHECK(k && q && v && decay && coef && state && seq_state && positions && out && (n_pf == 0 || pf_cu));
    MXH_CHECK(H > 0 && G > 0 && H % G == 0 && N > 0 && N <= 256 && P > 0 && H <= 65535 && n_seqs <= 65535);
    MXH_CHECK(ldk >= G * N && ldq >= G * N && ldv >= H * P && ldo >= H * P);
    const int lpc = N <= 64 ? 1 : N <= 128 ? 2 : 4;
    int threads = min(256, ((P * lpc + 63) / 64) * 64);
    const int cols = threads / lpc;
    const dim3 grid((P + cols - 1) / cols, H, n_seqs);
#define GO(NPL, LPC)                                                                                                 \
    do {                                                                                                             \
        if (delta)                                                                                                   \
            state_scan_kernel<NPL, LPC, true><<<grid, threads, 0, st>>>(k, ldk, q, ldq, v, ldv, decay, coef, skip,   \
                                                                        state, seq_state, positions, n_dec, pf_cu,  \
                                                                        out, ldo, H, G, N, P);                       \
        else                                                                                                         \
            state_scan_kernel<NPL, LPC, false><<<grid, threads, 0, st>>>(k, ldk, q, ldq, v, ldv, decay, coef, skip,  \
                                                                         state, seq_state, positions, n_dec, pf_cu, \
                                                                         out, ldo, H, G, N, P);                      \
    } while (0)
    if (N <= 16) GO(16, 1);
    else if (N <= 32) GO(32, 1);
    else if (N <= 64) GO(64, 1);
    else if (N <= 128) GO(64, 2);
    else GO(64, 4);
#undef GO
    return (int)hipGetLastError();
}
