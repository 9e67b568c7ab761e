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
    // addresses are clamped so that every load below is unconditional (all in flight together); what a lane must not
    // use is replaced by zero afterwards
    const int colc = min(col, P - 1);
    float* sp = state + (((long)(slot < 0 ? 0 : slot) * H + h) * N) * P + colc;
    float S[NPL];
#pragma unroll
    for (int j = 0; j < NPL; ++j) {
        const int e = part * NPL + j;
        const float x = sp[(long)min(e, N - 1) * P];
        S[j] = (!fresh && live && e < N) ? x : 0.f;
    }
    const float* kp = k + (long)g * N;
    const float* qp = q + (long)g * N;
    const float sk = skip ? skip[h] : 0.f;
    for (int i = threadIdx.x; i < 2 * NP; i += blockDim.x) {
        const int w = i / NP, e = i % NP;
        const float x = w ? qp[(long)row0 * ldq + min(e, N - 1)] : kp[(long)row0 * ldk + min(e, N - 1)];
        kq[0][w][e] = e < N ? x : 0.f;
    }
    const float* vp = v + (long)h * P + colc;
    const float* ap = decay + h;
    const float* cp = coef + h;
    // the next token's decay, write strength and value are requested one step ahead of their use
    float a_n = ap[(long)row0 * H], c_n = cp[(long)row0 * H], v_n = vp[(long)row0 * ldv];
    for (int t = 0; t < n; ++t) {
        const int row = row0 + t, b = t & 1;
        const float a = a_n, c = c_n, vv = live ? v_n : 0.f;
        __syncthreads();
        if (t + 1 < n) {
            for (int i = threadIdx.x; i < 2 * NP; i += blockDim.x) {
                const int w = i / NP, e = i % NP;
                const float x = w ? qp[(long)(row + 1) * ldq + min(e, N - 1)] : kp[(long)(row + 1) * ldk + min(e, N - 1)];
                kq[b ^ 1][w][e] = e < N ? x : 0.f;
            }
            a_n = ap[(long)(row + 1) * H];
            c_n = cp[(long)(row + 1) * H];
            v_n = vp[(long)(row + 1) * ldv];
        }
        const float* kb = &kq[b][0][part * NPL];
        const float* qb = &kq[b][1][part * NPL];
        float u;
        if constexpr (DELTA) {
            float d0 = 0.f, d1 = 0.f, d2 = 0.f, d3 = 0.f;  // four chains instead of one of NPL dependent adds
#pragma unroll
            for (int j = 0; j < NPL; j += 4) {
                S[j] *= a;
                S[j + 1] *= a;
                S[j + 2] *= a;
                S[j + 3] *= a;
                d0 += S[j] * kb[j];
                d1 += S[j + 1] * kb[j + 1];
                d2 += S[j + 2] * kb[j + 2];
                d3 += S[j + 3] * kb[j + 3];
            }
            const float d = group_sum<LPC>((d0 + d1) + (d2 + d3));
            u = c * (vv - d);
        } else {
#pragma unroll
            for (int j = 0; j < NPL; ++j) S[j] *= a;
            u = c * vv;
        }
        float o0 = 0.f, o1 = 0.f, o2 = 0.f, o3 = 0.f;
#pragma unroll
        for (int j = 0; j < NPL; j += 4) {
            S[j] += kb[j] * u;
            S[j + 1] += kb[j + 1] * u;
            S[j + 2] += kb[j + 2] * u;
            S[j + 3] += kb[j + 3] * u;
            o0 += S[j] * qb[j];
            o1 += S[j + 1] * qb[j + 1];
            o2 += S[j + 2] * qb[j + 2];
            o3 += S[j + 3] * qb[j + 3];
        }
        const float o = group_sum<LPC>((o0 + o1) + (o2 + o3));
        if (live && part == 0) out[(long)row * ldo + (long)h * P + col] = o + sk * vv;
    }
    if (slot >= 0 && live) {
#pragma unroll
        for (int j = 0; j < NPL; ++j)
            if (part * NPL + j < N) sp[(long)(part * NPL + j) * P] = S[j];
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
