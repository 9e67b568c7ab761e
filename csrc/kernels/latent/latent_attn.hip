// latent_attn.hip: causal softmax attention over a paged pool of per-token latents, in the weight-absorbed form:
// the rows are absorbed queries qa (one per token and head, `R` numbers), and a cached latent c_j serves as key AND
// value for every head:   out[row] = sum_j softmax_j(qa[row] . c_j) c_j   over the keys j <= the row's position.
//
// One kernel serves decode rows (one token per sequence, optionally split over key partitions that a second kernel
// merges) and prompt chunks (several tokens per sequence, causal inside the chunk). A workgroup owns BM consecutive
// (token, head) rows of one sequence (all heads of a token read the same latents, so the key tile in LDS is
// shared by BM rows) and streams the visible keys in tiles of BN through LDS with an online softmax. Scores,
// softmax and the accumulators are fp32 whatever the storage type (bf16 or fp32) of queries, cache and output.
//
// Thread layout: 8 lanes per row (lane l8 of row m is thread m * 8 + l8, so a row's lanes sit in one wave).
//   scores: lane l8 takes keys l8, l8 + 8, ... of the tile (BN / 8 dot products over R from LDS);
//   output: lane l8 accumulates columns 4 l8 + 32 i .. + 3 (i < RV, R <= 32 RV) for its row.
#include "../mx_common.h"

namespace {

template <bool B16>
MX_DEV float ldf(const void* p, long i) {
    if constexpr (B16) return bf16_to_f32(((const bf16_t*)p)[i]);
    else return ((const float*)p)[i];
}
template <bool B16>
MX_DEV void stf(void* p, long i, float v) {
    if constexpr (B16) ((bf16_t*)p)[i] = f32_to_bf16(v);
    else ((float*)p)[i] = v;
}

struct AttnArgs {
    const void* qa;
    long qs_t, qs_h;
    const void* cache;
    int bs, R;
    const int* bt;
    int bt_stride;
    const int* cu_q;  // null: one row per sequence (decode)
    const int* ctx;
    int n_seqs, row_base;
    void* out;
    long os_t, os_h;
    float scale;
    int H, parts, part_len;
    float* part_ml;
    float* part_o;
};

template <bool B16, int RV, int BN, int BM>
__global__ __launch_bounds__(BM * 8) void latent_attn_kernel(AttnArgs a) {
    constexpr int NTH = BM * 8, RW = RV * 32, RP = RW + 4, NJ = BN / 8;
    extern __shared__ __align__(16) float lds[];
    float* QA = lds;                 // [BM][RP], pre-multiplied by the softmax scale
    float* CT = QA + BM * RP;        // [BN][RP]
    float* PS = CT + BN * RP;        // [BM][BN + 1]
    const int tid = threadIdx.x, m = tid >> 3, l8 = tid & 7;
    const int H = a.H, R = a.R;

    // ---- which sequence and which of its (token, head) rows ----
    int seq = -1, g0 = 0, qlen = 1, crow0 = 0;
    {
        int tile = blockIdx.x;
        if (a.cu_q == nullptr) {
            const int tps = (H + BM - 1) / BM;
            seq = tile / tps;
            g0 = (tile - seq * tps) * BM;
            crow0 = seq;
            if (seq >= a.n_seqs) return;
        } else {
            for (int s = 0; s < a.n_seqs; ++s) {
                const int q = a.cu_q[s + 1] - a.cu_q[s];
                const int nt = (q * H + BM - 1) / BM;
                if (tile < nt) {
                    seq = s;
                    g0 = tile * BM;
                    qlen = q;
                    crow0 = a.cu_q[s];
                    break;
                }
                tile -= nt;
            }
            if (seq < 0) return;
        }
    }
    const int ctx = a.ctx[seq];
    const int g = g0 + m;
    const bool valid = g < qlen * H;
    const int tq = valid ? g / H : 0, hh = valid ? g - tq * H : 0;
    const int pos = ctx - qlen + tq;  // keys 0..pos are visible to this row
    const long trow = (long)a.row_base + crow0 + tq;
    // keys this workgroup streams: up to the last row's position, within its partition
    const int t_last = min(qlen - 1, (g0 + BM - 1) / H);
    int k_begin = 0, k_end = ctx - qlen + t_last + 1;
    const int part = blockIdx.y;
    if (a.parts > 1) {
        k_begin = part * a.part_len;
        k_end = min(k_end, k_begin + a.part_len);
    }

    for (int i = tid; i < BM * RW; i += NTH) {
        const int mm = i / RW, r = i - mm * RW;
        const int gg = g0 + mm;
        float v = 0.f;
        if (gg < qlen * H && r < R) {
            const int t2 = gg / H, h2 = gg - t2 * H;
            v = ldf<B16>(a.qa, ((long)a.row_base + crow0 + t2) * a.qs_t + (long)h2 * a.qs_h + r) * a.scale;
        }
        QA[mm * RP + r] = v;
    }

    float m_run = -INFINITY, l_run = 0.f;
    f32x4 acc[RV];
#pragma unroll
    for (int i = 0; i < RV; ++i) acc[i] = f32x4{0.f, 0.f, 0.f, 0.f};
    const int* btr = a.bt + (long)seq * a.bt_stride;

    for (int k0 = k_begin; k0 < k_end; k0 += BN) {
        __syncthreads();  // the previous tile's readers are done (and QA is written, first time round)
        for (int i = tid; i < BN * RW; i += NTH) {
            const int j = i / RW, r = i - j * RW;
            const int key = k0 + j;
            float v = 0.f;
            if (key < k_end && r < R) {
                const int blk = btr[key / a.bs];
                v = ldf<B16>(a.cache, ((long)blk * a.bs + (key % a.bs)) * R + r);
            }
            CT[j * RP + r] = v;
        }
        __syncthreads();
        float s[NJ];
#pragma unroll
        for (int jj = 0; jj < NJ; ++jj) s[jj] = 0.f;
        const f32x4* q4 = (const f32x4*)(QA + m * RP);
#pragma unroll 2
        for (int r4 = 0; r4 < RW / 4; ++r4) {
            const f32x4 qv = q4[r4];
#pragma unroll
            for (int jj = 0; jj < NJ; ++jj) {
                const f32x4 cv = ((const f32x4*)(CT + (l8 + 8 * jj) * RP))[r4];
                s[jj] += qv[0] * cv[0] + qv[1] * cv[1] + qv[2] * cv[2] + qv[3] * cv[3];
            }
        }
        float mx = -INFINITY;
#pragma unroll
        for (int jj = 0; jj < NJ; ++jj) {
            const int key = k0 + l8 + 8 * jj;
            if (!(valid && key < k_end && key <= pos)) s[jj] = -INFINITY;
            mx = fmaxf(mx, s[jj]);
        }
        mx = fmaxf(mx, __shfl_xor(mx, 1, 64));
        mx = fmaxf(mx, __shfl_xor(mx, 2, 64));
        mx = fmaxf(mx, __shfl_xor(mx, 4, 64));
        const float m_new = fmaxf(m_run, mx);
        float alpha = 1.f, ls = 0.f;
        if (m_new == -INFINITY) {
#pragma unroll
            for (int jj = 0; jj < NJ; ++jj) s[jj] = 0.f;
        } else {
            alpha = __expf(m_run - m_new);  // m_run = -inf -> 0
#pragma unroll
            for (int jj = 0; jj < NJ; ++jj) {
                s[jj] = __expf(s[jj] - m_new);  // masked (-inf) -> 0
                ls += s[jj];
            }
        }
        ls += __shfl_xor(ls, 1, 64);
        ls += __shfl_xor(ls, 2, 64);
        ls += __shfl_xor(ls, 4, 64);
        l_run = l_run * alpha + ls;
        m_run = m_new;
#pragma unroll
        for (int jj = 0; jj < NJ; ++jj) PS[m * (BN + 1) + l8 + 8 * jj] = s[jj];
#pragma unroll
        for (int i = 0; i < RV; ++i) acc[i] *= alpha;
        __syncthreads();
        const int jn = min(BN, k_end - k0);
        for (int j = 0; j < jn; ++j) {
            const float p = PS[m * (BN + 1) + j];
            const f32x4* c4 = (const f32x4*)(CT + j * RP);
#pragma unroll
            for (int i = 0; i < RV; ++i) acc[i] += p * c4[l8 + 8 * i];
        }
    }

    if (!valid) return;
    if (a.parts > 1) {
        const long prow = ((long)seq * H + hh) * a.parts + part;
        if (l8 == 0) {
            a.part_ml[prow * 2] = m_run;
            a.part_ml[prow * 2 + 1] = l_run;
        }
#pragma unroll
        for (int i = 0; i < RV; ++i)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int col = 4 * l8 + 32 * i + e;
                if (col < R) a.part_o[prow * R + col] = acc[i][e];
            }
        return;
    }
    const float inv = l_run > 0.f ? 1.f / l_run : 0.f;
    const long ob = trow * a.os_t + (long)hh * a.os_h;
#pragma unroll
    for (int i = 0; i < RV; ++i)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int col = 4 * l8 + 32 * i + e;
            if (col < R) stf<B16>(a.out, ob + col, acc[i][e] * inv);
        }
}

// one block per (sequence, head): out = sum_p e^(m_p - M) o_p / sum_p e^(m_p - M) l_p
template <bool B16>
__global__ __launch_bounds__(256) void latent_attn_merge_kernel(const float* part_ml, const float* part_o, int parts,
                                                                int R, int H, int row_base, void* out, long os_t,
                                                                long os_h) {
    const int seq = blockIdx.x / H, hh = blockIdx.x - seq * H;
    const long p0 = (long)blockIdx.x * parts;
    float M = -INFINITY;
    for (int p = 0; p < parts; ++p) M = fmaxf(M, part_ml[(p0 + p) * 2]);
    float L = 0.f;
    for (int p = 0; p < parts; ++p) {
        const float mp = part_ml[(p0 + p) * 2];
        if (mp != -INFINITY) L += __expf(mp - M) * part_ml[(p0 + p) * 2 + 1];
    }
    const float inv = L > 0.f ? 1.f / L : 0.f;
    for (int c = threadIdx.x; c < R; c += 256) {
        float o = 0.f;
        for (int p = 0; p < parts; ++p) {
            const float mp = part_ml[(p0 + p) * 2];
            if (mp != -INFINITY) o += __expf(mp - M) * part_o[(p0 + p) * R + c];
        }
        stf<B16>(out, ((long)row_base + seq) * os_t + (long)hh * os_h + c, o * inv);
    }
}

template <bool B16, int RV, int BN, int BM>
int launch(const AttnArgs& a, int n_rows, hipStream_t st) {
    constexpr int RP = RV * 32 + 4;
    constexpr size_t lds = sizeof(float) * ((size_t)(BM + BN) * RP + (size_t)BM * (BN + 1));
    static_assert(lds <= 64 * 1024, "tile does not fit the LDS of a workgroup");
    const int tiles = a.cu_q ? (n_rows * a.H + BM - 1) / BM + a.n_seqs : a.n_seqs * ((a.H + BM - 1) / BM);
    dim3 grid(tiles, a.parts);
    latent_attn_kernel<B16, RV, BN, BM><<<grid, BM * 8, lds, st>>>(a);
    return (int)hipGetLastError();
}

template <bool B16>
int dispatch(const AttnArgs& a, int n_rows, hipStream_t st) {
    const int rv = (a.R + 31) / 32;
    if (rv <= 1) return launch<B16, 1, 64, 32>(a, n_rows, st);
    if (rv <= 2) return launch<B16, 2, 64, 32>(a, n_rows, st);
    if (rv <= 3) return launch<B16, 3, 64, 32>(a, n_rows, st);
    if (rv <= 4) return launch<B16, 4, 64, 32>(a, n_rows, st);
    if (rv <= 6) return launch<B16, 6, 16, 32>(a, n_rows, st);
    if (rv <= 8) return launch<B16, 8, 16, 32>(a, n_rows, st);
    if (rv <= 12) return launch<B16, 12, 8, 16>(a, n_rows, st);
    if (rv <= 16) return launch<B16, 16, 8, 16>(a, n_rows, st);
    return (int)hipErrorInvalidValue;
}

}  // namespace

// qa / out element [token row * s_t + head * s_h + r]; cache [blocks][bs][R]; bt [n_seqs][bt_stride] block tables;
// cu_q: chunk row offsets (relative to row_base) of n_seqs prompt chunks, or null for one row per sequence;
// ctx: context length of each sequence including this step's rows; parts > 1 (decode only): every sequence's keys
// are split into partitions of part_len and merged through part_ml [n_seqs * H * parts][2], part_o [..][R].
extern "C" int mxl_latent_attn(const void* qa, long qs_t, long qs_h, const void* cache, int is16, int bs, int R,
                               const int* bt, int bt_stride, const int* cu_q, const int* ctx, int n_seqs, int n_rows,
                               int row_base, void* out, long os_t, long os_h, float scale, int H, int parts,
                               int part_len, float* part_ml, float* part_o, hipStream_t st) {
    if (n_seqs <= 0 || n_rows <= 0) return 0;
    if (!(qa && cache && bt && ctx && out && bs > 0 && R > 0 && R <= 512 && H > 0 && bt_stride > 0 && parts >= 1))
        return (int)hipErrorInvalidValue;
    if (parts > 1 && (cu_q || !part_ml || !part_o || part_len <= 0 || parts > 65535)) return (int)hipErrorInvalidValue;
    AttnArgs a{qa, qs_t, qs_h, cache, bs, R, bt, bt_stride, cu_q, ctx, n_seqs, row_base, out, os_t, os_h, scale,
               H, parts, part_len, part_ml, part_o};
    int rc = is16 ? dispatch<true>(a, n_rows, st) : dispatch<false>(a, n_rows, st);
    if (rc != 0 || parts == 1) return rc;
    if (is16) latent_attn_merge_kernel<true><<<n_seqs * H, 256, 0, st>>>(part_ml, part_o, parts, R, H, row_base, out, os_t, os_h);
    else latent_attn_merge_kernel<false><<<n_seqs * H, 256, 0, st>>>(part_ml, part_o, parts, R, H, row_base, out, os_t, os_h);
    return (int)hipGetLastError();
}
