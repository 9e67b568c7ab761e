// hybrid_attn.hip: causal softmax attention over paged key / value pools with a visible range that starts at a chunk
// border, a window's edge or position 0, and an optional sink term in the denominator (ops/hybrid.py
// masked_attention). Pools are token-major: keys [blocks, bs, G * dk], values [blocks, bs, G * dv], fp32 or bf16.
//
// attn_rows_kernel: one wave per (query row, query head). Keys are taken 64 at a time, one per lane: the lane forms
// its key's whole score against the query (held in LDS as fp32, pre-multiplied by the scale), the wave updates the
// running maximum and sum (fp32), and the lanes then share out the value columns, each accumulating
// sum_j p_j v_j[c] for its columns over the tile's keys. Scores, softmax and accumulators are fp32 for both pool
// formats. The sink is a virtual key of score 0 and value 0: the running maximum starts at 0 and the sum at 1.
#include "../mx_common.h"

namespace {

constexpr int DVU = 8;  // value columns per lane: heads of up to 512 numbers

template <bool B16>
MX_DEV float ld1(const void* p, long i) {
    if constexpr (B16) return bf16_to_f32(((const bf16_t*)p)[i]);
    else return ((const float*)p)[i];
}

// dot of a pool row with the fp32 query in LDS (n numbers, row and query 16-byte aligned when n % 8 == 0)
template <bool B16>
MX_DEV float dot_row(const void* base, long off, const float* q, int n) {
    float acc = 0.f;
    if ((n & 7) == 0) {
        if constexpr (B16) {
            const uint4* r = (const uint4*)((const bf16_t*)base + off);
            for (int i = 0; i < n / 8; ++i) {
                const uint4 w = r[i];
                const float* qq = q + i * 8;
                acc += __uint_as_float(w.x << 16) * qq[0] + __uint_as_float(w.x & 0xffff0000u) * qq[1];
                acc += __uint_as_float(w.y << 16) * qq[2] + __uint_as_float(w.y & 0xffff0000u) * qq[3];
                acc += __uint_as_float(w.z << 16) * qq[4] + __uint_as_float(w.z & 0xffff0000u) * qq[5];
                acc += __uint_as_float(w.w << 16) * qq[6] + __uint_as_float(w.w & 0xffff0000u) * qq[7];
            }
        } else {
            const float4* r = (const float4*)((const float*)base + off);
            for (int i = 0; i < n / 4; ++i) {
                const float4 w = r[i];
                const float* qq = q + i * 4;
                acc += w.x * qq[0] + w.y * qq[1] + w.z * qq[2] + w.w * qq[3];
            }
        }
        return acc;
    }
    for (int i = 0; i < n; ++i) acc += ld1<B16>(base, off + i) * q[i];
    return acc;
}

// grid (rows, H). cu_q == nullptr: row r is sequence r's single new token at position ctx[r] - 1; otherwise rows are
// chunks laid end to end, sequence s owning rows [cu_q[s], cu_q[s + 1]) that end at position ctx[s] - 1.
template <bool B16, bool O16>
__global__ __launch_bounds__(64) void attn_rows_kernel(const void* q, int ldq, const void* kc, const void* vc, int bs,
                                                       const int* bt, int bt_stride, const int* cu_q, const int* ctx,
                                                       int n_seqs, int row_base, void* out, int ldo, int H, int G,
                                                       int dk, int dv, float scale, int chunk, int window, int sink,
                                                       float out_scale) {
    extern __shared__ float lds[];  // [dk] query, [64] weights, [64] row offsets (as int pairs)
    float* qs = lds;
    float* ps = lds + dk;
    long* rowoff = (long*)(ps + 64 + ((dk & 1) ? 1 : 0));
    const int r = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    int s, pos;
    if (!cu_q) {
        s = r;
        pos = ctx[s] - 1;
    } else {
        int lo_ = 0, hi_ = n_seqs - 1;  // last s with cu_q[s] <= r
        while (lo_ < hi_) {
            const int mid = (lo_ + hi_ + 1) >> 1;
            if (cu_q[mid] <= r) lo_ = mid;
            else hi_ = mid - 1;
        }
        s = lo_;
        const int n = cu_q[s + 1] - cu_q[s];
        pos = ctx[s] - n + (r - cu_q[s]);
    }
    const int g = h / (H / G);
    const long qrow = (long)(row_base + r) * ldq + (long)h * dk;
    for (int e = lane; e < dk; e += 64) qs[e] = ld1<B16>(q, qrow + e) * scale;
    const int lo = chunk > 0 ? (pos / chunk) * chunk : window > 0 ? max(0, pos - window + 1) : 0;
    const int* table = bt + (long)s * bt_stride;
    float m = sink ? 0.f : -INFINITY, l = sink ? 1.f : 0.f;
    float acc[DVU];
#pragma unroll
    for (int u = 0; u < DVU; ++u) acc[u] = 0.f;
    __syncthreads();
    for (int j0 = lo; j0 <= pos; j0 += 64) {
        const int j = j0 + lane;
        const bool ok = j <= pos;
        float sc = -INFINITY;
        long tok = 0;
        if (ok) {
            tok = (long)table[j / bs] * bs + (j % bs);
            sc = dot_row<B16>(kc, (tok * G + g) * dk, qs, dk);
        }
        const float mn = fmaxf(m, wave_max(sc));
        const float p = ok ? expf(sc - mn) : 0.f;
        const float alpha = expf(m - mn);  // 0 on the first tile without a sink (m = -inf, mn finite: the tile has key lo)
        l = l * alpha + wave_sum(p);
        m = mn;
        __syncthreads();  // the previous tile's weights and offsets have been read
        ps[lane] = p;
        rowoff[lane] = (tok * G + g) * dv;
        __syncthreads();
        const int nk = min(64, pos - j0 + 1);
#pragma unroll
        for (int u = 0; u < DVU; ++u) {
            const int c = lane + u * 64;
            if (c < dv) {
                float a = acc[u] * alpha;
                for (int jj = 0; jj < nk; ++jj) a += ps[jj] * ld1<B16>(vc, rowoff[jj] + c);
                acc[u] = a;
            }
        }
    }
    const float inv = out_scale / l;
    const long orow = (long)(row_base + r) * ldo + (long)h * dv;
#pragma unroll
    for (int u = 0; u < DVU; ++u) {
        const int c = lane + u * 64;
        if (c < dv) {
            if constexpr (O16) ((bf16_t*)out)[orow + c] = f32_to_bf16(acc[u] * inv);
            else ((float*)out)[orow + c] = acc[u] * inv;
        }
    }
}

}  // namespace

#define MXH_CHECK(cond) \
    if (!(cond)) return (int)hipErrorInvalidValue

extern "C" int mxh_attention(const void* q, int ldq, int q16, const void* kc, const void* vc, int bs, const int* bt,
                             int bt_stride, const int* cu_q, const int* ctx, int n_seqs, int n_rows, int row_base,
                             void* out, int ldo, int o16, int H, int G, int dk, int dv, float scale, int chunk,
                             int window, int sink, float out_scale, hipStream_t st) {
    if (n_rows <= 0 || n_seqs <= 0) return 0;
    MXH_CHECK(q && kc && vc && bt && ctx && out && bs > 0 && bt_stride > 0);
    MXH_CHECK(H > 0 && G > 0 && H % G == 0 && dk > 0 && dv > 0 && dv <= 64 * DVU && dk <= 4096);
    MXH_CHECK(ldq >= H * dk && ldo >= H * dv && chunk >= 0 && window >= 0 && H <= 65535);
    MXH_CHECK(cu_q || n_rows == n_seqs);
    const dim3 grid(n_rows, H);
    const size_t sh = (size_t)(dk + 64 + 2) * sizeof(float) + 64 * sizeof(long);
#define GO(B, O)                                                                                                    \
    attn_rows_kernel<B, O><<<grid, 64, sh, st>>>(q, ldq, kc, vc, bs, bt, bt_stride, cu_q, ctx, n_seqs, row_base, out, \
                                                 ldo, H, G, dk, dv, scale, chunk, window, sink, out_scale)
    if (q16 && o16) GO(true, true);
    else if (q16) GO(true, false);
    else if (o16) GO(false, true);
    else GO(false, false);
#undef GO
    return (int)hipGetLastError();
}
