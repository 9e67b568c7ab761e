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
        __syncthreads();  // the previous tile's readers are done (and QA is written, on the first pass)
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

// one block per (sequence, head): out = sum_p e^(m_p - M) o_p / sum_p e^(m_p - M) l_p. The partitions' weights are
// worked out once into LDS (parts <= 1024), then every thread sums its columns over the partitions.
template <bool B16>
__global__ __launch_bounds__(256) void latent_attn_merge_kernel(const float* part_ml, const float* part_o, int parts,
                                                                int R, int H, int row_base, void* out, long os_t,
                                                                long os_h) {
    __shared__ float wgt[1024];
    __shared__ float red[8];
    const int seq = blockIdx.x / H, hh = blockIdx.x - seq * H;
    const long p0 = (long)blockIdx.x * parts;
    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    float mloc = -INFINITY;
    for (int p = tid; p < parts; p += 256) {
        const float mp = part_ml[(p0 + p) * 2];
        wgt[p] = mp;
        mloc = fmaxf(mloc, mp);
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) mloc = fmaxf(mloc, __shfl_xor(mloc, o, 64));
    if (lane == 0) red[wv] = mloc;
    __syncthreads();
    const float M = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    float lloc = 0.f;
    for (int p = tid; p < parts; p += 256) {
        const float mp = wgt[p];
        const float w = mp == -INFINITY ? 0.f : __expf(mp - M);
        wgt[p] = w;
        lloc += w * part_ml[(p0 + p) * 2 + 1];
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) lloc += __shfl_xor(lloc, o, 64);
    if (lane == 0) red[4 + wv] = lloc;
    __syncthreads();
    const float L = red[4] + red[5] + red[6] + red[7];
    const float inv = L > 0.f ? 1.f / L : 0.f;
    for (int c = tid; c < R; c += 256) {
        float o = 0.f;
#pragma unroll 4
        for (int p = 0; p < parts; ++p) o += wgt[p] * part_o[(p0 + p) * R + c];
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

// ---- the same attention on the matrix cores (bf16 storage, R a multiple of 8) ----------------------------------
// A workgroup of NW waves owns 16 NW consecutive (token, head) rows of one sequence; wave w holds rows 16 w .. + 15
// as MFMA 16x16x32 A fragments (absorbed queries, read once from HBM into registers). The visible keys stream in
// tiles of 32 latents through ONE LDS image [32][R_pad] shared by the waves, and the image serves both products:
//   S = qa . c^T : B fragment = 8 consecutive rank entries of one key  -> a 16-byte ds_read of the key's row;
//   O += P c     : B fragment = one rank entry of 8 consecutive keys   -> ds_read_b64_tr_b16, the hardware transpose
//                  (a 16-lane group reads a 4-key x 16-entry block, lane l gets entry l of the 4 keys).
// Scores, the online softmax and both accumulators are fp32; the weights are rounded to bf16 as MFMA operands.
MX_DEV float group_max16(float v) {
    v = fmaxf(v, __shfl_xor(v, 1, 64));
    v = fmaxf(v, __shfl_xor(v, 2, 64));
    v = fmaxf(v, __shfl_xor(v, 4, 64));
    return fmaxf(v, __shfl_xor(v, 8, 64));
}
MX_DEV float group_sum16(float v) {
    v += __shfl_xor(v, 1, 64);
    v += __shfl_xor(v, 2, 64);
    v += __shfl_xor(v, 4, 64);
    return v + __shfl_xor(v, 8, 64);
}

// RS = 2 splits the rank between two waves of a row tile: both compute the tile's full scores and softmax (no
// exchange, no extra barrier), each accumulates and writes one half of the output columns. Half the accumulators per
// wave let two waves share a SIMD at the widest ranks, which is what hides the latencies between a tile's steps.
template <int RV, int NW, int RS>
__global__ __launch_bounds__(NW * 64) __attribute__((amdgpu_waves_per_eu(RS == 2 ? 2 : 1)))
void latent_attn_mfma_kernel(AttnArgs a) {
    constexpr int RP = RV * 32, KT = 32, CSTR = RP * 2 + 16, PSTR = KT * 2 + 16, NTH = NW * 64;
    constexpr int BM = NW / RS * 16, NO = RV * 2 / RS;  // rows per workgroup, output column tiles per wave
    static_assert(NW % RS == 0 && (RV * 2) % RS == 0, "rank split");
    extern __shared__ __attribute__((aligned(16))) char smem[];
    char* c_lds = smem;                                   // [KT][CSTR] bf16 latents of the tile
    const int tid = threadIdx.x, wv = tid >> 6, lane = tid & 63, col = lane & 15, g = lane >> 4;
    const int wave = wv / RS, half = wv % RS;  // row tile of this wave, and which part of the rank it accumulates
    char* pw = smem + KT * CSTR + wv * 16 * PSTR;       // this wave's P [16][PSTR]
    const int H = a.H, R = a.R;
    const bf16_t* qa = (const bf16_t*)a.qa;
    const bf16_t* cache = (const bf16_t*)a.cache;

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
                    g0 = (nt - 1 - tile) * BM;  // a chunk's last rows see the most keys: their workgroups start first
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
    const int nrows = qlen * H;
    const int t_last = min(qlen - 1, (g0 + BM - 1) / H);
    int k_begin = 0, k_end = ctx - qlen + t_last + 1;
    const int part = blockIdx.y;
    if (a.parts > 1) {
        k_begin = part * a.part_len;
        k_end = min(k_end, k_begin + a.part_len);
    }
    // A fragments: row `col` of this wave
    bf16x8 qf[RV];
    {
        const int ga = g0 + 16 * wave + col;
        const bool va = ga < nrows;
        const int ta = va ? ga / H : 0, ha = va ? ga - ta * H : 0;
        const bf16_t* qr = qa + ((long)a.row_base + crow0 + ta) * a.qs_t + (long)ha * a.qs_h;
#pragma unroll
        for (int ks = 0; ks < RV; ++ks) {
            const int r = 32 * ks + 8 * g;
            u32x4 v = {0u, 0u, 0u, 0u};
            if (va && r < R) v = *(const u32x4*)(qr + r);
            qf[ks] = __builtin_bit_cast(bf16x8, v);
        }
    }
    // softmax / output rows 4 g + i of this wave
    int pos_i[4], head_i[4];
    long trow_i[4];
    bool valid_i[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int gi = g0 + 16 * wave + 4 * g + i;
        valid_i[i] = gi < nrows;
        const int t = valid_i[i] ? gi / H : 0;
        head_i[i] = valid_i[i] ? gi - t * H : 0;
        pos_i[i] = ctx - qlen + t;
        trow_i[i] = (long)a.row_base + crow0 + t;
    }
    float mrow[4], lrow[4];
    f32x4 oacc[NO];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        mrow[i] = -INFINITY;
        lrow[i] = 0.f;
    }
#pragma unroll
    for (int nt = 0; nt < NO; ++nt) oacc[nt] = (f32x4){0.f, 0.f, 0.f, 0.f};
    const int* btr = a.bt + (long)seq * a.bt_stride;
    const float scale = a.scale;
    const bool wave_active = g0 + 16 * wave < nrows;

    // A tile is KT * CPK 16-byte pieces. Each thread's first UB pieces of the NEXT tile are requested before the
    // current tile's products and stay in registers meanwhile (all of a tile when NTH * UB covers it); the rest
    // is loaded UB pieces at a time once the tile's turn has come.
    const int bs_shift = (a.bs & (a.bs - 1)) == 0 ? __builtin_ctz(a.bs) : -1;
    constexpr int CPK = RP / 8, TOTAL = KT * CPK, UB = (NW == 1 && RV > 8) || NW == 8 || (RS == 2 && RV > 12) ? 4 : 8;  // register room at the widest ranks
    u32x4 pre[UB];
    auto fetch = [&](int k0, int base, u32x4* v) {
#pragma unroll
        for (int u = 0; u < UB; ++u) {
            const int id = base + u * NTH + tid;
            const int p = id / CPK, c = id - p * CPK;
            const int key = k0 + p;
            v[u] = (u32x4){0u, 0u, 0u, 0u};
            if (id < TOTAL && key < k_end && c * 8 < R) {
                // block sizes are powers of two in practice: a shift instead of a division per piece
                const int bi = bs_shift >= 0 ? key >> bs_shift : key / a.bs;
                const int bo = key - bi * a.bs;
                v[u] = *(const u32x4*)(cache + ((long)btr[bi] * a.bs + bo) * R + c * 8);
            }
        }
    };
    auto stash = [&](int base, const u32x4* v) {
#pragma unroll
        for (int u = 0; u < UB; ++u) {
            const int id = base + u * NTH + tid;
            const int p = id / CPK, c = id - p * CPK;
            if (id < TOTAL) *(u32x4*)(c_lds + p * CSTR + c * 16) = v[u];
        }
    };
    if (k_begin < k_end) fetch(k_begin, 0, pre);
    for (int k0 = k_begin; k0 < k_end; k0 += KT) {
        __syncthreads();  // the previous tile's readers are done
        stash(0, pre);
        for (int base = NTH * UB; base < TOTAL; base += NTH * UB) {
            u32x4 v[UB];
            fetch(k0, base, v);
            stash(base, v);
        }
        __syncthreads();
        if (k0 + KT < k_end) fetch(k0 + KT, 0, pre);
        if (!wave_active) continue;  // a wave without rows only helps to fetch (the barriers are at the loop's top)
        // ---- S = qa c^T : 16 rows x 32 keys ----
        f32x4 sacc[2];
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            sacc[t] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < RV; ++ks) {
                const bf16x8 kf = *(const bf16x8*)(c_lds + (16 * t + col) * CSTR + (32 * ks + 8 * g) * 2);
                sacc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qf[ks], kf, sacc[t], 0, 0, 0);
            }
        }
        // ---- mask + online softmax (rows 4g+i, keys 16t+col) ----
        float alpha[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            float mx = -INFINITY;
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                const int key = k0 + 16 * t + col;
                float v = sacc[t][i] * scale;
                if (!valid_i[i] || key > pos_i[i] || key >= k_end) v = -INFINITY;
                sacc[t][i] = v;
                mx = fmaxf(mx, v);
            }
            mx = group_max16(mx);
            const float mn = fmaxf(mrow[i], mx);
            alpha[i] = mn == -INFINITY ? 1.f : __expf(mrow[i] - mn);
            float rs = 0.f;
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                const float pv = mn == -INFINITY ? 0.f : __expf(sacc[t][i] - mn);
                sacc[t][i] = pv;
                rs += pv;
            }
            lrow[i] = lrow[i] * alpha[i] + group_sum16(rs);
            mrow[i] = mn;
        }
        // the running maxima settle after the first tiles: rescale only when some row's maximum moved
        const bool moved = alpha[0] != 1.f || alpha[1] != 1.f || alpha[2] != 1.f || alpha[3] != 1.f;
        if (__builtin_amdgcn_ballot_w64(moved) != 0) {
#pragma unroll
            for (int nt = 0; nt < NO; ++nt)
#pragma unroll
                for (int i = 0; i < 4; ++i) oacc[nt][i] *= alpha[i];
        }
        // ---- P -> LDS (bf16), read back as the A fragment ----
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int i = 0; i < 4; ++i)
                *(bf16_t*)(pw + (4 * g + i) * PSTR + (16 * t + col) * 2) = f32_to_bf16(sacc[t][i]);
        __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): P visible to the wave (the same wave reads it)
        __builtin_amdgcn_wave_barrier();
        const bf16x8 pa = *(const bf16x8*)(pw + col * PSTR + (8 * g) * 2);
        // ---- O += P c ----
        const int q4 = col >> 2, p4 = col & 3;
        const char* vlo = c_lds + (8 * g + q4) * CSTR + 8 * p4 + half * NO * 32;
        const char* vhi = c_lds + (8 * g + 4 + q4) * CSTR + 8 * p4 + half * NO * 32;
#pragma unroll
        for (int nt = 0; nt < NO; ++nt) {
            const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((MX_LDS s16x4*)(vlo + nt * 32));
            const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((MX_LDS s16x4*)(vhi + nt * 32));
            // whole-vector reinterpretation (element-wise bit casts of the transposed read have been miscompiled)
            const u32x2 l2 = __builtin_bit_cast(u32x2, lo), h2 = __builtin_bit_cast(u32x2, hi);
            const u32x4 w4 = {l2[0], l2[1], h2[0], h2[1]};
            oacc[nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pa, __builtin_bit_cast(bf16x8, w4), oacc[nt], 0, 0, 0);
        }
        __builtin_amdgcn_s_waitcnt(0xc07f);  // the wave's P and tile reads have returned before either is rewritten
        __builtin_amdgcn_wave_barrier();
    }

    if (a.parts > 1) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            if (!valid_i[i]) continue;
            const long prow = ((long)seq * H + head_i[i]) * a.parts + part;
            if (col == 0 && half == 0) {
                a.part_ml[prow * 2] = mrow[i];
                a.part_ml[prow * 2 + 1] = lrow[i];
            }
#pragma unroll
            for (int nt = 0; nt < NO; ++nt) {
                const int r = 16 * (half * NO + nt) + col;
                if (r < R) a.part_o[prow * R + r] = oacc[nt][i];
            }
        }
        return;
    }
    bf16_t* out = (bf16_t*)a.out;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        if (!valid_i[i]) continue;
        const float inv = lrow[i] > 0.f ? 1.f / lrow[i] : 0.f;
        bf16_t* orow = out + trow_i[i] * a.os_t + (long)head_i[i] * a.os_h;
#pragma unroll
        for (int nt = 0; nt < NO; ++nt) {
            const int r = 16 * (half * NO + nt) + col;
            if (r < R) orow[r] = f32_to_bf16(oacc[nt][i] * inv);
        }
    }
}

template <int RV, int NW, int RS>
int launch_mfma(const AttnArgs& a, int n_rows, hipStream_t st) {
    constexpr int RP = RV * 32, BM = NW / RS * 16;
    constexpr size_t lds = (size_t)32 * (RP * 2 + 16) + (size_t)NW * 16 * (32 * 2 + 16);
    static_assert(lds <= 64 * 1024, "tile does not fit the LDS of a workgroup");
    const int tiles = a.cu_q ? (n_rows * a.H + BM - 1) / BM + a.n_seqs : a.n_seqs * ((a.H + BM - 1) / BM);
    dim3 grid(tiles, a.parts);
    latent_attn_mfma_kernel<RV, NW, RS><<<grid, NW * 64, lds, st>>>(a);
    return (int)hipGetLastError();
}

template <int RV>
int dispatch_mfma_nw(const AttnArgs& a, int n_rows, hipStream_t st) {
    // Row tiles per workgroup: prompt chunks four. A decode row set is one token's H heads: up to 16 take one row
    // tile, up to 32 two, more four. Ranks of 256 and more split each row tile between two waves (RS 2); narrower
    // ones keep one wave per row tile, with a second wave that only helps to fetch when there is a single row tile.
    const int rows = a.cu_q ? 64 : a.H;
    if constexpr (RV >= 8 && RV % 2 == 0) {
        if (rows <= 16) return launch_mfma<RV, 2, 2>(a, n_rows, st);
        if (rows <= 32) return launch_mfma<RV, 4, 2>(a, n_rows, st);
        return launch_mfma<RV, 8, 2>(a, n_rows, st);
    } else {
        if (rows <= 32) return launch_mfma<RV, 2, 1>(a, n_rows, st);
        return launch_mfma<RV, 4, 1>(a, n_rows, st);
    }
}

int dispatch_mfma(const AttnArgs& a, int n_rows, hipStream_t st) {
    const int rv = (a.R + 31) / 32;
    if (rv <= 1) return dispatch_mfma_nw<1>(a, n_rows, st);
    if (rv <= 2) return dispatch_mfma_nw<2>(a, n_rows, st);
    if (rv <= 3) return dispatch_mfma_nw<3>(a, n_rows, st);
    if (rv <= 4) return dispatch_mfma_nw<4>(a, n_rows, st);
    if (rv <= 6) return dispatch_mfma_nw<6>(a, n_rows, st);
    if (rv <= 8) return dispatch_mfma_nw<8>(a, n_rows, st);
    if (rv <= 12) return dispatch_mfma_nw<12>(a, n_rows, st);
    if (rv <= 16) return dispatch_mfma_nw<16>(a, n_rows, st);
    return (int)hipErrorInvalidValue;
}

// the matrix-core kernel reads queries and latents in 16-byte pieces
bool mfma_ok(const AttnArgs& a) {
    return a.R % 8 == 0 && a.qs_t % 8 == 0 && a.qs_h % 8 == 0 && ((uintptr_t)a.qa & 15) == 0 &&
           ((uintptr_t)a.cache & 15) == 0;
}

}  // namespace

// qa / out element [token row * s_t + head * s_h + r]; cache [blocks][bs][R]; bt [n_seqs][bt_stride] block tables;
// cu_q: chunk row offsets (relative to row_base) of n_seqs prompt chunks, or null for one row per sequence;
// ctx: context length of each sequence including this step's rows; impl: 0 auto, 1 the VALU kernel; parts > 1 (decode only): every sequence's keys
// are split into partitions of part_len and merged through part_ml [n_seqs * H * parts][2], part_o [..][R].
extern "C" int mxl_latent_attn(const void* qa, long qs_t, long qs_h, const void* cache, int is16, int bs, int R,
                               const int* bt, int bt_stride, const int* cu_q, const int* ctx, int n_seqs, int n_rows,
                               int row_base, void* out, long os_t, long os_h, float scale, int H, int parts,
                               int part_len, float* part_ml, float* part_o, int impl, hipStream_t st) {
    if (n_seqs <= 0 || n_rows <= 0) return 0;
    if (!(qa && cache && bt && ctx && out && bs > 0 && R > 0 && R <= 512 && H > 0 && bt_stride > 0 && parts >= 1))
        return (int)hipErrorInvalidValue;
    if (parts > 1 && (cu_q || !part_ml || !part_o || part_len <= 0 || parts > 1024)) return (int)hipErrorInvalidValue;
    AttnArgs a{qa, qs_t, qs_h, cache, bs, R, bt, bt_stride, cu_q, ctx, n_seqs, row_base, out, os_t, os_h, scale,
               H, parts, part_len, part_ml, part_o};
    // impl 0: matrix cores where the layout allows (bf16, 16-byte pieces), else the fp32 VALU kernel; 1: VALU always
    int rc;
    if (is16 && impl == 0 && mfma_ok(a)) rc = dispatch_mfma(a, n_rows, st);
    else rc = is16 ? dispatch<true>(a, n_rows, st) : dispatch<false>(a, n_rows, st);
    if (rc != 0 || parts == 1) return rc;
    if (is16) latent_attn_merge_kernel<true><<<n_seqs * H, 256, 0, st>>>(part_ml, part_o, parts, R, H, row_base, out, os_t, os_h);
    else latent_attn_merge_kernel<false><<<n_seqs * H, 256, 0, st>>>(part_ml, part_o, parts, R, H, row_base, out, os_t, os_h);
    return (int)hipGetLastError();
}
