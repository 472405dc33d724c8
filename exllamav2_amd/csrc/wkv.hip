// wkv.hip -- a linear-attention mixer with a per-channel, data-dependent decay (RWKV-style time mixing) for gfx950, + its C ABI.
//
// Per head, with r, k (key channels i = 0 .. N) and v (value channels j = 0 .. P) of the token, a decay w_i in (0, 1) and a bonus u_i
// that only the current token gets, the state S (N x P, fp32) gives
//     o_j = sum_i r_i (S_ij + u_i k_i v_j),        S_ij <- w_i S_ij + k_i v_j,
// the head's o is divided by its root mean square, multiplied by a weight per channel and by the gate silu(g), and leaves in the
// operand dtype for the output projection.  The decay comes as d = log(-log w) (w = exp(-exp(d)), evaluated here in fp32).
//
// The five projections read five blends of the mixer's input h with the previous token's input h':  h + (h' - h) * mu_s.
// wkv_mix_kernel makes them from the fp32 input rows: h' is the row in front when that belongs to the same sequence, else what the
// sequence's slot keeps, zeros at position 0.
//
// Rows of a step are a flat list; a span is the run of consecutive rows one sequence brings (span i = rows span_row0[i] ..
// + span_rows[i], slot and first position = row_seq / row_pos of its first row).  A span at position 0 starts from zeros whatever
// its slot holds.  Everything here is fp32 except the operand-dtype outputs.
#include "hw.h"
#include "errors.h"
#include <stdint.h>

template <typename T> DEV float wk_ld(const T* p);
template <> DEV float wk_ld<u16>(const u16* p) { return bf16_to_f32(*p); }
template <> DEV float wk_ld<float>(const float* p) { return *p; }
template <typename T> DEV void wk_st(T* p, float v);
template <> DEV void wk_st<u16>(u16* p, float v) { *p = f32_to_bf16(v); }
template <> DEV void wk_st<float>(float* p, float v) { *p = v; }

extern "C" int exl2_span_last_rows(const float* src, int ld, float* slot_rows, int width, const int* span_row0, const int* span_rows,
                                   int spans, const int* row_seq, void* stream);

// ---- the blends -------------------------------------------------------------------------------------------------------------------

struct MixArgs
{
    const float* h; int width;               // [rows, width]
    float* prev;                             // [slots, width]
    const void* mu; int n_mix;               // [n_mix, width] operand dtype
    void* out; long long out_stride;         // blend s at out + s * out_stride: [rows, width] operand dtype
    const int* row_seq; const int* row_pos;
    int fused;                               // single-row spans: the slot is rolled here
};

// grid (rows, width / 256)
template <typename T>
KERNEL void __launch_bounds__(256) wkv_mix_kernel(const MixArgs a)
{
    const int r = bid_x(), i = bid_y() * 256 + tid();
    if (i >= a.width) return;
    const int pos = a.row_pos[r], sq = a.row_seq[r];
    const float hv = a.h[(long long)r * a.width + i];
    float hp = 0.0f;
    if (pos > 0) hp = (!a.fused && r > 0 && a.row_seq[r - 1] == sq) ? a.h[(long long)(r - 1) * a.width + i] : a.prev[(long long)sq * a.width + i];
    if (a.fused) a.prev[(long long)sq * a.width + i] = hv;
    const float d = hp - hv;
    for (int s = 0; s < a.n_mix; s++)
        wk_st<T>((T*)a.out + s * a.out_stride + (long long)r * a.width + i, fmaf(d, wk_ld<T>((const T*)a.mu + (long long)s * a.width + i), hv));
}

// ---- the recurrence, token by token ---------------------------------------------------------------------------------------------------

#define WKV_CHUNK 16                         // tokens staged in LDS per round
#define WKV_MAX_NPT 256                      // state rows per thread

struct WkvArgs
{
    const float* r; const float* k; const float* v; const float* g; int ld;      // [rows, ld] each: head h at h * N (r, k) or h * P (v, g)
    const float* dlog; int ldd;              // [rows, ldd]: log(-log w), head h at h * N
    const float* u;                          // [heads, N]
    const float* norm_w;                     // [heads * P]
    void* out; int ldo;                      // [rows, ldo] operand dtype (or fp32)
    float* state;                            // [slots, heads, N, P]
    const int* span_row0; const int* span_rows; const int* row_seq; const int* row_pos;
    int heads, N, P, KS;                     // KS = threads that share a column of the state (blockDim = P * KS rounded up to waves)
    float eps;
};

// Workgroup = one (span, head): thread (j, p) holds rows n = j, j + KS, .. of column p of the state in registers for the whole span.
// Tokens are taken WKV_CHUNK at a time: r, k, the decay and v are staged in LDS, every thread steps its rows through the chunk keeping
// one partial sum per token, the KS partial sums of a column are added at the chunk's end, and a wave per token takes the head's
// root mean square and writes the normed, gated row.
template <typename T, int NPT>
KERNEL void __launch_bounds__(256) wkv_scan_kernel(const WkvArgs a)
{
    DYN_SMEM(smem);
    const int h = bid_x(), sp = bid_y();
    const int n_tok = a.span_rows[sp], r0 = a.span_row0[sp];
    const int pos0 = a.row_pos[r0];
    const int P = a.P, N = a.N, KS = a.KS;
    const int t = tid(), nt = nthreads();
    const bool owner = t < P * KS;
    const int p = t % P, j = t / P;
    float* s_r = (float*)smem;                                   // [CHUNK, N]
    float* s_k = s_r + WKV_CHUNK * N;                            // [CHUNK, N]
    float* s_w = s_k + WKV_CHUNK * N;                            // [CHUNK, N]
    float* s_v = s_w + WKV_CHUNK * N;                            // [CHUNK, P]
    float* s_o = s_v + WKV_CHUNK * P;                            // [CHUNK, P]
    float* s_part = s_o + WKV_CHUNK * P;                         // [CHUNK, KS, P]
    float* s_u = s_part + WKV_CHUNK * KS * P;                    // [N]
    float* st = a.state + ((long long)a.row_seq[r0] * a.heads + h) * (long long)N * P;
    float S[NPT];
    #pragma unroll
    for (int i = 0; i < NPT; i++)
    {
        const int n = j + KS * i;
        S[i] = (owner && pos0 > 0 && n < N) ? st[(long long)n * P + p] : 0.0f;
    }
    for (int i = t; i < N; i += nt) s_u[i] = a.u[h * N + i];
    for (int c0 = 0; c0 < n_tok; c0 += WKV_CHUNK)
    {
        const int nc = min(WKV_CHUNK, n_tok - c0);
        block_sync();
        for (int i = t; i < nc * N; i += nt)
        {
            const long long row = r0 + c0 + i / N;
            const int n = i % N;
            s_r[i] = a.r[row * a.ld + h * N + n];
            s_k[i] = a.k[row * a.ld + h * N + n];
            s_w[i] = expf(-expf(a.dlog[row * a.ldd + h * N + n]));
        }
        for (int i = t; i < nc * P; i += nt) s_v[i] = a.v[(long long)(r0 + c0 + i / P) * a.ld + h * P + i % P];
        block_sync();
        for (int kk = 0; owner && kk < nc; kk++)
        {
            const float vv = s_v[kk * P + p];
            float part = 0.0f;
            #pragma unroll
            for (int i = 0; i < NPT; i++)
            {
                const int n = j + KS * i;
                if (n < N)
                {
                    const float kv = s_k[kk * N + n] * vv;
                    part = fmaf(s_r[kk * N + n], fmaf(s_u[n], kv, S[i]), part);
                    S[i] = fmaf(s_w[kk * N + n], S[i], kv);
                }
            }
            s_part[(kk * KS + j) * P + p] = part;
        }
        block_sync();
        for (int i = t; i < nc * P; i += nt)
        {
            const int kk = i / P, pp = i % P;
            float ov = 0.0f;
            for (int jj = 0; jj < KS; jj++) ov += s_part[(kk * KS + jj) * P + pp];
            s_o[i] = ov;
        }
        block_sync();
        for (int kk = wave_id(); kk < nc; kk += nt / 64)
        {
            float ss = 0.0f;
            for (int pp = lane_id(); pp < P; pp += 64) { const float ov = s_o[kk * P + pp]; ss = fmaf(ov, ov, ss); }
            ss = wave_allreduce_add(ss);
            const float rinv = 1.0f / sqrtf(ss / (float)P + a.eps);
            const long long row = r0 + c0 + kk;
            for (int pp = lane_id(); pp < P; pp += 64)
            {
                const float gv = a.g[row * a.ld + h * P + pp];
                const float o = s_o[kk * P + pp] * rinv * a.norm_w[h * P + pp] * (gv / (1.0f + expf(-gv)));
                wk_st<T>((T*)a.out + row * a.ldo + h * P + pp, o);
            }
        }
    }
    #pragma unroll
    for (int i = 0; i < NPT; i++)
    {
        const int n = j + KS * i;
        if (owner && n < N) st[(long long)n * P + p] = S[i];
    }
}

// ---- the same recurrence in chunks (portions of prompts) ------------------------------------------------------------------------------
// Inside a chunk of WKC_L tokens the recurrence unrolls.  With l_t = log w_t = -exp(d_t) (per key channel), c_t = l_1 + .. + l_t and
// c_0 = 0:
//     o_t = (r_t * exp(c_{t-1}))^T S_in + sum_{s < t} A_ts v_s + (r_t . (u * k_t)) v_t,   A_ts = sum_i r_t[i] k_s[i] exp(c_{t-1}[i] - c_s[i]),
//     S_out = diag(exp(c_L)) S_in + sum_s diag(exp(c_L - c_s)) k_s v_s^T.
// Every exponent is a difference of the running sum taken the right way round (<= 0), evaluated per (t, s, channel): no factor
// exp(-c_s) that a fast decay would overflow.  Three launches make every (chunk, head) of a step independent work: (1) each chunk's
// own contribution Z to S_out and its total decay, (2) the carry over a span's chunks, one thread per state element (Z is replaced by
// the state ENTERING the chunk, the slot takes the state after the last), (3) each chunk's outputs with the head norm and gate.

#define WKC_L 64

struct WkvChunkArgs
{
    WkvArgs a;
    const int* span_chunk0; int spans;       // chunks in front of each span
    float* zbuf;                             // [chunks, heads, N, P]
    float* dbuf;                             // [chunks, heads, N]
};

// chunk c of the step -> its span, first row and row count
DEV void wkc_locate(const WkvChunkArgs& g, int c, int& sp, int& r0, int& n)
{
    sp = 0;
    for (int i = 1; i < g.spans; i++) if (g.span_chunk0[i] <= c) sp = i;
    const int first = (c - g.span_chunk0[sp]) * WKC_L;
    r0 = g.a.span_row0[sp] + first;
    n = min(WKC_L, g.a.span_rows[sp] - first);
}

// cc[0] = 0, cc[t + 1] = c_t for the chunk's n tokens (rows of NS floats); all threads call it
DEV void wkc_log_decay_sums(const WkvArgs& a, int h, int r0, int n, float* cc, int NS)
{
    const int N = a.N;
    for (int i = tid(); i < (n + 1) * N; i += nthreads())
    {
        const int t = i / N, ch = i % N;
        cc[t * NS + ch] = t == 0 ? 0.0f : -expf(a.dlog[(long long)(r0 + t - 1) * a.ldd + h * N + ch]);
    }
    block_sync();
    // running sums in two levels: segments of 8 tokens by N x 8 threads, then every channel's thread adds the sum of the segments in
    // front to the later segments (independent updates: only the 8 segment totals form a chain)
    for (int i = tid(); i < N * (WKC_L / 8); i += nthreads())
    {
        const int ch = i % N, t0 = (i / N) * 8;
        float run = 0.0f;
        #pragma unroll
        for (int q = 1; q <= 8; q++)
            if (t0 + q <= n) { run += cc[(t0 + q) * NS + ch]; cc[(t0 + q) * NS + ch] = run; }
    }
    block_sync();
    for (int ch = tid(); ch < N; ch += nthreads())
    {
        float off[WKC_L / 8];
        float run = 0.0f;
        #pragma unroll
        for (int sg = 0; sg < WKC_L / 8; sg++)
        {
            off[sg] = run;
            if (sg * 8 < n) run += cc[min(sg * 8 + 8, n) * NS + ch];
        }
        #pragma unroll
        for (int sg = 1; sg < WKC_L / 8; sg++)
            #pragma unroll
            for (int q = 1; q <= 8; q++)
                if (sg * 8 + q <= n) cc[(sg * 8 + q) * NS + ch] += off[sg];
    }
    block_sync();
}

// grid (chunks, heads)
KERNEL void __launch_bounds__(512) wkv_chunk_state_kernel(const WkvChunkArgs g)
{
    DYN_SMEM(smem);
    const WkvArgs& a = g.a;
    const int c = bid_x(), h = bid_y(), N = a.N, P = a.P, NS = N + 1;
    int sp, r0, n;
    wkc_locate(g, c, sp, r0, n);
    float* sv = (float*)smem;                                    // [L][P] (first: 16-byte aligned rows when P % 4 == 0)
    float* cc = sv + WKC_L * P;                                  // [L + 1][NS]
    float* kd = cc + (WKC_L + 1) * NS;                           // [L][NS]
    wkc_log_decay_sums(a, h, r0, n, cc, NS);
    for (int i = tid(); i < n * N; i += nthreads())
    {
        const int t = i / N, ch = i % N;
        kd[t * NS + ch] = expf(cc[n * NS + ch] - cc[(t + 1) * NS + ch]) * a.k[(long long)(r0 + t) * a.ld + h * N + ch];
    }
    for (int i = tid(); i < n * P; i += nthreads()) sv[i] = a.v[(long long)(r0 + i / P) * a.ld + h * P + i % P];
    block_sync();
    float* z = g.zbuf + ((long long)c * a.heads + h) * N * P;
    if (N % 4 == 0 && P % 4 == 0)
    {
        // 4 x 4 outputs per thread: every staged value feeds four products
        for (int e = tid(); e < (N / 4) * (P / 4); e += nthreads())
        {
            const int ch = (e / (P / 4)) * 4, j = (e % (P / 4)) * 4;
            float acc[4][4] = {};
            #pragma unroll 2
            for (int t = 0; t < n; t++)
            {
                const f32x4 vv = *(const f32x4*)(sv + t * P + j);
                #pragma unroll
                for (int q = 0; q < 4; q++)
                {
                    const float kq = kd[t * NS + ch + q];
                    acc[q][0] = fmaf(kq, vv[0], acc[q][0]); acc[q][1] = fmaf(kq, vv[1], acc[q][1]);
                    acc[q][2] = fmaf(kq, vv[2], acc[q][2]); acc[q][3] = fmaf(kq, vv[3], acc[q][3]);
                }
            }
            #pragma unroll
            for (int q = 0; q < 4; q++) *(f32x4*)(z + (ch + q) * P + j) = (f32x4){acc[q][0], acc[q][1], acc[q][2], acc[q][3]};
        }
    }
    else
        for (int e = tid(); e < N * P; e += nthreads())
        {
            const int ch = e / P, j = e % P;
            float acc = 0.0f;
            #pragma unroll 4
            for (int t = 0; t < n; t++) acc = fmaf(kd[t * NS + ch], sv[t * P + j], acc);
            z[e] = acc;
        }
    for (int ch = tid(); ch < N; ch += nthreads()) g.dbuf[((long long)c * a.heads + h) * N + ch] = expf(cc[n * NS + ch]);
}

// grid (spans, heads, N * P / 256)
KERNEL void __launch_bounds__(256) wkv_chunk_carry_kernel(const WkvChunkArgs g)
{
    const WkvArgs& a = g.a;
    const int sp = bid_x(), h = bid_y(), e = bid_z() * 256 + tid();
    const int N = a.N, P = a.P;
    if (e >= N * P) return;
    const int r0 = a.span_row0[sp], chunks = (a.span_rows[sp] + WKC_L - 1) / WKC_L, c0 = g.span_chunk0[sp];
    float* st = a.state + ((long long)a.row_seq[r0] * a.heads + h) * (long long)N * P;
    float S = a.row_pos[r0] > 0 ? st[e] : 0.0f;
    for (int c = c0; c < c0 + chunks; c++)
    {
        float* z = g.zbuf + ((long long)c * a.heads + h) * N * P;
        const float own = z[e];
        z[e] = S;
        S = fmaf(g.dbuf[((long long)c * a.heads + h) * N + e / P], S, own);
    }
    st[e] = S;
}

// grid (chunks, heads)
template <typename T>
KERNEL void __launch_bounds__(1024) wkv_chunk_out_kernel(const WkvChunkArgs g)
{
    DYN_SMEM(smem);
    const WkvArgs& a = g.a;
    const int c = bid_x(), h = bid_y(), N = a.N, P = a.P, NS = N + 1, LS = WKC_L + 1;
    int sp, r0, n;
    wkc_locate(g, c, sp, r0, n);
    // four regions, two of them used twice (so that two workgroups share a CU's LDS at 64 x 64): the decay sums give way to the
    // values, the keys to the outputs; the state entering the chunk is read from memory where it is used
    const int PS = max(NS, P);
    float* cc = (float*)smem;                                    // [L + 1][PS]: decay sums (rows of NS), later the values [L][P]
    float* sr = cc + (WKC_L + 1) * PS;                           // [L][NS]
    float* sk = sr + WKC_L * NS;                                 // [L][PS]: keys (rows of NS), later the outputs [L][P]
    float* sA = sk + WKC_L * PS;                                 // [L][LS]
    float* su = sA + WKC_L * LS;                                 // [N]
    float* sv = cc; float* so = sk;
    const float* sS = g.zbuf + ((long long)c * a.heads + h) * N * P;
    wkc_log_decay_sums(a, h, r0, n, cc, NS);
    for (int i = tid(); i < n * N; i += nthreads())
    {
        const int t = i / N, ch = i % N;
        const long long at = (long long)(r0 + t) * a.ld + h * N + ch;
        sr[t * NS + ch] = a.r[at];
        sk[t * NS + ch] = a.k[at];
    }
    for (int ch = tid(); ch < N; ch += nthreads()) su[ch] = a.u[h * N + ch];
    block_sync();
    // A[t][s], s < t: a run of WKC_L threads takes rows t and WKC_L - 1 - t together (t + (WKC_L - 1 - t) entries below the diagonal:
    // every lane has work); consecutive threads take consecutive s (rows of sk / cc NS apart: distinct banks).  The diagonal and the
    // zeros above it come first.
    for (int e = tid(); e < WKC_L * WKC_L; e += nthreads())
    {
        const int t = e / WKC_L, s2 = e % WKC_L;
        if (s2 > t) sA[t * LS + s2] = 0.0f;
    }
    for (int t = tid(); t < WKC_L; t += nthreads())              // the diagonal: one thread per row, the rows side by side in a wave
    {
        float acc = 0.0f;
        if (t < n)
            #pragma unroll 8
            for (int ch = 0; ch < N; ch++) acc = fmaf(sr[t * NS + ch] * su[ch], sk[t * NS + ch], acc);
        sA[t * LS + t] = acc;
    }
    for (int e = tid(); e < (WKC_L / 2) * WKC_L; e += nthreads())
    {
        const int pair = e / WKC_L, l = e % WKC_L;
        const int t = l < pair ? pair : WKC_L - 1 - pair, s2 = l < pair ? l : l - pair;
        if (s2 >= t || t >= n) continue;
        const float* rt = sr + t * NS; const float* ct = cc + t * NS;
        const float* ks = sk + s2 * NS; const float* cs = cc + (s2 + 1) * NS;
        float acc = 0.0f;
        #pragma unroll 8
        for (int ch = 0; ch < N; ch++) acc = fmaf(rt[ch] * ks[ch], fast_exp(ct[ch] - cs[ch]), acc);
        sA[t * LS + s2] = acc;
    }
    block_sync();
    for (int i = tid(); i < n * N; i += nthreads())
    {
        const int t = i / N, ch = i % N;
        sr[t * NS + ch] *= expf(cc[t * NS + ch]);
    }
    block_sync();                                                // the decay sums and the keys have been used: their regions take v and o
    for (int i = tid(); i < n * P; i += nthreads()) sv[i] = a.v[(long long)(r0 + i / P) * a.ld + h * P + i % P];
    block_sync();
    // four rows of the chunk per thread share every read of the state and of a value row (A is zero above the diagonal)
    for (int e = tid(); e < (WKC_L / 4) * P; e += nthreads())
    {
        const int t0 = (e / P) * 4, j = e % P;
        if (t0 >= n) continue;
        float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
        #pragma unroll 4
        for (int ch = 0; ch < N; ch++)
        {
            const float sv2 = sS[ch * P + j];
            #pragma unroll
            for (int q = 0; q < 4; q++) acc[q] = fmaf(sr[(t0 + q) * NS + ch], sv2, acc[q]);
        }
        const int s_hi = min(t0 + 3, n - 1);
        #pragma unroll 4
        for (int s2 = 0; s2 <= s_hi; s2++)
        {
            const float vv = sv[s2 * P + j];
            #pragma unroll
            for (int q = 0; q < 4; q++) acc[q] = fmaf(sA[(t0 + q) * LS + s2], vv, acc[q]);
        }
        #pragma unroll
        for (int q = 0; q < 4; q++) if (t0 + q < n) so[(t0 + q) * P + j] = acc[q];
    }
    block_sync();
    for (int t = wave_id(); t < n; t += nthreads() / 64)
    {
        float ss = 0.0f;
        for (int j = lane_id(); j < P; j += 64) { const float ov = so[t * P + j]; ss = fmaf(ov, ov, ss); }
        ss = wave_allreduce_add(ss);
        const float rinv = 1.0f / sqrtf(ss / (float)P + a.eps);
        const long long row = r0 + t;
        for (int j = lane_id(); j < P; j += 64)
        {
            const float gv = a.g[row * a.ld + h * P + j];
            wk_st<T>((T*)a.out + row * a.ldo + h * P + j, so[t * P + j] * rinv * a.norm_w[h * P + j] * (gv / (1.0f + expf(-gv))));
        }
    }
}

static size_t wkc_out_smem(int N, int P)
{
    const size_t ps = N + 1 > P ? N + 1 : P;
    return sizeof(float) * ((size_t)(2 * WKC_L + 1) * ps + (size_t)WKC_L * (N + 1) + (size_t)WKC_L * (WKC_L + 1) + N);
}

// ---- C ABI ----------------------------------------------------------------------------------------------------------------------

extern "C" int exl2_wkv_mix(const float* h, float* prev, const void* mu, int n_mix, void* out, long long out_stride, const int* row_seq,
                            const int* row_pos, const int* span_row0, const int* span_rows, int spans, int max_span_rows, int dtype,
                            int rows, int width, void* stream)
{
    EXL2_REQUIRE(h && prev && mu && out && row_seq && row_pos && span_row0 && span_rows, "wkv_mix: null operand");
    EXL2_REQUIRE(dtype == 0 || dtype == 1, "wkv_mix: dtype must be 0 (bfloat16) or 1 (float32)");
    EXL2_REQUIRE(n_mix > 0 && width > 0 && out_stride >= (long long)rows * width, "wkv_mix: bad shape");
    if (rows <= 0 || spans <= 0) return EXL2_OK;
    MixArgs a;
    a.h = h; a.width = width; a.prev = prev; a.mu = mu; a.n_mix = n_mix; a.out = out; a.out_stride = out_stride; a.row_seq = row_seq;
    a.row_pos = row_pos; a.fused = max_span_rows == 1;
    const dim3 grid(rows, (width + 255) / 256);
    if (dtype == 0) LAUNCH(wkv_mix_kernel<u16>, grid, dim3(256), 0, stream, a);
    else LAUNCH(wkv_mix_kernel<float>, grid, dim3(256), 0, stream, a);
    HIP_TRY(hipGetLastError());
    if (!a.fused) return exl2_span_last_rows(h, width, prev, width, span_row0, span_rows, spans, row_seq, stream);
    return EXL2_OK;
}

template <typename T>
static void wkv_scan_launch(const WkvArgs& a, int npt, dim3 grid, dim3 block, size_t smem, void* stream)
{
    if (npt <= 8) LAUNCH((wkv_scan_kernel<T, 8>), grid, block, smem, stream, a);
    else if (npt <= 16) LAUNCH((wkv_scan_kernel<T, 16>), grid, block, smem, stream, a);
    else if (npt <= 32) LAUNCH((wkv_scan_kernel<T, 32>), grid, block, smem, stream, a);
    else if (npt <= 64) LAUNCH((wkv_scan_kernel<T, 64>), grid, block, smem, stream, a);
    else if (npt <= 128) LAUNCH((wkv_scan_kernel<T, 128>), grid, block, smem, stream, a);
    else LAUNCH((wkv_scan_kernel<T, WKV_MAX_NPT>), grid, block, smem, stream, a);
}

extern "C" int exl2_wkv_scan(const float* r, const float* k, const float* v, const float* g, int ld, const float* dlog, int ldd,
                             const float* u, const float* norm_w, void* out, int ldo, int out_f32, float* state,
                             const int* span_row0, const int* span_rows, int spans, const int* row_seq, const int* row_pos,
                             int heads, int n_key, int n_val, float eps, void* stream)
{
    EXL2_REQUIRE(r && k && v && g && dlog && u && norm_w && out && state && span_row0 && span_rows && row_seq && row_pos,
                 "wkv_scan: null operand");
    EXL2_REQUIRE(heads > 0 && n_key > 0 && n_val > 0 && n_val <= 256, "wkv_scan: state %d x %d", n_key, n_val);
    if (spans <= 0) return EXL2_OK;
    int ks = 256 / n_val;
    if (ks < 1) ks = 1;
    if (ks > n_key) ks = n_key;
    const int npt = (n_key + ks - 1) / ks;
    EXL2_REQUIRE(npt <= WKV_MAX_NPT, "wkv_scan: state %d x %d needs %d rows per thread (at most %d)", n_key, n_val, npt, WKV_MAX_NPT);
    WkvArgs a;
    a.r = r; a.k = k; a.v = v; a.g = g; a.ld = ld; a.dlog = dlog; a.ldd = ldd; a.u = u; a.norm_w = norm_w; a.out = out; a.ldo = ldo;
    a.state = state; a.span_row0 = span_row0; a.span_rows = span_rows; a.row_seq = row_seq; a.row_pos = row_pos;
    a.heads = heads; a.N = n_key; a.P = n_val; a.KS = ks; a.eps = eps;
    const size_t smem = sizeof(float) * ((size_t)WKV_CHUNK * (3 * n_key + 2 * n_val + (size_t)ks * n_val) + n_key);
    EXL2_REQUIRE(smem <= 150 * 1024, "wkv_scan: state %d x %d does not fit the staging buffers", n_key, n_val);
    if (smem > 48 * 1024)
    {
        static bool attr_done[EXL2_MAX_DEVICES];
        if (exl2_first_on_device(attr_done))
        {
            (void)hipFuncSetAttribute((const void*)wkv_scan_kernel<u16, 128>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
            (void)hipFuncSetAttribute((const void*)wkv_scan_kernel<float, 128>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
            (void)hipFuncSetAttribute((const void*)wkv_scan_kernel<u16, WKV_MAX_NPT>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
            (void)hipFuncSetAttribute((const void*)wkv_scan_kernel<float, WKV_MAX_NPT>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
            (void)hipFuncSetAttribute((const void*)wkv_scan_kernel<u16, 64>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
            (void)hipFuncSetAttribute((const void*)wkv_scan_kernel<float, 64>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        }
    }
    const dim3 grid(heads, spans), block((n_val * ks + 63) / 64 * 64);
    if (out_f32) wkv_scan_launch<float>(a, npt, grid, block, smem, stream);
    else wkv_scan_launch<u16>(a, npt, grid, block, smem, stream);
    HIP_TRY(hipGetLastError());
    return EXL2_OK;
}

/* 1 if exl2_wkv_scan_chunked takes this state shape (its staging buffers fit the LDS) */
extern "C" int exl2_wkv_scan_chunked_supported(int n_key, int n_val)
{
    return n_key > 0 && n_val > 0 && wkc_out_smem(n_key, n_val) <= 150 * 1024;
}

extern "C" int exl2_wkv_scan_chunked(const float* r, const float* k, const float* v, const float* g, int ld, const float* dlog, int ldd,
                                     const float* u, const float* norm_w, void* out, int ldo, int out_f32, float* state,
                                     const int* span_row0, const int* span_rows, const int* span_chunk0, int spans, int chunk,
                                     int total_chunks, const int* row_seq, const int* row_pos, float* zbuf, float* dbuf,
                                     int heads, int n_key, int n_val, float eps, void* stream)
{
    EXL2_REQUIRE(r && k && v && g && dlog && u && norm_w && out && state && span_row0 && span_rows && span_chunk0 && row_seq && row_pos
                 && zbuf && dbuf, "wkv_scan_chunked: null operand");
    EXL2_REQUIRE(chunk == WKC_L, "wkv_scan_chunked: chunks are %d rows", WKC_L);
    EXL2_REQUIRE(heads > 0 && exl2_wkv_scan_chunked_supported(n_key, n_val), "wkv_scan_chunked: state %d x %d does not fit", n_key, n_val);
    if (spans <= 0 || total_chunks <= 0) return EXL2_OK;
    WkvChunkArgs c;
    WkvArgs& a = c.a;
    a.r = r; a.k = k; a.v = v; a.g = g; a.ld = ld; a.dlog = dlog; a.ldd = ldd; a.u = u; a.norm_w = norm_w; a.out = out; a.ldo = ldo;
    a.state = state; a.span_row0 = span_row0; a.span_rows = span_rows; a.row_seq = row_seq; a.row_pos = row_pos;
    a.heads = heads; a.N = n_key; a.P = n_val; a.KS = 1; a.eps = eps;
    c.span_chunk0 = span_chunk0; c.spans = spans; c.zbuf = zbuf; c.dbuf = dbuf;
    static bool attr_done[EXL2_MAX_DEVICES];
    if (exl2_first_on_device(attr_done))
    {
        (void)hipFuncSetAttribute((const void*)wkv_chunk_state_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        (void)hipFuncSetAttribute((const void*)wkv_chunk_out_kernel<u16>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        (void)hipFuncSetAttribute((const void*)wkv_chunk_out_kernel<float>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    }
    const size_t sm1 = sizeof(float) * ((size_t)(2 * WKC_L + 1) * (n_key + 1) + (size_t)WKC_L * n_val);
    LAUNCH(wkv_chunk_state_kernel, dim3(total_chunks, heads), dim3(512), sm1, stream, c);
    LAUNCH(wkv_chunk_carry_kernel, dim3(spans, heads, (n_key * n_val + 255) / 256), dim3(256), 0, stream, c);
    if (out_f32) LAUNCH(wkv_chunk_out_kernel<float>, dim3(total_chunks, heads), dim3(1024), wkc_out_smem(n_key, n_val), stream, c);
    else LAUNCH(wkv_chunk_out_kernel<u16>, dim3(total_chunks, heads), dim3(1024), wkc_out_smem(n_key, n_val), stream, c);
    HIP_TRY(hipGetLastError());
    return EXL2_OK;
}
