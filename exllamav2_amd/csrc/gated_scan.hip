// gated_scan.hip -- two linear-attention recurrences over a matrix state per head, for gfx950, + their C ABI.
//
// Per head, with the state S (N key channels x P value channels, fp32, one per (slot, head)):
//   mode 0, "forget gate writes":   f = l + (1 - l) sigmoid(z_f)  per key channel (l = a learned lower bound),  q = silu(z_q),
//       S <- diag(f) S + (1 - f) v^T,    o = S^T q;
//   mode 1, "gated delta rule":     q, k made unit vectors per head (x / sqrt(sum x^2 + 1e-6)), q also times q_scale,
//       beta = sigmoid(z_b),  g = exp(-exp(A) softplus(z_a + a_bias))  (one number per head),
//       S <- g S,   u = beta (v - S^T k),   S <- S + k u^T,   o = S^T q        (the read-out sees the token's own write).
// The head's o is divided by its root mean square over P, multiplied by a weight per value channel (shared by the heads) and, in
// mode 1, by silu of an output gate, and leaves in the operand dtype for the output projection.  Query / key heads may be fewer than
// value heads (head h reads q / k head h / (heads / qk_heads)).  Inputs are the fp32 outputs of the mixer's projections (mode 1: of
// its short convolutions); gates, decays, unit norms and the state are fp32 throughout.
//
// Rows of a step are a flat list; a span is the run of consecutive rows one sequence brings (span i = rows span_row0[i] ..
// + span_rows[i], slot and first position = row_seq / row_pos of its first row).  A span at position 0 starts from zeros whatever
// its slot holds.
#include "hw.h"
#include "errors.h"
#include <stdint.h>

template <typename T> DEV void gs_st(T* p, float v);
template <> DEV void gs_st<u16>(u16* p, float v) { *p = f32_to_bf16(v); }
template <> DEV void gs_st<float>(float* p, float v) { *p = v; }

DEV float gs_sigmoid(float z) { return 1.0f / (1.0f + expf(-z)); }
DEV float gs_softplus(float z) { return z > 20.0f ? z : log1pf(expf(z)); }

#define GS_CHUNK 16                          // tokens staged in LDS at a time
#define GS_MAX_NPT 256                       // state rows per thread
#define GS_MAX_N 1024                        // key channels per head (16 per lane while a wave normalises a token's q and k)

enum { GS_FORGET_WRITES = 0, GS_DELTA = 1 };

struct GatedScanArgs
{
    const float* q; int ldq;                 // [rows, ldq]: q head g at g * N (mode 0: pre-activation)
    const float* k; int ldk;                 // mode 1: keys, head g at g * N;  mode 0: the forget gate's pre-activation, head h at h * N
    const float* v; int ldv;                 // head h at h * P
    const float* gate; int ldg;              // mode 1: output gate pre-activation, head h at h * P (nullable)
    const float* beta; int ldb;              // mode 1: [rows, ldb], head h at h (pre-sigmoid)
    const float* dt; int lddt;               // mode 1: [rows, lddt], head h at h
    const float* dt_bias; const float* a_log;        // mode 1: [heads]
    const float* lower;                      // mode 0: [heads * N]
    const float* norm_w;                     // [P]
    void* out; int ldo;                      // [rows, ldo] operand dtype (or fp32): head h at h * P
    float* state;                            // [slots, heads, N, P]
    const int* span_row0; const int* span_rows; const int* row_seq; const int* row_pos;
    int heads, qk_heads, N, P, KS;           // KS (a power of two <= 64) lanes share a column of the state
    float q_scale, eps;
};

// Workgroup = one (span, head): thread t = p * KS + j holds rows n = j, j + KS, .. of column p of the state in registers for the whole
// span; the KS lanes of a column are neighbours in one wave, so the two sums over key channels that a token needs (S^T k for the delta
// rule, S^T q for the read-out) close with lane exchanges, no barrier.  Tokens are taken GS_CHUNK at a time: a wave per token turns
// the raw projections into what the recurrence reads (gates, unit vectors, decay) and stages it in LDS, every thread steps its rows
// through the chunk, and a wave per token takes the head's root mean square and writes the normed (gated) row.
template <typename T, int NPT, int MODE>
KERNEL void __launch_bounds__(256) gated_scan_kernel(const GatedScanArgs a)
{
    DYN_SMEM(smem);
    const int h = bid_x(), sp = bid_y();
    const int n_tok = a.span_rows[sp], r0 = a.span_row0[sp];
    const int pos0 = a.row_pos[r0];
    const int P = a.P, N = a.N, KS = a.KS;
    const int t = tid(), nt = nthreads();
    const bool owner = t < P * KS;
    const int p = owner ? t / KS : 0, j = t % KS;
    const int hq = h / (a.heads / a.qk_heads);
    float* s_q = (float*)smem;                                   // [CHUNK, N]
    float* s_k = s_q + GS_CHUNK * N;                             // [CHUNK, N]  mode 1: unit keys; mode 0: forget gates
    float* s_v = s_k + GS_CHUNK * N;                             // [CHUNK, P]
    float* s_o = s_v + GS_CHUNK * P;                             // [CHUNK, P]
    float* s_b = s_o + GS_CHUNK * P;                             // [CHUNK] beta
    float* s_g = s_b + GS_CHUNK;                                 // [CHUNK] decay
    float* st = a.state + ((long long)a.row_seq[r0] * a.heads + h) * (long long)N * P;
    float S[NPT];
    #pragma unroll
    for (int i = 0; i < NPT; i++)
    {
        const int n = j + KS * i;
        S[i] = (owner && pos0 > 0 && n < N) ? st[(long long)n * P + p] : 0.0f;
    }
    for (int c0 = 0; c0 < n_tok; c0 += GS_CHUNK)
    {
        const int nc = min(GS_CHUNK, n_tok - c0);
        block_sync();
        for (int kk = wave_id(); kk < nc; kk += nt / 64)
        {
            const long long row = r0 + c0 + kk;
            if (MODE == GS_DELTA)
            {
                float qv[GS_MAX_N / 64], kv[GS_MAX_N / 64];
                float sq = 0.0f, sk = 0.0f;
                #pragma unroll
                for (int e = 0; e < GS_MAX_N / 64; e++)
                {
                    const int n = lane_id() + 64 * e;
                    qv[e] = n < N ? a.q[row * a.ldq + hq * N + n] : 0.0f;
                    kv[e] = n < N ? a.k[row * a.ldk + hq * N + n] : 0.0f;
                    sq = fmaf(qv[e], qv[e], sq);
                    sk = fmaf(kv[e], kv[e], sk);
                }
                sq = wave_allreduce_add(sq);
                sk = wave_allreduce_add(sk);
                const float mq = a.q_scale / sqrtf(sq + 1e-6f), mk = 1.0f / sqrtf(sk + 1e-6f);
                #pragma unroll
                for (int e = 0; e < GS_MAX_N / 64; e++)
                {
                    const int n = lane_id() + 64 * e;
                    if (n < N) { s_q[kk * N + n] = qv[e] * mq; s_k[kk * N + n] = kv[e] * mk; }
                }
                if (lane_id() == 0)
                {
                    s_b[kk] = gs_sigmoid(a.beta[row * a.ldb + h]);
                    s_g[kk] = expf(-expf(a.a_log[h]) * gs_softplus(a.dt[row * a.lddt + h] + a.dt_bias[h]));
                }
            }
            else
            {
                for (int n = lane_id(); n < N; n += 64)
                {
                    const float zq = a.q[row * a.ldq + h * N + n];
                    const float lo = a.lower[h * N + n];
                    s_q[kk * N + n] = zq * gs_sigmoid(zq);
                    s_k[kk * N + n] = fmaf(1.0f - lo, gs_sigmoid(a.k[row * a.ldk + h * N + n]), lo);
                }
            }
            for (int pp = lane_id(); pp < P; pp += 64) s_v[kk * P + pp] = a.v[row * a.ldv + h * P + pp];
        }
        block_sync();
        for (int kk = 0; kk < nc; kk++)
        {
            const float vv = s_v[kk * P + p];
            float o = 0.0f;
            if (MODE == GS_DELTA)
            {
                const float g = s_g[kk];
                float kt = 0.0f;
                #pragma unroll
                for (int i = 0; i < NPT; i++)
                {
                    const int n = j + KS * i;
                    if (n < N) { S[i] *= g; kt = fmaf(S[i], s_k[kk * N + n], kt); }
                }
                for (int m = 1; m < KS; m <<= 1) kt += shfl_xor_f32(kt, m);
                const float u = s_b[kk] * (vv - kt);
                #pragma unroll
                for (int i = 0; i < NPT; i++)
                {
                    const int n = j + KS * i;
                    if (n < N) { S[i] = fmaf(s_k[kk * N + n], u, S[i]); o = fmaf(S[i], s_q[kk * N + n], o); }
                }
            }
            else
            {
                #pragma unroll
                for (int i = 0; i < NPT; i++)
                {
                    const int n = j + KS * i;
                    if (n < N)
                    {
                        const float f = s_k[kk * N + n];
                        S[i] = fmaf(f, S[i], (1.0f - f) * vv);
                        o = fmaf(S[i], s_q[kk * N + n], o);
                    }
                }
            }
            for (int m = 1; m < KS; m <<= 1) o += shfl_xor_f32(o, m);
            if (owner && j == 0) s_o[kk * P + p] = o;
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
                float o = s_o[kk * P + pp] * rinv * a.norm_w[pp];
                if (a.gate) { const float gv = a.gate[row * a.ldg + h * P + pp]; o *= gv * gs_sigmoid(gv); }
                gs_st<T>((T*)a.out + row * a.ldo + h * P + pp, o);
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

// ---- the same recurrences for portions of prompts: columns of the state dealt to workgroups -------------------------------------------
// The value columns of a head's state never meet inside the recurrence (u_p = beta (v_p - S[:, p] . k), o_p = S[:, p] . q), so a
// span's walk is dealt to (head, block of GSC_COLS columns) workgroups: GSC_KS = 16 lanes share a column, each holds N / 16 rows in
// registers, and a token costs a thread a handful of fused multiply-adds and four lane exchanges per sum instead of a pass over
// N / 2 rows.  Tokens are taken GSC_CHUNK at a time; the raw projections of the NEXT batch of tokens are requested into registers before a batch
// is stepped through, so their latency hides behind it, and turned into gates / unit vectors / decays when they are written to LDS.
// The raw read-out goes to o_raw fp32 [rows, heads * P]; the head norm needs the whole head and is head_norm_gate_kernel's.

#define GSC_KS 16
#define GSC_COLS 16                          // 256 threads = 16 columns x 16 lanes
#define GSC_CHUNK 32
#define GSC_TPW (GSC_CHUNK / 4)              // tokens a wave stages at a time
#define GSC_MAX_N 256                        // key channels: 4 per lane while a wave stages a token, NPT = N / 16 <= 16 rows per thread

// rows of the state a thread holds: FULL (N == 16 * NPT, no row outside the state): NPT consecutive ones, so that a token's k and q
// come as 16-byte LDS reads; otherwise every 16th, guarded
#define GSC_ROW(i) (FULL ? j * NPT + (i) : j + GSC_KS * (i))

template <int NPT, int MODE, bool FULL>
KERNEL void __launch_bounds__(256) gated_scan_cols_kernel(const GatedScanArgs a, float* o_raw)
{
    DYN_SMEM(smem);
    const int h = bid_x(), sp = bid_y(), cb = bid_z();
    const int n_tok = a.span_rows[sp], r0 = a.span_row0[sp];
    const int pos0 = a.row_pos[r0];
    const int P = a.P, N = FULL ? GSC_KS * NPT : a.N;
    const int t = tid(), lane = lane_id(), wv = wave_id();
    const int pl = t / GSC_KS, j = t % GSC_KS;
    const int p = cb * GSC_COLS + pl;
    const bool owner = p < P;
    const int pc = owner ? p : P - 1;
    const int hq = h / (a.heads / a.qk_heads);
    float* s_q = (float*)smem;                                   // [CHUNK, N]
    float* s_k = s_q + GSC_CHUNK * N;                            // [CHUNK, N]
    float* s_v = s_k + GSC_CHUNK * N;                            // [CHUNK, COLS]
    float* s_b = s_v + GSC_CHUNK * GSC_COLS;                     // [CHUNK]
    float* s_g = s_b + GSC_CHUNK;                                // [CHUNK]
    float* st = a.state + ((long long)a.row_seq[r0] * a.heads + h) * (long long)N * P;
    float S[NPT];
    #pragma unroll
    for (int i = 0; i < NPT; i++)
    {
        const int n = GSC_ROW(i);
        S[i] = (owner && pos0 > 0 && n < N) ? st[(long long)n * P + p] : 0.0f;
    }
    const float a_neg = MODE == GS_DELTA ? -expf(a.a_log[h]) : 0.0f, dtb = MODE == GS_DELTA ? a.dt_bias[h] : 0.0f;
    // what a thread keeps of the next batch of tokens while the current one is stepped through
    float rq[GSC_TPW][GSC_MAX_N / 64], rk[GSC_TPW][GSC_MAX_N / 64], rv[2], rb = 0.0f, rd = 0.0f;
    const int qh = MODE == GS_DELTA ? hq : h;

    auto request = [&](int c0)
    {
        const int nc = min(GSC_CHUNK, n_tok - c0);
        #pragma unroll
        for (int u = 0; u < GSC_TPW; u++)
        {
            const int kk = wv + 4 * u;
            const long long row = r0 + c0 + min(kk, nc - 1);
            #pragma unroll
            for (int e = 0; e < GSC_MAX_N / 64; e++)
            {
                const int n = lane + 64 * e;
                rq[u][e] = n < N ? a.q[row * a.ldq + qh * N + n] : 0.0f;
                rk[u][e] = n < N ? a.k[row * a.ldk + qh * N + n] : 0.0f;
            }
        }
        #pragma unroll
        for (int u = 0; u < 2; u++)
        {
            const int kk = t / GSC_COLS + 16 * u, col = cb * GSC_COLS + t % GSC_COLS;
            rv[u] = (kk < nc && col < P) ? a.v[(long long)(r0 + c0 + kk) * a.ldv + h * P + col] : 0.0f;
        }
        if (MODE == GS_DELTA && t < GSC_CHUNK)
        {
            const long long row = r0 + c0 + min(t, nc - 1);
            rb = a.beta[row * a.ldb + h];
            rd = a.dt[row * a.lddt + h];
        }
    };

    auto publish = [&]()
    {
        // (the sums of squares of all the wave's tokens first, then their reductions side by side: sixteen independent exchanges
        // instead of a chain of them)
        float sq[GSC_TPW], sk[GSC_TPW];
        if (MODE == GS_DELTA)
        {
            #pragma unroll
            for (int u = 0; u < GSC_TPW; u++)
            {
                sq[u] = sk[u] = 0.0f;
                #pragma unroll
                for (int e = 0; e < GSC_MAX_N / 64; e++) { sq[u] = fmaf(rq[u][e], rq[u][e], sq[u]); sk[u] = fmaf(rk[u][e], rk[u][e], sk[u]); }
            }
            #pragma unroll
            for (int u = 0; u < GSC_TPW; u++) { sq[u] = wave_allreduce_add(sq[u]); sk[u] = wave_allreduce_add(sk[u]); }
        }
        #pragma unroll
        for (int u = 0; u < GSC_TPW; u++)
        {
            const int kk = wv + 4 * u;
            if (MODE == GS_DELTA)
            {
                const float mq = a.q_scale / sqrtf(sq[u] + 1e-6f), mk = 1.0f / sqrtf(sk[u] + 1e-6f);
                #pragma unroll
                for (int e = 0; e < GSC_MAX_N / 64; e++)
                {
                    const int n = lane + 64 * e;
                    if (n < N) { s_q[kk * N + n] = rq[u][e] * mq; s_k[kk * N + n] = rk[u][e] * mk; }
                }
            }
            else
            {
                #pragma unroll
                for (int e = 0; e < GSC_MAX_N / 64; e++)
                {
                    const int n = lane + 64 * e;
                    if (n < N)
                    {
                        const float lo = a.lower[h * N + n];
                        s_q[kk * N + n] = rq[u][e] * gs_sigmoid(rq[u][e]);
                        s_k[kk * N + n] = fmaf(1.0f - lo, gs_sigmoid(rk[u][e]), lo);
                    }
                }
            }
        }
        #pragma unroll
        for (int u = 0; u < 2; u++) s_v[(t / GSC_COLS + 16 * u) * GSC_COLS + t % GSC_COLS] = rv[u];
        if (MODE == GS_DELTA && t < GSC_CHUNK)
        {
            s_b[t] = gs_sigmoid(rb);
            s_g[t] = expf(a_neg * gs_softplus(rd + dtb));
        }
    };

    request(0);
    for (int c0 = 0; c0 < n_tok; c0 += GSC_CHUNK)
    {
        const int nc = min(GSC_CHUNK, n_tok - c0);
        block_sync_lds();                                        // the batch before has been stepped through by every thread
        publish();
        block_sync_lds();
        if (c0 + GSC_CHUNK < n_tok) request(c0 + GSC_CHUNK);
        float* orow = o_raw + (long long)(r0 + c0) * a.heads * P + h * P + p;
        // (four tokens unrolled: only the state's own update chains from token to token -- the sums that close a read-out and the
        // LDS reads of the tokens behind overlap with it; two partial sums halve each chain)
        #pragma unroll 4
        for (int kk = 0; kk < nc; kk++)
        {
            const float vv = s_v[kk * GSC_COLS + pl];
            float o = 0.0f;
            float kr[NPT], qr[NPT];                              // the token's k (or forget gate) and q at this thread's rows
            if (FULL)
            {
                #pragma unroll
                for (int c = 0; c < NPT / 4; c++)
                {
                    const f32x4 k4 = *(const f32x4*)(s_k + kk * N + j * NPT + 4 * c), q4 = *(const f32x4*)(s_q + kk * N + j * NPT + 4 * c);
                    #pragma unroll
                    for (int e = 0; e < 4; e++) { kr[4 * c + e] = k4[e]; qr[4 * c + e] = q4[e]; }
                }
            }
            else
            {
                #pragma unroll
                for (int i = 0; i < NPT; i++)
                {
                    const int n = GSC_ROW(i);
                    kr[i] = n < N ? s_k[kk * N + n] : 0.0f;
                    qr[i] = n < N ? s_q[kk * N + n] : 0.0f;
                }
            }
            if (MODE == GS_DELTA)
            {
                const float g = s_g[kk];
                float kt[2] = {0.0f, 0.0f}, o2 = 0.0f;
                #pragma unroll
                for (int i = 0; i < NPT; i++) { S[i] *= g; kt[i & 1] = fmaf(S[i], kr[i], kt[i & 1]); }
                const float u = s_b[kk] * (vv - row16_allreduce_add(kt[0] + kt[1]));
                #pragma unroll
                for (int i = 0; i < NPT; i++)
                {
                    S[i] = fmaf(kr[i], u, S[i]);
                    if (i & 1) o2 = fmaf(S[i], qr[i], o2); else o = fmaf(S[i], qr[i], o);
                }
                o += o2;
            }
            else
            {
                float o2 = 0.0f;
                #pragma unroll
                for (int i = 0; i < NPT; i++)
                {
                    S[i] = fmaf(kr[i], S[i] - vv, vv);           // f S + (1 - f) v (rows outside the state read f = q = 0 and are never stored)
                    if (i & 1) o2 = fmaf(S[i], qr[i], o2); else o = fmaf(S[i], qr[i], o);
                }
                o += o2;
            }
            o = row16_allreduce_add(o);
            if (owner && j == 0) orow[(long long)kk * a.heads * P] = o;
        }
    }
    #pragma unroll
    for (int i = 0; i < NPT; i++)
    {
        const int n = GSC_ROW(i);
        if (owner && n < N) st[(long long)n * P + p] = S[i];
    }
    (void)pc;
}

// grid (rows, heads), one wave: out = o / sqrt(mean(o^2) + eps) * norm_w (* silu(gate))
template <typename T>
KERNEL void __launch_bounds__(64) head_norm_gate_kernel(const float* o_raw, const float* norm_w, const float* gate, int ldg, void* out, int ldo,
                                                         int heads, int P, float eps)
{
    const long long row = bid_x();
    const int h = bid_y();
    const float* o = o_raw + row * heads * P + h * P;
    float ss = 0.0f;
    for (int pp = lane_id(); pp < P; pp += 64) ss = fmaf(o[pp], o[pp], ss);
    ss = wave_allreduce_add(ss);
    const float rinv = 1.0f / sqrtf(ss / (float)P + eps);
    for (int pp = lane_id(); pp < P; pp += 64)
    {
        float v = o[pp] * rinv * norm_w[pp];
        if (gate) { const float gv = gate[row * ldg + h * P + pp]; v *= gv * gs_sigmoid(gv); }
        gs_st<T>((T*)out + row * ldo + h * P + pp, v);
    }
}

template <typename T, int MODE>
static void gated_scan_launch(const GatedScanArgs& a, int npt, dim3 grid, dim3 block, size_t smem, void* stream)
{
    if (npt <= 16) LAUNCH((gated_scan_kernel<T, 16, MODE>), grid, block, smem, stream, a);
    else if (npt <= 64) LAUNCH((gated_scan_kernel<T, 64, MODE>), grid, block, smem, stream, a);
    else LAUNCH((gated_scan_kernel<T, GS_MAX_NPT, MODE>), grid, block, smem, stream, a);
}

/* The recurrence over the rows of every span, state read from and left in state[slot of the span][head].  mode 0: k is the forget
   gate's pre-activation (heads x n_key), lower its lower bound, qk_heads == heads; gate / beta / dt / dt_bias / a_log unused.
   mode 1: q / k hold qk_heads heads, beta / dt one value per head, gate nullable; lower unused.  All inputs fp32. */
extern "C" int exl2_gated_scan(int mode, const float* q, int ldq, const float* k, int ldk, const float* v, int ldv, const float* gate,
                               int ldg, const float* beta, int ldb, const float* dt, int lddt, const float* dt_bias, const float* a_log,
                               const float* lower, const float* norm_w, void* out, int ldo, int out_f32, float* state,
                               const int* span_row0, const int* span_rows, int spans, const int* row_seq, const int* row_pos, int heads,
                               int qk_heads, int n_key, int n_val, float q_scale, float eps, void* stream)
{
    EXL2_REQUIRE(mode == GS_FORGET_WRITES || mode == GS_DELTA, "gated_scan: mode must be 0 (forget gate writes) or 1 (delta rule)");
    EXL2_REQUIRE(q && k && v && norm_w && out && state && span_row0 && span_rows && row_seq && row_pos, "gated_scan: null operand");
    EXL2_REQUIRE(mode != GS_FORGET_WRITES || lower, "gated_scan: the forget gate needs its lower bound");
    EXL2_REQUIRE(mode != GS_DELTA || (beta && dt && dt_bias && a_log), "gated_scan: the delta rule needs beta and the decay's inputs");
    EXL2_REQUIRE(heads > 0 && qk_heads > 0 && heads % qk_heads == 0 && (mode == GS_DELTA || qk_heads == heads), "gated_scan: %d heads over %d query / key heads", heads, qk_heads);
    EXL2_REQUIRE(n_key > 0 && n_key <= GS_MAX_N && n_val > 0 && n_val <= 256, "gated_scan: state %d x %d", n_key, n_val);
    if (spans <= 0) return EXL2_OK;
    int ks = 1;
    while (ks * 2 <= 64 && n_val * ks * 2 <= 256 && ks * 2 <= n_key) ks *= 2;
    const int npt = (n_key + ks - 1) / ks;
    EXL2_REQUIRE(npt <= GS_MAX_NPT, "gated_scan: state %d x %d needs %d rows per thread (at most %d)", n_key, n_val, npt, GS_MAX_NPT);
    GatedScanArgs a;
    a.q = q; a.ldq = ldq; a.k = k; a.ldk = ldk; a.v = v; a.ldv = ldv; a.gate = gate; a.ldg = ldg; a.beta = beta; a.ldb = ldb; a.dt = dt;
    a.lddt = lddt; a.dt_bias = dt_bias; a.a_log = a_log; a.lower = lower; a.norm_w = norm_w; a.out = out; a.ldo = ldo; a.state = state;
    a.span_row0 = span_row0; a.span_rows = span_rows; a.row_seq = row_seq; a.row_pos = row_pos;
    a.heads = heads; a.qk_heads = qk_heads; a.N = n_key; a.P = n_val; a.KS = ks; a.q_scale = q_scale; a.eps = eps;
    const size_t smem = sizeof(float) * ((size_t)GS_CHUNK * (2 * n_key + 2 * n_val + 2));
    if (smem > 48 * 1024)
    {
        static bool attr_done[EXL2_MAX_DEVICES];
        if (exl2_first_on_device(attr_done))
        {
            (void)hipFuncSetAttribute((const void*)gated_scan_kernel<u16, GS_MAX_NPT, GS_FORGET_WRITES>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
            (void)hipFuncSetAttribute((const void*)gated_scan_kernel<float, GS_MAX_NPT, GS_FORGET_WRITES>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
            (void)hipFuncSetAttribute((const void*)gated_scan_kernel<u16, GS_MAX_NPT, GS_DELTA>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
            (void)hipFuncSetAttribute((const void*)gated_scan_kernel<float, GS_MAX_NPT, GS_DELTA>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
            (void)hipFuncSetAttribute((const void*)gated_scan_kernel<u16, 64, GS_FORGET_WRITES>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
            (void)hipFuncSetAttribute((const void*)gated_scan_kernel<float, 64, GS_FORGET_WRITES>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
            (void)hipFuncSetAttribute((const void*)gated_scan_kernel<u16, 64, GS_DELTA>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
            (void)hipFuncSetAttribute((const void*)gated_scan_kernel<float, 64, GS_DELTA>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        }
    }
    const dim3 grid(heads, spans), block((n_val * ks + 63) / 64 * 64);
    if (mode == GS_DELTA)
    {
        if (out_f32) gated_scan_launch<float, GS_DELTA>(a, npt, grid, block, smem, stream);
        else gated_scan_launch<u16, GS_DELTA>(a, npt, grid, block, smem, stream);
    }
    else
    {
        if (out_f32) gated_scan_launch<float, GS_FORGET_WRITES>(a, npt, grid, block, smem, stream);
        else gated_scan_launch<u16, GS_FORGET_WRITES>(a, npt, grid, block, smem, stream);
    }
    HIP_TRY(hipGetLastError());
    return EXL2_OK;
}

/* 1 if exl2_gated_scan_cols takes this state shape */
extern "C" int exl2_gated_scan_cols_supported(int n_key, int n_val)
{
    return n_key > 0 && n_key <= GSC_MAX_N && n_val > 0 ? 1 : 0;
}

/* exl2_gated_scan for portions of prompts: a span's walk dealt to (head, 16 value columns) workgroups, the next tokens' inputs in
   flight behind the current one; the head norm (and gate) as a second launch over o_raw (scratch, fp32 [rows, heads * n_val]).  Same
   operands and results as exl2_gated_scan (sums associate differently: results agree to rounding). */
extern "C" int exl2_gated_scan_cols(int mode, const float* q, int ldq, const float* k, int ldk, const float* v, int ldv, const float* gate,
                                    int ldg, const float* beta, int ldb, const float* dt, int lddt, const float* dt_bias,
                                    const float* a_log, const float* lower, const float* norm_w, void* out, int ldo, int out_f32,
                                    float* state, const int* span_row0, const int* span_rows, int spans, const int* row_seq,
                                    const int* row_pos, int rows, float* o_raw, int heads, int qk_heads, int n_key, int n_val,
                                    float q_scale, float eps, void* stream)
{
    EXL2_REQUIRE(mode == GS_FORGET_WRITES || mode == GS_DELTA, "gated_scan_cols: mode must be 0 (forget gate writes) or 1 (delta rule)");
    EXL2_REQUIRE(q && k && v && norm_w && out && state && o_raw && span_row0 && span_rows && row_seq && row_pos, "gated_scan_cols: null operand");
    EXL2_REQUIRE(mode != GS_FORGET_WRITES || lower, "gated_scan_cols: the forget gate needs its lower bound");
    EXL2_REQUIRE(mode != GS_DELTA || (beta && dt && dt_bias && a_log), "gated_scan_cols: the delta rule needs beta and the decay's inputs");
    EXL2_REQUIRE(heads > 0 && qk_heads > 0 && heads % qk_heads == 0 && (mode == GS_DELTA || qk_heads == heads), "gated_scan_cols: %d heads over %d query / key heads", heads, qk_heads);
    EXL2_REQUIRE(exl2_gated_scan_cols_supported(n_key, n_val), "gated_scan_cols: state %d x %d", n_key, n_val);
    if (spans <= 0 || rows <= 0) return EXL2_OK;
    GatedScanArgs a;
    a.q = q; a.ldq = ldq; a.k = k; a.ldk = ldk; a.v = v; a.ldv = ldv; a.gate = gate; a.ldg = ldg; a.beta = beta; a.ldb = ldb; a.dt = dt;
    a.lddt = lddt; a.dt_bias = dt_bias; a.a_log = a_log; a.lower = lower; a.norm_w = norm_w; a.out = out; a.ldo = ldo; a.state = state;
    a.span_row0 = span_row0; a.span_rows = span_rows; a.row_seq = row_seq; a.row_pos = row_pos;
    a.heads = heads; a.qk_heads = qk_heads; a.N = n_key; a.P = n_val; a.KS = GSC_KS; a.q_scale = q_scale; a.eps = eps;
    const size_t smem = sizeof(float) * ((size_t)GSC_CHUNK * (2 * n_key + GSC_COLS + 2));
    if (smem > 48 * 1024)
    {
        static bool attr_done[EXL2_MAX_DEVICES];
        if (exl2_first_on_device(attr_done))
        {
            (void)hipFuncSetAttribute((const void*)gated_scan_cols_kernel<16, GS_FORGET_WRITES, false>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
            (void)hipFuncSetAttribute((const void*)gated_scan_cols_kernel<16, GS_DELTA, false>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
            (void)hipFuncSetAttribute((const void*)gated_scan_cols_kernel<16, GS_FORGET_WRITES, true>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
            (void)hipFuncSetAttribute((const void*)gated_scan_cols_kernel<16, GS_DELTA, true>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        }
    }
    const dim3 grid(heads, spans, (n_val + GSC_COLS - 1) / GSC_COLS);
    const int npt = (n_key + GSC_KS - 1) / GSC_KS;
    const bool full = n_key == GSC_KS * 4 || n_key == GSC_KS * 8 || n_key == GSC_KS * 16;
#define GSC_LAUNCH(NPT_, MODE_) do { if (full) LAUNCH((gated_scan_cols_kernel<NPT_, MODE_, true>), grid, dim3(256), smem, stream, a, o_raw); \
                                     else LAUNCH((gated_scan_cols_kernel<NPT_, MODE_, false>), grid, dim3(256), smem, stream, a, o_raw); } while (0)
    if (mode == GS_DELTA)
    {
        if (npt <= 4) GSC_LAUNCH(4, GS_DELTA); else if (npt <= 8) GSC_LAUNCH(8, GS_DELTA); else GSC_LAUNCH(16, GS_DELTA);
    }
    else
    {
        if (npt <= 4) GSC_LAUNCH(4, GS_FORGET_WRITES); else if (npt <= 8) GSC_LAUNCH(8, GS_FORGET_WRITES); else GSC_LAUNCH(16, GS_FORGET_WRITES);
    }
#undef GSC_LAUNCH
    const float* gt = mode == GS_DELTA ? gate : nullptr;
    if (out_f32) LAUNCH(head_norm_gate_kernel<float>, dim3(rows, heads), dim3(64), 0, stream, (const float*)o_raw, norm_w, gt, ldg, out, ldo, heads, n_val, eps);
    else LAUNCH(head_norm_gate_kernel<u16>, dim3(rows, heads), dim3(64), 0, stream, (const float*)o_raw, norm_w, gt, ldg, out, ldo, heads, n_val, eps);
    HIP_TRY(hipGetLastError());
    return EXL2_OK;
}
