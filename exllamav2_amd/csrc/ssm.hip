// ssm.hip -- the recurrent half of a state-space mixer (selective scan with one scalar decay per head) for gfx950, + its C ABI:
//   * the short causal convolution per channel with its bias and SiLU, over rows that continue a sequence (the last taps - 1
//     inputs of every sequence are kept per slot),
//   * the scan  S <- exp(-exp(A) dt) S + dt B u^T,  y = S^T C + D u  per head over the rows of each sequence's portion, with
//     dt = softplus(dt_raw + dt_bias); the state S [state, vdim] is fp32 and lives per (slot, head),
//   * the gate and the group-wise RMS norm  out = rms_g(y * silu(z)) * w.
// Rows of a step are a flat list; a SPAN is the run of consecutive rows that one sequence brings (span i = rows span_row0[i] ..
// + span_rows[i], its slot and first position are row_seq / row_pos of its first row).  A span that starts at position 0 starts
// from a zero state and zero convolution history whatever its slot held before, so slots need no clearing when they are reused.
// All arithmetic is fp32; inputs are the fp32 outputs of the mixer's input projection.
#include "hw.h"
#include "errors.h"
#include <stdint.h>

template <typename T> DEV float ss_ld(const T* p);
template <> DEV float ss_ld<u16>(const u16* p) { return bf16_to_f32(*p); }
template <> DEV float ss_ld<float>(const float* p) { return *p; }
template <typename T> DEV void ss_st(T* p, float v);
template <> DEV void ss_st<u16>(u16* p, float v) { *p = f32_to_bf16(v); }
template <> DEV void ss_st<float>(float* p, float v) { *p = v; }

DEV float ss_silu(float z) { return z / (1.0f + expf(-z)); }
DEV float ss_softplus(float z) { return z > 20.0f ? z : log1pf(expf(z)); }

// ---- causal convolution + SiLU ------------------------------------------------------------------------------------------------

#define CONV_MAX_TAPS 16
#define CONV_TOKENS 32                       // consecutive rows of a span that one workgroup walks

struct ConvArgs
{
    const float* in; int ld;                 // [rows, ld]: the channels start at the pointer
    const void* w; const void* bias;         // [channels, taps], [channels]
    void* out; int ldo;                      // [rows, ldo] fp32, or the operand dtype (out_f32 == 0)
    int out_f32;
    int residual;                            // 0: out = silu(conv + bias);  1: out = in + conv + bias (no activation)
    float* tail;                             // [slots, taps - 1, channels]: inputs of the last taps - 1 positions of every sequence
    const int* span_row0; const int* span_rows; const int* row_seq; const int* row_pos;
    int channels, taps;
    int roll_tail;                           // every span is one walk: the convolution kernel rolls the tails itself
};

// grid (channel blocks, token chunks, spans): thread = one channel over CONV_TOKENS consecutive rows of a span; the window of the
// last taps inputs slides through registers (MAXT of them: the smallest of 4 / 8 / 16 that holds the taps) and all of the walk's
// inputs are requested before the first is used.  Inputs in front of the span come from the slot's tail, inputs in front of the
// sequence are zero.  (Four channels per thread with 16-byte accesses measured slower: 120 against 74 us at 2048 x 4352.)
template <typename T, int MAXT>
KERNEL void __launch_bounds__(256) conv_silu_kernel(const ConvArgs a)
{
    const int c = bid_x() * 256 + tid();
    const int sp = bid_z();
    const int n = a.span_rows[sp];
    const int t0 = bid_y() * CONV_TOKENS;
    if (c >= a.channels || t0 >= n) return;
    const int r0 = a.span_row0[sp];
    const int pos0 = a.row_pos[r0];
    const float* tail = a.tail + (long long)a.row_seq[r0] * (a.taps - 1) * a.channels;
    const int t1 = min(n, t0 + CONV_TOKENS);
    float xin[CONV_TOKENS];
    #pragma unroll
    for (int i = 0; i < CONV_TOKENS; i++) xin[i] = t0 + i < t1 ? a.in[(long long)(r0 + t0 + i) * a.ld + c] : 0.0f;
    float w[MAXT], win[MAXT];
    #pragma unroll
    for (int k = 0; k < MAXT; k++) w[k] = k < a.taps ? ss_ld<T>((const T*)a.w + (long long)c * a.taps + k) : 0.0f;
    const float bias = a.bias ? ss_ld<T>((const T*)a.bias + c) : 0.0f;
    // win[k] = input at token t - (taps - 1) + k; before the first shift slot k holds token t0 - (taps - 1) + (k - 1); tokens are
    // counted within the span, token -d is position pos0 - d
    #pragma unroll
    for (int k = 0; k < MAXT; k++)
    {
        win[k] = 0.0f;
        if (k >= 1 && k < a.taps)
        {
            const int tok = t0 - (a.taps - 1) + (k - 1);
            if (tok >= 0) win[k] = a.in[(long long)(r0 + tok) * a.ld + c];
            else if (pos0 + tok >= 0) win[k] = tail[(long long)(a.taps - 1 + tok) * a.channels + c];
        }
    }
    #pragma unroll
    for (int i = 0; i < CONV_TOKENS; i++)
    {
        if (t0 + i >= t1) break;
        #pragma unroll
        for (int k = 0; k < MAXT - 1; k++) win[k] = win[k + 1];
        float acc = bias;
        #pragma unroll
        for (int k = 0; k < MAXT; k++)
        {
            if (k == a.taps - 1) win[k] = xin[i];                // after the shift the newest value belongs at index taps - 1
            if (k < a.taps) acc = fmaf(w[k], win[k], acc);
        }
        const float o = a.residual ? xin[i] + acc : ss_silu(acc);
        if (a.out_f32) ((float*)a.out)[(long long)(r0 + t0 + i) * a.ldo + c] = o;
        else ss_st<T>((T*)a.out + (long long)(r0 + t0 + i) * a.ldo + c, o);
    }
    if (a.roll_tail && a.taps > 1)
    {
        // the span is this one walk, so this thread alone reads and writes channel c of the slot's tail: the inputs of the
        // sequence's last taps - 1 positions (rows of the span where it is long enough, the old tail shifted where it is not)
        float* tl = a.tail + (long long)a.row_seq[r0] * (a.taps - 1) * a.channels;
        float nv[MAXT];
        #pragma unroll
        for (int k = 0; k < MAXT - 1; k++)
        {
            nv[k] = 0.0f;
            if (k < a.taps - 1)
            {
                const int tok = n - (a.taps - 1) + k;
                if (tok >= 0) nv[k] = a.in[(long long)(r0 + tok) * a.ld + c];
                else if (pos0 + tok >= 0) nv[k] = tl[(long long)(a.taps - 1 + tok) * a.channels + c];
            }
        }
        #pragma unroll
        for (int k = 0; k < MAXT - 1; k++)
            if (k < a.taps - 1) tl[(long long)k * a.channels + c] = nv[k];
    }
}

// The tails after a step with spans of several walks (the first walk reads the old tail while the last would write the new one, so
// the roll is a launch of its own there): for every span the inputs of its last taps - 1 positions (rows of the span where it is long enough,
// the old tail shifted where it is not).  One thread per (span, channel) reads all it needs before it writes.
KERNEL void __launch_bounds__(256) conv_tail_kernel(const ConvArgs a)
{
    const int c = bid_x() * 256 + tid();
    const int sp = bid_y();
    if (c >= a.channels) return;
    const int n = a.span_rows[sp], r0 = a.span_row0[sp];
    const int pos0 = a.row_pos[r0];
    float* tail = a.tail + (long long)a.row_seq[r0] * (a.taps - 1) * a.channels;
    float nv[CONV_MAX_TAPS];
    #pragma unroll
    for (int k = 0; k < CONV_MAX_TAPS - 1; k++)
    {
        nv[k] = 0.0f;
        if (k < a.taps - 1)
        {
            const int tok = n - (a.taps - 1) + k;                   // token of the span that lands in tail slot k
            if (tok >= 0) nv[k] = a.in[(long long)(r0 + tok) * a.ld + c];
            else if (pos0 + tok >= 0) nv[k] = tail[(long long)(a.taps - 1 + tok) * a.channels + c];
        }
    }
    #pragma unroll
    for (int k = 0; k < CONV_MAX_TAPS - 1; k++)
        if (k < a.taps - 1) tail[(long long)k * a.channels + c] = nv[k];
}

// ---- selective scan -------------------------------------------------------------------------------------------------------------

#define SCAN_CHUNK 16                        // tokens staged in LDS per round
#define SCAN_MAX_NPT 128                     // state rows per thread

struct ScanArgs
{
    const float* u; int ldu;                 // [rows, ldu]: head h's inputs at h * vdim
    const float* B; const float* C; int ldbc; // [rows, ldbc]: group g's vectors at g * state
    const float* dt; int lddt;               // [rows, lddt]: raw step sizes, head h at h
    const float* dt_bias; const float* A_log; const float* D;       // [heads]
    float* y; int ldy;                       // [rows, ldy]
    float* state;                            // [slots, heads, state, vdim]
    const int* span_row0; const int* span_rows; const int* row_seq; const int* row_pos;
    int heads, groups, N, P, KS;             // KS = threads that share a column of the state (blockDim = P * KS)
};

// Workgroup = one (span, head), P * KS threads (+ idle ones up to a whole wave): thread (j, p) holds rows n = j, j + KS, .. of column p of the state in registers
// for the whole span.  Tokens are taken SCAN_CHUNK at a time: their u, B, C, step size and decay are staged in LDS, every thread
// steps its rows through the chunk keeping one partial dot product per token, and the partial sums of a column's KS threads
// are added at the chunk's end (two barriers per chunk, none per token).
template <int NPT>
KERNEL void __launch_bounds__(256) scan_kernel(const ScanArgs a)
{
    DYN_SMEM(smem);
    const int h = bid_x(), sp = bid_y();
    const int n_tok = a.span_rows[sp], r0 = a.span_row0[sp];
    const int pos0 = a.row_pos[r0];
    const int g = h / (a.heads / a.groups);
    const int P = a.P, N = a.N, KS = a.KS;
    const int t = tid(), nt = nthreads();                      // P * KS rounded up to whole waves: the rest only help staging
    const bool owner = t < P * KS;
    const int p = t % P, j = t / P;
    float* s_u = (float*)smem;                                   // [CHUNK, P]
    float* s_B = s_u + SCAN_CHUNK * P;                           // [CHUNK, N]
    float* s_C = s_B + SCAN_CHUNK * N;                           // [CHUNK, N]
    float* s_dt = s_C + SCAN_CHUNK * N;                          // [CHUNK] step size, [CHUNK] decay
    float* s_part = s_dt + 2 * SCAN_CHUNK;                       // [CHUNK, KS, P]
    float* st = a.state + ((long long)a.row_seq[r0] * a.heads + h) * (long long)N * P;
    float S[NPT];
    #pragma unroll
    for (int i = 0; i < NPT; i++)
    {
        const int n = j + KS * i;
        S[i] = (owner && pos0 > 0 && n < N) ? st[(long long)n * P + p] : 0.0f;
    }
    const float neg_a = -expf(a.A_log[h]), dtb = a.dt_bias[h], Dh = a.D[h];
    for (int c0 = 0; c0 < n_tok; c0 += SCAN_CHUNK)
    {
        const int nc = min(SCAN_CHUNK, n_tok - c0);
        block_sync();
        for (int i = t; i < nc * P; i += nt) s_u[i] = a.u[(long long)(r0 + c0 + i / P) * a.ldu + h * P + i % P];
        for (int i = t; i < nc * N; i += nt)
        {
            const long long row = r0 + c0 + i / N;
            s_B[i] = a.B[row * a.ldbc + g * N + i % N];
            s_C[i] = a.C[row * a.ldbc + g * N + i % N];
        }
        if (t < nc)
        {
            const float d = ss_softplus(a.dt[(long long)(r0 + c0 + t) * a.lddt + h] + dtb);
            s_dt[t] = d;
            s_dt[SCAN_CHUNK + t] = expf(neg_a * d);
        }
        block_sync();
        for (int k = 0; owner && k < nc; k++)
        {
            const float d = s_dt[k], decay = s_dt[SCAN_CHUNK + k];
            const float du = d * s_u[k * P + p];
            float part = 0.0f;
            #pragma unroll
            for (int i = 0; i < NPT; i++)
            {
                const int n = j + KS * i;
                if (n < N)
                {
                    S[i] = fmaf(decay, S[i], du * s_B[k * N + n]);
                    part = fmaf(S[i], s_C[k * N + n], part);
                }
            }
            s_part[(k * KS + j) * P + p] = part;
        }
        block_sync();
        for (int i = t; i < nc * P; i += nt)
        {
            const int k = i / P, pp = i % P;
            float yv = 0.0f;
            for (int jj = 0; jj < KS; jj++) yv += s_part[(k * KS + jj) * P + pp];
            a.y[(long long)(r0 + c0 + k) * a.ldy + h * P + pp] = fmaf(Dh, s_u[k * P + pp], yv);
        }
    }
    #pragma unroll
    for (int i = 0; i < NPT; i++)
    {
        const int n = j + KS * i;
        if (owner && n < N) st[(long long)n * P + p] = S[i];
    }
}

// ---- the same scan in chunks (portions of prompts) ----------------------------------------------------------------------------------
// Inside a chunk of SSD_L tokens the recurrence unrolls into small matrix products (all fp32 FMA, 4 x 4 register tiles over LDS):
// with l_t = the log decay of token t, c_t = l_1 + .. + l_t, x_t = d_t u_t,
//     y_t = exp(c_t) S_in^T C_t + sum_{s <= t} exp(c_t - c_s) (C_t . B_s) x_s + D u_t,      S_out = exp(c_L) S_in + sum_s exp(c_L - c_s) B_s x_s^T.
// Three launches make every (chunk, head) of a step independent work: (1) each chunk's own contribution Z to S_out and its total
// decay, (2) the carry over a span's chunks, one thread per state element (Z is replaced by the state ENTERING the chunk, the slot
// takes the state after the last), (3) each chunk's outputs.  Every exponent is <= 0.

#define SSD_L 64

struct SsdArgs
{
    ScanArgs s;
    float* zbuf;                             // [chunks of the step, heads, N, P]
    float* dbuf;                             // [chunks of the step, heads]: exp(c_L)
    const int* span_chunk0;                  // first chunk of every span
    int nh;                                  // rows of the state the output kernel stages at a time (divides N, a multiple of 4)
};

// step sizes, log decays and their running sum for the chunk's tokens (rows past the chunk's end: zeros); thread t < SSD_L = token t
DEV void ssd_stage_decay(const ScanArgs& a, int h, long long row0, int lc, float* s_dt, float* s_cum)
{
    const int t = tid();
    if (t < SSD_L)
    {
        float d = 0.0f;
        if (t < lc) d = ss_softplus(a.dt[(row0 + t) * a.lddt + h] + a.dt_bias[h]);
        s_dt[t] = d;
        s_cum[t] = -expf(a.A_log[h]) * d;
    }
    block_sync();
    if (t == 0)
    {
        float c = 0.0f;
        for (int i = 0; i < SSD_L; i++) { c += s_cum[i]; s_cum[i] = c; }
    }
    block_sync();
}

KERNEL void __launch_bounds__(256) ssd_chunk_state_kernel(const SsdArgs g)
{
    DYN_SMEM(smem);
    const ScanArgs& a = g.s;
    const int c = bid_x(), h = bid_y(), sp = bid_z();
    const int n_tok = a.span_rows[sp];
    if (c * SSD_L >= n_tok) return;
    const long long row0 = a.span_row0[sp] + c * SSD_L;
    const int lc = min(SSD_L, n_tok - c * SSD_L);
    const int N = a.N, P = a.P, grp = h / (a.heads / a.groups), t = tid();
    float* s_dt = (float*)smem;                                  // [L]
    float* s_cum = s_dt + SSD_L;                                 // [L]
    float* s_B = s_cum + SSD_L;                                  // [L][N]: B_s exp(c_L - c_s)
    float* s_X = s_B + SSD_L * N;                                // [L][P]: d_s u_s
    ssd_stage_decay(a, h, row0, lc, s_dt, s_cum);
    const float c_end = s_cum[SSD_L - 1];
    // (16-byte loads, four in flight per thread: the staging loops are latency-bound otherwise)
    const f32x4 zero4 = {0.0f, 0.0f, 0.0f, 0.0f};
    #pragma unroll 4
    for (int i = t; i < SSD_L * N / 4; i += 256)
    {
        const int tok = i / (N / 4), n = (i % (N / 4)) * 4;
        const f32x4 b = tok < lc ? *(const f32x4*)(a.B + (row0 + tok) * a.ldbc + grp * N + n) : zero4;
        const float w = expf(c_end - s_cum[tok]);
        *(f32x4*)(s_B + tok * N + n) = (f32x4){b[0] * w, b[1] * w, b[2] * w, b[3] * w};
    }
    #pragma unroll 4
    for (int i = t; i < SSD_L * P / 4; i += 256)
    {
        const int tok = i / (P / 4), p = (i % (P / 4)) * 4;
        const f32x4 x = tok < lc ? *(const f32x4*)(a.u + (row0 + tok) * a.ldu + h * P + p) : zero4;
        const float d = s_dt[tok];
        *(f32x4*)(s_X + tok * P + p) = (f32x4){x[0] * d, x[1] * d, x[2] * d, x[3] * d};
    }
    block_sync();
    float* z = g.zbuf + ((long long)(g.span_chunk0[sp] + c) * a.heads + h) * (long long)N * P;
    const int tp = P / 4, tiles = (N / 4) * tp;
    for (int tile = t; tile < tiles; tile += 256)
    {
        const int n0 = (tile / tp) * 4, p0 = (tile % tp) * 4;
        float acc[4][4] = {};
        for (int k = 0; k < SSD_L; k++)
        {
            const f32x4 b = *(const f32x4*)(s_B + k * N + n0), x = *(const f32x4*)(s_X + k * P + p0);
            #pragma unroll
            for (int i = 0; i < 4; i++)
                #pragma unroll
                for (int j = 0; j < 4; j++) acc[i][j] = fmaf(b[i], x[j], acc[i][j]);
        }
        #pragma unroll
        for (int i = 0; i < 4; i++) *(f32x4*)(z + (long long)(n0 + i) * P + p0) = (f32x4){acc[i][0], acc[i][1], acc[i][2], acc[i][3]};
    }
    if (t == 0) g.dbuf[(long long)(g.span_chunk0[sp] + c) * a.heads + h] = expf(c_end);
}

// grid (ceil(N P / 256), heads, spans)
KERNEL void __launch_bounds__(256) ssd_carry_kernel(const SsdArgs g)
{
    const ScanArgs& a = g.s;
    const int e = bid_x() * 256 + tid(), h = bid_y(), sp = bid_z();
    const long long NP = (long long)a.N * a.P;
    if (e >= NP) return;
    const int r0 = a.span_row0[sp];
    const int chunks = (a.span_rows[sp] + SSD_L - 1) / SSD_L;
    float* st = a.state + ((long long)a.row_seq[r0] * a.heads + h) * NP + e;
    float S = a.row_pos[r0] > 0 ? *st : 0.0f;
    const long long c0 = g.span_chunk0[sp];
    int c = 0;
    for (; c + 4 <= chunks; c += 4)                              // the loads of four chunks leave together, the chain follows
    {
        float zv[4], dv[4];
        #pragma unroll
        for (int i = 0; i < 4; i++)
        {
            zv[i] = g.zbuf[((c0 + c + i) * a.heads + h) * NP + e];
            dv[i] = g.dbuf[(c0 + c + i) * a.heads + h];
        }
        #pragma unroll
        for (int i = 0; i < 4; i++)
        {
            g.zbuf[((c0 + c + i) * a.heads + h) * NP + e] = S;
            S = fmaf(dv[i], S, zv[i]);
        }
    }
    for (; c < chunks; c++)
    {
        const float zv = g.zbuf[((c0 + c) * a.heads + h) * NP + e], dv = g.dbuf[(c0 + c) * a.heads + h];
        g.zbuf[((c0 + c) * a.heads + h) * NP + e] = S;
        S = fmaf(dv, S, zv);
    }
    *st = S;
}

// The state dimension goes by in slices of g.nh rows so that the staged images stay small enough for two workgroups per CU: per
// slice the C and B columns are staged, M accumulates C . B, then the slice of the entering state takes B's place and the
// inter-chunk product accumulates C . S.  M's 4 x 4 register tile is rows ra + 16 i x columns cb + 16 j (lanes walk consecutive
// rows: conflict-free 16-byte LDS reads; the pairs j > i lie above the diagonal and are skipped); y tiles are 4 tokens x 4 values.
#define SSD_YT 2                             // y tiles per thread: vdim <= 128

KERNEL void __launch_bounds__(256, 2) ssd_chunk_out_kernel(const SsdArgs g)
{
    DYN_SMEM(smem);
    const ScanArgs& a = g.s;
    const int c = bid_x(), h = bid_y(), sp = bid_z();
    const int n_tok = a.span_rows[sp];
    if (c * SSD_L >= n_tok) return;
    const long long row0 = a.span_row0[sp] + c * SSD_L;
    const int lc = min(SSD_L, n_tok - c * SSD_L);
    const int N = a.N, P = a.P, nh = g.nh, grp = h / (a.heads / a.groups), t = tid();
    const int NS = nh + 4, MS = SSD_L + 4;
    float* s_dt = (float*)smem;                                  // [L]
    float* s_cum = s_dt + SSD_L;                                 // [L]
    float* s_C = s_cum + SSD_L;                                  // [L][NS]
    float* s_BS = s_C + SSD_L * NS;                              // [L][NS] B, then [nh][P] the slice of the state entering the chunk
    float* s_X = s_BS + max(SSD_L * NS, nh * P);                 // [L][P]
    float* s_M = s_X + SSD_L * P;                                // [L][MS]
    ssd_stage_decay(a, h, row0, lc, s_dt, s_cum);
    const f32x4 zero4 = {0.0f, 0.0f, 0.0f, 0.0f};
    #pragma unroll 4
    for (int i = t; i < SSD_L * P / 4; i += 256)
    {
        const int tok = i / (P / 4), p = (i % (P / 4)) * 4;
        const f32x4 x = tok < lc ? *(const f32x4*)(a.u + (row0 + tok) * a.ldu + h * P + p) : zero4;
        const float d = s_dt[tok];
        *(f32x4*)(s_X + tok * P + p) = (f32x4){x[0] * d, x[1] * d, x[2] * d, x[3] * d};
    }
    const int ra = t / 16, cb = t % 16;
    const int tp = P / 4, tiles = (SSD_L / 4) * tp;
    const float* zin = g.zbuf + ((long long)(g.span_chunk0[sp] + c) * a.heads + h) * (long long)N * P;
    float macc[4][4] = {};
    float inter[SSD_YT][4][4] = {};
    for (int n0 = 0; n0 < N; n0 += nh)
    {
        block_sync();                                            // the previous slice's readers are done
        #pragma unroll 4
        for (int i = t; i < SSD_L * nh / 4; i += 256)
        {
            const int tok = i / (nh / 4), n = (i % (nh / 4)) * 4;
            const bool live = tok < lc;
            *(f32x4*)(s_C + tok * NS + n) = live ? *(const f32x4*)(a.C + (row0 + tok) * a.ldbc + grp * N + n0 + n) : zero4;
            *(f32x4*)(s_BS + tok * NS + n) = live ? *(const f32x4*)(a.B + (row0 + tok) * a.ldbc + grp * N + n0 + n) : zero4;
        }
        block_sync();
        for (int n = 0; n < nh; n += 4)
        {
            f32x4 cv[4], bv[4];
            #pragma unroll
            for (int i = 0; i < 4; i++) { cv[i] = *(const f32x4*)(s_C + (ra + 16 * i) * NS + n); bv[i] = *(const f32x4*)(s_BS + (cb + 16 * i) * NS + n); }
            #pragma unroll
            for (int i = 0; i < 4; i++)
                #pragma unroll
                for (int j = 0; j < 4; j++)
                    if (j <= i)
                    {
                        #pragma unroll
                        for (int k = 0; k < 4; k++) macc[i][j] = fmaf(cv[i][k], bv[j][k], macc[i][j]);
                    }
        }
        block_sync();                                            // B is no longer needed: its place takes the state's slice
        #pragma unroll 4
        for (int i = t * 4; i < nh * P; i += 1024) *(f32x4*)(s_BS + i) = *(const f32x4*)(zin + (long long)n0 * P + i);
        block_sync();
        #pragma unroll
        for (int yt = 0; yt < SSD_YT; yt++)
        {
            const int tile = t + 256 * yt;
            if (tile >= tiles) break;
            const int t0 = (tile / tp) * 4, p0 = (tile % tp) * 4;
            if (t0 >= lc) continue;
            for (int n = 0; n < nh; n += 4)
            {
                f32x4 cv[4], sv[4];
                #pragma unroll
                for (int i = 0; i < 4; i++) { cv[i] = *(const f32x4*)(s_C + (t0 + i) * NS + n); sv[i] = *(const f32x4*)(s_BS + (n + i) * P + p0); }
                #pragma unroll
                for (int i = 0; i < 4; i++)
                    #pragma unroll
                    for (int k = 0; k < 4; k++)
                        #pragma unroll
                        for (int j = 0; j < 4; j++) inter[yt][i][j] = fmaf(cv[i][k], sv[k][j], inter[yt][i][j]);
            }
        }
    }
    // M[t][s] = (C_t . B_s) exp(c_t - c_s) for s <= t, 0 above the diagonal
    #pragma unroll
    for (int i = 0; i < 4; i++)
        #pragma unroll
        for (int j = 0; j < 4; j++)
        {
            const int tt = ra + 16 * i, ss = cb + 16 * j;
            s_M[tt * MS + ss] = ss <= tt ? macc[i][j] * expf(s_cum[tt] - s_cum[ss]) : 0.0f;
        }
    block_sync();
    const float Dh = a.D[h];
    #pragma unroll
    for (int yt = 0; yt < SSD_YT; yt++)
    {
        const int tile = t + 256 * yt;
        if (tile >= tiles) break;
        const int t0 = (tile / tp) * 4, p0 = (tile % tp) * 4;
        if (t0 >= lc) continue;
        float intra[4][4] = {};
        for (int s0 = 0; s0 <= t0; s0 += 4)
        {
            f32x4 mv[4], xv[4];
            #pragma unroll
            for (int i = 0; i < 4; i++) { mv[i] = *(const f32x4*)(s_M + (t0 + i) * MS + s0); xv[i] = *(const f32x4*)(s_X + (s0 + i) * P + p0); }
            #pragma unroll
            for (int i = 0; i < 4; i++)
                #pragma unroll
                for (int k = 0; k < 4; k++)
                    #pragma unroll
                    for (int j = 0; j < 4; j++) intra[i][j] = fmaf(mv[i][k], xv[k][j], intra[i][j]);
        }
        #pragma unroll
        for (int i = 0; i < 4; i++)
        {
            if (t0 + i >= lc) break;
            const float e = expf(s_cum[t0 + i]);
            const f32x4 uv = *(const f32x4*)(a.u + (row0 + t0 + i) * a.ldu + h * P + p0);
            f32x4 y;
            #pragma unroll
            for (int j = 0; j < 4; j++) y[j] = fmaf(e, inter[yt][i][j], intra[i][j]) + Dh * uv[j];
            *(f32x4*)(a.y + (row0 + t0 + i) * a.ldy + h * P + p0) = y;
        }
    }
}

// ---- gate + group-wise RMS norm -------------------------------------------------------------------------------------------------

// grid (rows, norm groups): out[r, part] = rms(y[r, part] * silu(z[r, part])) * w[part].  Parts of up to 256 * GN_EPT values are held in
// registers between the two passes (all of a thread's loads leave together); longer parts are read twice.
#define GN_EPT 16

template <typename T>
KERNEL void __launch_bounds__(256) gated_group_norm_kernel(const float* y, int ldy, const float* z, int ldz, const T* w, void* out, int ldo,
                                                            int out_f32, int part, float eps)
{
    SHARED float red[4];
    const int r = bid_x(), o0 = bid_y() * part;
    const float* yr = y + (long long)r * ldy + o0;
    const float* zr = z + (long long)r * ldz + o0;
    const bool held = part <= 256 * GN_EPT;
    float v[GN_EPT];
    float ss = 0.0f;
    if (held)
    {
        float yv[GN_EPT], zv[GN_EPT];
        #pragma unroll
        for (int e = 0; e < GN_EPT; e++)
        {
            const int i = tid() + 256 * e;
            yv[e] = i < part ? yr[i] : 0.0f;
            zv[e] = i < part ? zr[i] : 0.0f;
        }
        #pragma unroll
        for (int e = 0; e < GN_EPT; e++) { v[e] = yv[e] * ss_silu(zv[e]); ss = fmaf(v[e], v[e], ss); }
    }
    else
        for (int i = tid(); i < part; i += 256) { const float x = yr[i] * ss_silu(zr[i]); ss = fmaf(x, x, ss); }
    ss = wave_allreduce_add(ss);
    if (lane_id() == 0) red[wave_id()] = ss;
    block_sync();
    const float rinv = 1.0f / sqrtf((red[0] + red[1] + red[2] + red[3]) / (float)part + eps);
    if (held)
    {
        #pragma unroll
        for (int e = 0; e < GN_EPT; e++)
        {
            const int i = tid() + 256 * e;
            if (i >= part) break;
            const float o = v[e] * rinv * ss_ld<T>(w + o0 + i);
            if (out_f32) ((float*)out)[(long long)r * ldo + o0 + i] = o; else ss_st<T>((T*)out + (long long)r * ldo + o0 + i, o);
        }
        return;
    }
    for (int i = tid(); i < part; i += 256)
    {
        const float o = yr[i] * ss_silu(zr[i]) * rinv * ss_ld<T>(w + o0 + i);
        if (out_f32) ((float*)out)[(long long)r * ldo + o0 + i] = o; else ss_st<T>((T*)out + (long long)r * ldo + o0 + i, o);
    }
}

// ---- C ABI ----------------------------------------------------------------------------------------------------------------------

extern "C" int exl2_conv_rows_ex(const float* in, int ld, const void* w, const void* bias, void* out, int ldo, int out_f32, int residual,
                                 float* tail, const int* span_row0, const int* span_rows, int spans, int max_span_rows,
                                 const int* row_seq, const int* row_pos, int dtype, int channels, int taps, void* stream);

extern "C" int exl2_conv_silu_rows(const float* in, int ld, const void* w, const void* bias, float* out, int ldo, float* tail,
                                   const int* span_row0, const int* span_rows, int spans, int max_span_rows, const int* row_seq,
                                   const int* row_pos, int dtype, int channels, int taps, void* stream)
{
    return exl2_conv_rows_ex(in, ld, w, bias, out, ldo, 1, 0, tail, span_row0, span_rows, spans, max_span_rows, row_seq, row_pos, dtype,
                             channels, taps, stream);
}

/* The same convolution with a choice of output: residual = 0: silu(conv + bias); 1: in + conv + bias, no activation (what a
   sublayer reads when its input passes a short convolution beside the identity).  out fp32, or the operand dtype with out_f32 = 0. */
extern "C" int exl2_conv_rows_ex(const float* in, int ld, const void* w, const void* bias, void* out, int ldo, int out_f32, int residual,
                                 float* tail, const int* span_row0, const int* span_rows, int spans, int max_span_rows,
                                 const int* row_seq, const int* row_pos, int dtype, int channels, int taps, void* stream)
{
    EXL2_REQUIRE(in && w && out && tail && span_row0 && span_rows && row_seq && row_pos, "conv_silu_rows: null operand");
    EXL2_REQUIRE(dtype == 0 || dtype == 1, "conv_silu_rows: dtype must be 0 (bfloat16) or 1 (float32)");
    EXL2_REQUIRE(taps >= 1 && taps <= CONV_MAX_TAPS, "conv_silu_rows: %d taps (1 .. %d)", taps, CONV_MAX_TAPS);
    EXL2_REQUIRE(channels > 0 && ld >= channels && ldo >= channels, "conv_silu_rows: bad shape");
    if (spans <= 0 || max_span_rows <= 0) return EXL2_OK;
    ConvArgs a;
    a.in = in; a.ld = ld; a.w = w; a.bias = bias; a.out = out; a.ldo = ldo; a.tail = tail; a.span_row0 = span_row0; a.span_rows = span_rows;
    a.row_seq = row_seq; a.row_pos = row_pos; a.channels = channels; a.taps = taps;
    a.out_f32 = out_f32 || dtype == 1; a.residual = residual;
    a.roll_tail = max_span_rows <= CONV_TOKENS;
    const dim3 grid((channels + 255) / 256, (max_span_rows + CONV_TOKENS - 1) / CONV_TOKENS, spans);
    if (dtype == 0)
    {
        if (taps <= 4) LAUNCH((conv_silu_kernel<u16, 4>), grid, dim3(256), 0, stream, a);
        else if (taps <= 8) LAUNCH((conv_silu_kernel<u16, 8>), grid, dim3(256), 0, stream, a);
        else LAUNCH((conv_silu_kernel<u16, CONV_MAX_TAPS>), grid, dim3(256), 0, stream, a);
    }
    else
    {
        if (taps <= 4) LAUNCH((conv_silu_kernel<float, 4>), grid, dim3(256), 0, stream, a);
        else if (taps <= 8) LAUNCH((conv_silu_kernel<float, 8>), grid, dim3(256), 0, stream, a);
        else LAUNCH((conv_silu_kernel<float, CONV_MAX_TAPS>), grid, dim3(256), 0, stream, a);
    }
    if (taps > 1 && !a.roll_tail) LAUNCH(conv_tail_kernel, dim3((channels + 255) / 256, spans), dim3(256), 0, stream, a);
    HIP_TRY(hipGetLastError());
    return EXL2_OK;
}

extern "C" int exl2_ssm_scan(const float* u, int ldu, const float* B, const float* C, int ldbc, const float* dt, int lddt,
                             const float* dt_bias, const float* A_log, const float* D, float* y, int ldy, float* state,
                             const int* span_row0, const int* span_rows, int spans, const int* row_seq, const int* row_pos,
                             int heads, int groups, int n_state, int vdim, void* stream)
{
    EXL2_REQUIRE(u && B && C && dt && dt_bias && A_log && D && y && state && span_row0 && span_rows && row_seq && row_pos,
                 "ssm_scan: null operand");
    EXL2_REQUIRE(heads > 0 && groups > 0 && heads % groups == 0, "ssm_scan: %d heads in %d groups", heads, groups);
    EXL2_REQUIRE(n_state > 0 && vdim > 0 && vdim <= 256, "ssm_scan: state %d x %d", n_state, vdim);
    if (spans <= 0) return EXL2_OK;
    int ks = 256 / vdim;
    if (ks < 1) ks = 1;
    if (ks > n_state) ks = n_state;
    const int npt = (n_state + ks - 1) / ks;
    EXL2_REQUIRE(npt <= SCAN_MAX_NPT, "ssm_scan: state %d x %d needs %d rows per thread (at most %d)", n_state, vdim, npt, SCAN_MAX_NPT);
    ScanArgs a;
    a.u = u; a.ldu = ldu; a.B = B; a.C = C; a.ldbc = ldbc; a.dt = dt; a.lddt = lddt; a.dt_bias = dt_bias; a.A_log = A_log; a.D = D;
    a.y = y; a.ldy = ldy; a.state = state; a.span_row0 = span_row0; a.span_rows = span_rows; a.row_seq = row_seq; a.row_pos = row_pos;
    a.heads = heads; a.groups = groups; a.N = n_state; a.P = vdim; a.KS = ks;
    const size_t smem = sizeof(float) * ((size_t)SCAN_CHUNK * (vdim + 2 * n_state + 2 + (size_t)ks * vdim));
    EXL2_REQUIRE(smem <= 64 * 1024, "ssm_scan: state %d x %d does not fit the staging buffers", n_state, vdim);
    const dim3 grid(heads, spans), block((vdim * ks + 63) / 64 * 64);
    if (npt <= 8) LAUNCH(scan_kernel<8>, grid, block, smem, stream, a);
    else if (npt <= 16) LAUNCH(scan_kernel<16>, grid, block, smem, stream, a);
    else if (npt <= 32) LAUNCH(scan_kernel<32>, grid, block, smem, stream, a);
    else if (npt <= 64) LAUNCH(scan_kernel<64>, grid, block, smem, stream, a);
    else LAUNCH(scan_kernel<SCAN_MAX_NPT>, grid, block, smem, stream, a);
    HIP_TRY(hipGetLastError());
    return EXL2_OK;
}

static size_t ssd_out_smem(int nh, int P)
{
    const size_t bs = (size_t)SSD_L * (nh + 4) > (size_t)nh * P ? (size_t)SSD_L * (nh + 4) : (size_t)nh * P;
    return sizeof(float) * (2 * SSD_L + (size_t)SSD_L * (nh + 4) + bs + (size_t)SSD_L * P + (size_t)SSD_L * (SSD_L + 4));
}

// the slice of the state dimension the output kernel stages: the largest N / {1, 2, 4, 8} (a multiple of 4) whose images let two
// workgroups share a CU's LDS, else the smallest that fits at all; 0: none fits
static int ssd_slice(int N, int P)
{
    int fits = 0;
    for (int parts = 1; parts <= 8; parts *= 2)
    {
        if (N % (4 * parts) != 0) break;
        const int nh = N / parts;
        const size_t sm = ssd_out_smem(nh, P);
        if (sm <= 76 * 1024) return nh;
        if (sm <= 160 * 1024 - 256) fits = nh;
    }
    return fits;
}

/* 1 if exl2_ssm_scan_chunked takes this shape (sizes in fours that fit the LDS), 0 otherwise */
extern "C" int exl2_ssm_scan_chunked_supported(int n_state, int vdim)
{
    return n_state > 0 && vdim > 0 && n_state % 4 == 0 && vdim % 4 == 0 && vdim <= 64 * SSD_YT && ssd_slice(n_state, vdim) > 0
           && sizeof(float) * (2 * SSD_L + (size_t)SSD_L * (n_state + vdim)) <= 160 * 1024 - 256;
}

extern "C" int exl2_ssm_scan_chunked(const float* u, int ldu, const float* B, const float* C, int ldbc, const float* dt, int lddt,
                                     const float* dt_bias, const float* A_log, const float* D, float* y, int ldy, float* state,
                                     const int* span_row0, const int* span_rows, const int* span_chunk0, int spans, int max_span_rows,
                                     int chunk, const int* row_seq, const int* row_pos, float* zbuf, float* dbuf,
                                     int heads, int groups, int n_state, int vdim, void* stream)
{
    EXL2_REQUIRE(u && B && C && dt && dt_bias && A_log && D && y && state && span_row0 && span_rows && span_chunk0 && row_seq && row_pos
                 && zbuf && dbuf, "ssm_scan_chunked: null operand");
    EXL2_REQUIRE(chunk == SSD_L, "ssm_scan_chunked: chunks of %d rows (the span table was made for %d)", SSD_L, chunk);
    EXL2_REQUIRE(heads > 0 && groups > 0 && heads % groups == 0, "ssm_scan_chunked: %d heads in %d groups", heads, groups);
    EXL2_REQUIRE(exl2_ssm_scan_chunked_supported(n_state, vdim), "ssm_scan_chunked: state %d x %d outside the chunked form", n_state, vdim);
    EXL2_REQUIRE(ldu % 4 == 0 && ldy % 4 == 0 && ldbc % 4 == 0 && ((uintptr_t)u % 16) == 0 && ((uintptr_t)y % 16) == 0
                 && ((uintptr_t)B % 16) == 0 && ((uintptr_t)C % 16) == 0 && ((uintptr_t)zbuf % 16) == 0,
                 "ssm_scan_chunked: rows of u / B / C / y must be 16-byte aligned");
    if (spans <= 0 || max_span_rows <= 0) return EXL2_OK;
    SsdArgs g;
    ScanArgs& a = g.s;
    a.u = u; a.ldu = ldu; a.B = B; a.C = C; a.ldbc = ldbc; a.dt = dt; a.lddt = lddt; a.dt_bias = dt_bias; a.A_log = A_log; a.D = D;
    a.y = y; a.ldy = ldy; a.state = state; a.span_row0 = span_row0; a.span_rows = span_rows; a.row_seq = row_seq; a.row_pos = row_pos;
    a.heads = heads; a.groups = groups; a.N = n_state; a.P = vdim; a.KS = 0;
    g.zbuf = zbuf; g.dbuf = dbuf; g.span_chunk0 = span_chunk0; g.nh = ssd_slice(n_state, vdim);
    const size_t smem1 = sizeof(float) * (2 * SSD_L + (size_t)SSD_L * (n_state + vdim)), smem3 = ssd_out_smem(g.nh, vdim);
    static bool attr_done[EXL2_MAX_DEVICES];
    if (exl2_first_on_device(attr_done))
    {
        (void)hipFuncSetAttribute((const void*)ssd_chunk_state_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        (void)hipFuncSetAttribute((const void*)ssd_chunk_out_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    }
    const int chunks = (max_span_rows + SSD_L - 1) / SSD_L;
    LAUNCH(ssd_chunk_state_kernel, dim3(chunks, heads, spans), dim3(256), smem1, stream, g);
    LAUNCH(ssd_carry_kernel, dim3((n_state * vdim + 255) / 256, heads, spans), dim3(256), 0, stream, g);
    LAUNCH(ssd_chunk_out_kernel, dim3(chunks, heads, spans), dim3(256), smem3, stream, g);
    HIP_TRY(hipGetLastError());
    return EXL2_OK;
}

extern "C" int exl2_gated_group_norm(const float* y, int ldy, const float* z, int ldz, const void* w, void* out, int ldo, int out_f32,
                                     int dtype, int rows, int dim, int groups, float eps, void* stream)
{
    EXL2_REQUIRE(y && z && w && out, "gated_group_norm: null operand");
    EXL2_REQUIRE(dtype == 0 || dtype == 1, "gated_group_norm: dtype must be 0 (bfloat16) or 1 (float32)");
    EXL2_REQUIRE(dim > 0 && groups > 0 && dim % groups == 0, "gated_group_norm: %d values in %d groups", dim, groups);
    if (rows <= 0) return EXL2_OK;
    if (dtype == 0) LAUNCH(gated_group_norm_kernel<u16>, dim3(rows, groups), dim3(256), 0, stream, y, ldy, z, ldz, (const u16*)w, out, ldo, out_f32, dim / groups, eps);
    else LAUNCH(gated_group_norm_kernel<float>, dim3(rows, groups), dim3(256), 0, stream, y, ldy, z, ldz, (const float*)w, out, ldo, 1, dim / groups, eps);
    HIP_TRY(hipGetLastError());
    return EXL2_OK;
}
