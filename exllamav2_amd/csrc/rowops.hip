// rowops.hip -- the row-wise steps around the dense linears (dense.hip), fp32 arithmetic throughout, + their C ABI:
//   * embedding gather times a scale into the fp32 residual stream (+ its operand-dtype copy for the next linear),
//   * RMS norm of a (strided) fp32 row slice with a plain weight w or a zero-centred one (1 + w), optional row gather,
//   * the pre-norm residual step  x <- x + y  with the layer norm (weight and bias) that feeds the next sublayer,
//   * the post-norm residual step  x <- norm(alpha x + y) (1 + w), where y is a linear's fp32 output or the weighted sum of a
//     token's chosen experts (identity experts contribute the token's own x),
//   * the pre-norm residual step  x <- x + y (+ the sum of a token's expert outputs)  with an RMS norm whose gain is ONE number and
//     a token shift  h + (h' - h) * shift  towards the previous token's normed row (kept per sequence slot),
//   * the sandwich-normed residual step  x <- x + mult n_g(sublayer) w_out  with the grouped RMS norm  n_g(x) w_in  that feeds the next
//     sublayer (and, for single-token steps, the short convolution over the last normed rows of the sequence),
//   * a token embedding plus a hashed (previous token, token) embedding under a grouped RMS norm (the previous token kept per slot),
//   * the sparse-MoE router (softmax over all experts, selection by score + correction, weights from the uncorrected scores; or
//     sigmoid scores, selection and weights by the scores themselves) and the per-expert row lists the grouped linear reads.
// Element type T of weights / operand copies: u16 = bfloat16 bits, float.
#include "hw.h"
#include "errors.h"
#include <stdint.h>

template <typename T> DEV float ro_ld(const T* p);
template <> DEV float ro_ld<u16>(const u16* p) { return bf16_to_f32(*p); }
template <> DEV float ro_ld<float>(const float* p) { return *p; }
template <typename T> DEV void ro_st(T* p, float v);
template <> DEV void ro_st<u16>(u16* p, float v) { *p = f32_to_bf16(v); }
template <> DEV void ro_st<float>(float* p, float v) { *p = v; }

// sum over the 256 threads of a workgroup (every thread gets it)
DEV float block_sum_256(float v, float* part)
{
    v = wave_allreduce_add(v);
    block_sync();
    if (lane_id() == 0) part[wave_id()] = v;
    block_sync();
    return part[0] + part[1] + part[2] + part[3];
}

// ---- embedding ------------------------------------------------------------------------------------------------------------

template <typename T>
KERNEL void __launch_bounds__(256) embed_scale_kernel(const T* table, const int* ids, float* x32, T* xh, int width, int vocab, float scale)
{
    const int r = bid_x();
    int id = ids[r];
    id = min(max(id, 0), vocab - 1);
    const T* src = table + (long long)id * width;
    for (int i = tid(); i < width; i += 256)
    {
        const float v = ro_ld<T>(src + i) * scale;
        x32[(long long)r * width + i] = v;
        if (xh && (void*)xh != (void*)x32) ro_st<T>(xh + (long long)r * width + i, v);
    }
}

// ---- RMS norm of a row slice ------------------------------------------------------------------------------------------------

template <typename T>
KERNEL void __launch_bounds__(256) rms_rows_kernel(const float* x, int ldx, const T* w, int one_plus, void* y, int ldy, int y_f32,
                                                    const int* row_idx, int dim, float eps)
{
    SHARED float part[4];
    const int r = bid_x();
    const float* xr = x + (long long)(row_idx ? row_idx[r] : r) * ldx;
    float ss = 0.0f;
    for (int i = tid(); i < dim; i += 256) { const float v = xr[i]; ss = fmaf(v, v, ss); }
    ss = block_sum_256(ss, part);
    const float rinv = 1.0f / sqrtf(ss / (float)dim + eps);
    for (int i = tid(); i < dim; i += 256)
    {
        const float wv = ro_ld<T>(w + i) + (one_plus ? 1.0f : 0.0f);
        const float v = xr[i] * rinv * wv;
        if (y_f32) ((float*)y)[(long long)r * ldy + i] = v; else ro_st<T>((T*)y + (long long)r * ldy + i, v);
    }
}

// ---- x <- norm(alpha x + y) (1 + w) -------------------------------------------------------------------------------------------

struct PostNormArgs
{
    float* x; void* xh; const float* y; const void* w;
    int width; float alpha, eps;
    // sparse-MoE form (y == nullptr): y = sum_k moe_w[r, k] * (moe_ids[r, k] >= n_real ? x[r] : moe_y[r * top + k])
    const float* moe_y; const int* moe_ids; const float* moe_w; int top, n_real;
};

template <typename T>
KERNEL void __launch_bounds__(256) post_norm_kernel(const PostNormArgs a)
{
    DYN_SMEM(smem);
    SHARED float part[4];
    float* v = (float*)smem;                                     // the row before the norm
    const int r = bid_x();
    float* xr = a.x + (long long)r * a.width;
    float ss = 0.0f;
    for (int i = tid(); i < a.width; i += 256)
    {
        const float xv = xr[i];
        float yv;
        if (a.y) yv = a.y[(long long)r * a.width + i];
        else
        {
            yv = 0.0f;
            for (int k = 0; k < a.top; k++)
            {
                const int e = a.moe_ids[r * a.top + k];
                const float src = e >= a.n_real ? xv : a.moe_y[((long long)r * a.top + k) * a.width + i];
                yv = fmaf(a.moe_w[r * a.top + k], src, yv);
            }
        }
        const float s = fmaf(a.alpha, xv, yv);
        v[i] = s;
        ss = fmaf(s, s, ss);
    }
    ss = block_sum_256(ss, part);
    const float rinv = 1.0f / sqrtf(ss / (float)a.width + a.eps);
    T* xh = (T*)a.xh;
    for (int i = tid(); i < a.width; i += 256)
    {
        const float o = v[i] * rinv * (1.0f + ro_ld<T>((const T*)a.w + i));
        xr[i] = o;
        if (xh && (void*)xh != (void*)a.x) ro_st<T>(xh + (long long)r * a.width + i, o);
    }
}

// ---- x <- x + y, then layer norm (mean removed, weight and bias) -------------------------------------------------------------------
// The residual step of a pre-norm layer and the norm in front of the next sublayer as one launch: the fp32 stream takes the
// sublayer's output (y, nullable), and the normalised row goes out in the operand dtype (w nullable: only the addition).  The
// variance is the mean of the squared deviations from the mean (two passes over the row held in LDS).

struct LayerNormArgs
{
    float* x; const float* y; const void* w; const void* b; void* out; int out_f32;
    const int* row_idx;                      // nullable: output row r is made from stream row row_idx[r] (no addition then)
    int width; float eps;
};

template <typename T>
KERNEL void __launch_bounds__(256) add_layer_norm_kernel(const LayerNormArgs a)
{
    DYN_SMEM(smem);
    SHARED float part[4];
    float* v = (float*)smem;
    const int r = bid_x();
    const long long src = a.row_idx ? a.row_idx[r] : r;
    float* xr = a.x + src * a.width;
    float s = 0.0f;
    for (int i = tid(); i < a.width; i += 256)
    {
        float xv = xr[i];
        if (a.y) { xv += a.y[src * a.width + i]; xr[i] = xv; }
        v[i] = xv;
        s += xv;
    }
    if (!a.w) return;
    const float mean = block_sum_256(s, part) / (float)a.width;
    float ss = 0.0f;
    for (int i = tid(); i < a.width; i += 256) { const float d = v[i] - mean; ss = fmaf(d, d, ss); }
    ss = block_sum_256(ss, part);
    const float rinv = 1.0f / sqrtf(ss / (float)a.width + a.eps);
    for (int i = tid(); i < a.width; i += 256)
    {
        const float o = (v[i] - mean) * rinv * ro_ld<T>((const T*)a.w + i) + (a.b ? ro_ld<T>((const T*)a.b + i) : 0.0f);
        if (a.out_f32) ((float*)a.out)[(long long)r * a.width + i] = o; else ro_st<T>((T*)a.out + (long long)r * a.width + i, o);
    }
}

// The same step for rows of up to 256 * 4 * LN_VPT values in fours: a thread keeps its values in registers between the passes (no
// LDS image), all its 16-byte loads leave together, results go out as 16-byte (fp32) or 8-byte (bfloat16) stores.
#define LN_VPT 4

template <typename T> DEV f32x4 ro_ld4(const T* p);
template <> DEV f32x4 ro_ld4<float>(const float* p) { return *(const f32x4*)p; }
template <> DEV f32x4 ro_ld4<u16>(const u16* p)
{
    const u32x2 v = *(const u32x2*)p;
    return (f32x4){as_f32(v[0] << 16), as_f32(v[0] & 0xffff0000u), as_f32(v[1] << 16), as_f32(v[1] & 0xffff0000u)};
}

template <typename T>
KERNEL void __launch_bounds__(256) add_layer_norm_vec_kernel(const LayerNormArgs a)
{
    SHARED float part[4];
    const int r = bid_x();
    const long long src = a.row_idx ? a.row_idx[r] : r;
    const int nvec = a.width / 4;
    f32x4* xr = (f32x4*)(a.x + src * a.width);
    const f32x4* yr = a.y ? (const f32x4*)(a.y + src * a.width) : nullptr;
    f32x4 v[LN_VPT], yv[LN_VPT];
    #pragma unroll
    for (int e = 0; e < LN_VPT; e++)
    {
        const int i = tid() + 256 * e;
        v[e] = i < nvec ? xr[i] : (f32x4){0.0f, 0.0f, 0.0f, 0.0f};
        yv[e] = (yr && i < nvec) ? yr[i] : (f32x4){0.0f, 0.0f, 0.0f, 0.0f};
    }
    float s = 0.0f;
    #pragma unroll
    for (int e = 0; e < LN_VPT; e++)
    {
        const int i = tid() + 256 * e;
        if (yr)
        {
            v[e][0] += yv[e][0]; v[e][1] += yv[e][1]; v[e][2] += yv[e][2]; v[e][3] += yv[e][3];
            if (i < nvec) xr[i] = v[e];
        }
        s += (v[e][0] + v[e][1]) + (v[e][2] + v[e][3]);
    }
    if (!a.w) return;
    const float mean = block_sum_256(s, part) / (float)a.width;
    float ss = 0.0f;
    #pragma unroll
    for (int e = 0; e < LN_VPT; e++)
    {
        if (tid() + 256 * e >= nvec) break;
        #pragma unroll
        for (int k = 0; k < 4; k++) { const float d = v[e][k] - mean; ss = fmaf(d, d, ss); }
    }
    ss = block_sum_256(ss, part);
    const float rinv = 1.0f / sqrtf(ss / (float)a.width + a.eps);
    #pragma unroll
    for (int e = 0; e < LN_VPT; e++)
    {
        const int i = tid() + 256 * e;
        if (i >= nvec) break;
        const f32x4 wv = ro_ld4<T>((const T*)a.w + 4 * i);
        const f32x4 bv = a.b ? ro_ld4<T>((const T*)a.b + 4 * i) : (f32x4){0.0f, 0.0f, 0.0f, 0.0f};
        f32x4 o;
        #pragma unroll
        for (int k = 0; k < 4; k++) o[k] = (v[e][k] - mean) * rinv * wv[k] + bv[k];
        if (a.out_f32) *(f32x4*)((float*)a.out + (long long)r * a.width + 4 * i) = o;
        else *(u32x2*)((u16*)a.out + (long long)r * a.width + 4 * i) =
                 (u32x2){(u32)f32_to_bf16(o[0]) | ((u32)f32_to_bf16(o[1]) << 16), (u32)f32_to_bf16(o[2]) | ((u32)f32_to_bf16(o[3]) << 16)};
    }
}

// ---- x <- x + y, RMS norm with a scalar gain, token shift --------------------------------------------------------------------------
// hn[r] = x[r] / sqrt(mean(x[r]^2) + eps) * gain after the stream took the sublayer's output: y (nullable) and / or the sum of the
// `top` expert outputs of the row (moe_y rows r * top .. + top, nullable).  With a shift vector the consumer reads
// out[r] = hn[r] + (hn' - hn[r]) * shift, hn' = the normed row of the sequence's previous token: the row in front of r when that
// belongs to the same sequence, else what the slot keeps (prev fp32 [slots, width]), zeros at position 0.  Steps whose spans are
// single rows (decoding) do everything in ONE launch and roll the slot; otherwise hn goes to a buffer, a second launch shifts
// (every row independent) and a third rolls the slots from the spans' last rows -- nothing reads a slot after it was rolled.

struct RmsShiftArgs
{
    float* x; const float* y; const float* moe_y; int top;
    float* hn;                               // fp32 [rows, width] (multi-row spans with a shift), else unused
    void* out; int out_f32;                  // [rows, width] operand dtype or fp32
    const void* shift;                       // [width] operand dtype (nullable: out = hn)
    float* prev;                             // fp32 [slots, width]
    const int* row_seq; const int* row_pos; const int* row_idx;
    int width; float gain, eps; int fused;   // fused: single-row spans, shift and slot roll inside the norm launch
};

template <typename T>
KERNEL void __launch_bounds__(256) add_rms_shift_kernel(const RmsShiftArgs a)
{
    DYN_SMEM(smem);
    SHARED float part[4];
    float* v = (float*)smem;
    const int r = bid_x();
    const long long src = a.row_idx ? a.row_idx[r] : r;
    float* xr = a.x + src * a.width;
    float ss = 0.0f;
    for (int i = tid(); i < a.width; i += 256)
    {
        float xv = xr[i];
        if (a.y || a.moe_y)
        {
            if (a.y) xv += a.y[src * a.width + i];
            for (int k = 0; k < (a.moe_y ? a.top : 0); k++) xv += a.moe_y[(src * a.top + k) * a.width + i];
            xr[i] = xv;
        }
        v[i] = xv;
        ss = fmaf(xv, xv, ss);
    }
    if (!a.out && !a.hn) return;                                 // only the addition
    ss = block_sum_256(ss, part);
    const float mul = a.gain / sqrtf(ss / (float)a.width + a.eps);
    if (a.shift && !a.fused)
    {
        for (int i = tid(); i < a.width; i += 256) a.hn[(long long)r * a.width + i] = v[i] * mul;
        return;
    }
    float* pv = nullptr; bool first = true;
    if (a.shift) { pv = a.prev + (long long)a.row_seq[r] * a.width; first = a.row_pos[r] == 0; }
    for (int i = tid(); i < a.width; i += 256)
    {
        const float hn = v[i] * mul;
        float o = hn;
        if (a.shift)
        {
            const float hp = first ? 0.0f : pv[i];
            o = fmaf(hp - hn, ro_ld<T>((const T*)a.shift + i), hn);
            pv[i] = hn;
        }
        if (a.out_f32) ((float*)a.out)[(long long)r * a.width + i] = o; else ro_st<T>((T*)a.out + (long long)r * a.width + i, o);
    }
}

// grid (rows, width / 256): out[r] = hn[r] + (hn' - hn[r]) * shift
template <typename T>
KERNEL void __launch_bounds__(256) token_shift_kernel(const RmsShiftArgs a)
{
    const int r = bid_x(), i = bid_y() * 256 + tid();
    if (i >= a.width) return;
    const int pos = a.row_pos[r], sq = a.row_seq[r];
    float hp = 0.0f;
    if (pos > 0) hp = (r > 0 && a.row_seq[r - 1] == sq) ? a.hn[(long long)(r - 1) * a.width + i] : a.prev[(long long)sq * a.width + i];
    const float hn = a.hn[(long long)r * a.width + i];
    const float o = fmaf(hp - hn, ro_ld<T>((const T*)a.shift + i), hn);
    if (a.out_f32) ((float*)a.out)[(long long)r * a.width + i] = o; else ro_st<T>((T*)a.out + (long long)r * a.width + i, o);
}

// grid (spans, width / 256): slot of span s <- row (last of the span) of src fp32 [rows, ld]
KERNEL void __launch_bounds__(256) span_last_row_kernel(const float* src, int ld, float* slot_rows, int width, const int* span_row0,
                                                         const int* span_rows, const int* row_seq)
{
    const int s = bid_x(), i = bid_y() * 256 + tid();
    if (i >= width) return;
    const int last = span_row0[s] + span_rows[s] - 1;
    slot_rows[(long long)row_seq[last] * width + i] = src[(long long)last * ld + i];
}

// ---- sandwich-normed residual step ---------------------------------------------------------------------------------------------
// n_g(v) = v cut into `groups` equal runs, each divided by sqrt(mean(run^2) + eps).  One launch per row does
//     x <- x + mult * n_g(t) w_out,   t = ya y + yb y2 + the sum of the row's `top` expert rows      (any of the three may be absent)
//     hn = n_g(x) w_in                                                                              (w_in nullable: only the addition)
// i.e. the norm BEHIND a sublayer, the residual addition and the norm IN FRONT of the next sublayer.  The consumer of hn may read it
// through a short causal convolution over the sequence, out = hn + sum_j c[:, j] hn_(p - taps + 1 + j): steps whose spans are single
// rows (decoding) do that here too, from the slot's tail [slots, taps - 1, width] of the last normed rows, and roll the tail (a thread
// reads and writes only its own channels); otherwise hn goes out in fp32 and the convolution is exl2_conv_rows_ex's.

struct SandwichArgs
{
    float* x;
    const float* y; float ya; const float* y2; float yb; const float* moe_y; int top;
    const void* w_out; float mult;
    const void* w_in;
    void* out; int out_f32;
    const int* row_idx;                      // nullable: output row r is made from stream row row_idx[r] (no addition then)
    const void* conv_w; float* tail; const int* row_seq; const int* row_pos; int taps;      // conv_w nullable
    int width, groups; float eps;
};

template <typename T>
KERNEL void __launch_bounds__(256) sandwich_norm_kernel(const SandwichArgs a)
{
    DYN_SMEM(smem);
    SHARED float part[4];
    float* v = (float*)smem;
    const int r = bid_x();
    const long long src = a.row_idx ? a.row_idx[r] : r;
    float* xr = a.x + src * a.width;
    const int gs = a.width / a.groups;
    if (a.y || a.y2 || a.moe_y)
    {
        for (int i = tid(); i < a.width; i += 256)
        {
            float t = 0.0f;
            if (a.y) t = a.ya * a.y[src * a.width + i];
            if (a.y2) t = fmaf(a.yb, a.y2[src * a.width + i], t);
            for (int k = 0; k < (a.moe_y ? a.top : 0); k++) t += a.moe_y[(src * a.top + k) * a.width + i];
            v[i] = t;
        }
        for (int g = 0; g < a.groups; g++)
        {
            float ss = 0.0f;
            for (int i = g * gs + tid(); i < (g + 1) * gs; i += 256) ss = fmaf(v[i], v[i], ss);
            ss = block_sum_256(ss, part);
            const float mul = a.mult / sqrtf(ss / (float)gs + a.eps);
            for (int i = g * gs + tid(); i < (g + 1) * gs; i += 256)
            {
                const float xv = fmaf(v[i] * mul, ro_ld<T>((const T*)a.w_out + i), xr[i]);
                xr[i] = xv;
                v[i] = xv;
            }
        }
    }
    else
        for (int i = tid(); i < a.width; i += 256) v[i] = xr[i];
    if (!a.out) return;
    const bool conv = a.conv_w != nullptr && a.taps > 1;
    float* tl = nullptr; int pos = 0;
    if (conv) { tl = a.tail + (long long)a.row_seq[r] * (a.taps - 1) * a.width; pos = a.row_pos[r]; }
    for (int g = 0; g < a.groups; g++)
    {
        float ss = 0.0f;
        for (int i = g * gs + tid(); i < (g + 1) * gs; i += 256) ss = fmaf(v[i], v[i], ss);
        ss = block_sum_256(ss, part);
        const float rinv = 1.0f / sqrtf(ss / (float)gs + a.eps);
        for (int i = g * gs + tid(); i < (g + 1) * gs; i += 256)
        {
            const float hn = v[i] * rinv * ro_ld<T>((const T*)a.w_in + i);
            float o = hn;
            if (a.conv_w)
            {
                const T* cw = (const T*)a.conv_w + (long long)i * a.taps;
                float acc = ro_ld<T>(cw + a.taps - 1) * hn;
                float carry = hn;                                // walks the tail from its newest entry: entry j moves to j - 1
                for (int j = a.taps - 2; j >= 0; j--)
                {
                    const float old = pos - (a.taps - 1 - j) >= 0 ? tl[(long long)j * a.width + i] : 0.0f;
                    acc = fmaf(ro_ld<T>(cw + j), old, acc);
                    tl[(long long)j * a.width + i] = carry;
                    carry = old;
                }
                o = hn + acc;
            }
            if (a.out_f32) ((float*)a.out)[(long long)r * a.width + i] = o; else ro_st<T>((T*)a.out + (long long)r * a.width + i, o);
        }
    }
}

// The same step for rows of up to 256 * 4 * NC values in fours, up to SW_MAX_GROUPS norm groups of a multiple of four values and
// up to SW_MAX_TAPS taps: a thread keeps its values in registers, every operand of the launch -- the sublayer's outputs, the stream,
// both weights, the convolution's weights and the slot's tail -- is requested before the first is used, and the sums of all groups
// close in ONE exchange through LDS per norm.
#define SW_MAX_GROUPS 8
#define SW_MAX_TAPS 4

template <int NC>
DEV void sw_group_sums(const f32x4* v, const int* grp, const bool* live, int groups, float* part, float* sums)
{
    float ss[SW_MAX_GROUPS];
    #pragma unroll
    for (int g = 0; g < SW_MAX_GROUPS; g++) ss[g] = 0.0f;
    #pragma unroll
    for (int e = 0; e < NC; e++)
    {
        const float q = live[e] ? (v[e][0] * v[e][0] + v[e][1] * v[e][1]) + (v[e][2] * v[e][2] + v[e][3] * v[e][3]) : 0.0f;
        #pragma unroll
        for (int g = 0; g < SW_MAX_GROUPS; g++) ss[g] += grp[e] == g ? q : 0.0f;
    }
    block_sync();                                                // the exchange buffer may still be read from the norm before
    #pragma unroll
    for (int g = 0; g < SW_MAX_GROUPS; g++)
        if (g < groups)
        {
            const float w = wave_allreduce_add(ss[g]);
            if (lane_id() == 0) part[wave_id() * SW_MAX_GROUPS + g] = w;
        }
    block_sync();
    #pragma unroll
    for (int g = 0; g < SW_MAX_GROUPS; g++)
        sums[g] = g < groups ? (part[g] + part[SW_MAX_GROUPS + g]) + (part[2 * SW_MAX_GROUPS + g] + part[3 * SW_MAX_GROUPS + g]) : 0.0f;
}

template <typename T, int NC>
KERNEL void __launch_bounds__(256) sandwich_norm_vec_kernel(const SandwichArgs a)
{
    SHARED float part[4 * SW_MAX_GROUPS];
    const int r = bid_x();
    const long long src = a.row_idx ? a.row_idx[r] : r;
    float* xr = a.x + src * a.width;
    const int gs = a.width / a.groups;
    const bool pending = a.y || a.y2 || a.moe_y;
    const bool conv = a.conv_w != nullptr;
    f32x4 xv[NC], tv[NC], wo[NC], wi[NC], tl[NC][SW_MAX_TAPS - 1];
    float cw[NC][4][SW_MAX_TAPS];
    int grp[NC]; bool live[NC];
    float* tail = nullptr; int pos = 0;
    if (conv && a.taps > 1) { tail = a.tail + (long long)a.row_seq[r] * (a.taps - 1) * a.width; pos = a.row_pos[r]; }
    const f32x4 zero4 = {0.0f, 0.0f, 0.0f, 0.0f};
    #pragma unroll
    for (int e = 0; e < NC; e++)
    {
        const int i = 4 * (tid() + 256 * e);
        live[e] = i < a.width;
        grp[e] = live[e] ? i / gs : -1;
        xv[e] = tv[e] = wo[e] = wi[e] = zero4;
        if (!live[e]) continue;
        xv[e] = *(const f32x4*)(xr + i);
        if (pending)
        {
            wo[e] = ro_ld4<T>((const T*)a.w_out + i);
            if (a.y) { const f32x4 y = *(const f32x4*)(a.y + src * a.width + i); tv[e] = a.ya * y; }
            if (a.y2) { const f32x4 y = *(const f32x4*)(a.y2 + src * a.width + i); tv[e] += a.yb * y; }
            for (int k = 0; k < (a.moe_y ? a.top : 0); k++) tv[e] += *(const f32x4*)(a.moe_y + (src * a.top + k) * a.width + i);
        }
        if (a.out) wi[e] = ro_ld4<T>((const T*)a.w_in + i);
        if (conv)
        {
            if (a.taps == 4)                                       // a channel's four taps are one 8- or 16-byte load
            {
                #pragma unroll
                for (int k = 0; k < 4; k++)
                {
                    const f32x4 w4 = ro_ld4<T>((const T*)a.conv_w + (long long)(i + k) * 4);
                    #pragma unroll
                    for (int j = 0; j < SW_MAX_TAPS; j++) cw[e][k][j] = w4[j];
                }
            }
            else
            {
                #pragma unroll
                for (int k = 0; k < 4; k++)
                    #pragma unroll
                    for (int j = 0; j < SW_MAX_TAPS; j++)
                        cw[e][k][j] = j < a.taps ? ro_ld<T>((const T*)a.conv_w + (long long)(i + k) * a.taps + j) : 0.0f;
            }
            #pragma unroll
            for (int j = 0; j < SW_MAX_TAPS - 1; j++)
                tl[e][j] = (j < a.taps - 1 && pos - (a.taps - 1 - j) >= 0) ? *(const f32x4*)(tail + (long long)j * a.width + i) : zero4;
        }
    }
    float sums[SW_MAX_GROUPS];
    if (pending)
    {
        sw_group_sums<NC>(tv, grp, live, a.groups, part, sums);
        #pragma unroll
        for (int e = 0; e < NC; e++)
        {
            if (!live[e]) continue;
            float s = 0.0f;
            #pragma unroll
            for (int g = 0; g < SW_MAX_GROUPS; g++) s = grp[e] == g ? sums[g] : s;
            const float mul = a.mult / sqrtf(s / (float)gs + a.eps);
            #pragma unroll
            for (int k = 0; k < 4; k++) xv[e][k] = fmaf(tv[e][k] * mul, wo[e][k], xv[e][k]);
            *(f32x4*)(xr + 4 * (tid() + 256 * e)) = xv[e];
        }
    }
    if (!a.out) return;
    sw_group_sums<NC>(xv, grp, live, a.groups, part, sums);
    #pragma unroll
    for (int e = 0; e < NC; e++)
    {
        if (!live[e]) continue;
        const int i = 4 * (tid() + 256 * e);
        float s = 0.0f;
        #pragma unroll
        for (int g = 0; g < SW_MAX_GROUPS; g++) s = grp[e] == g ? sums[g] : s;
        const float rinv = 1.0f / sqrtf(s / (float)gs + a.eps);
        f32x4 hn, o;
        #pragma unroll
        for (int k = 0; k < 4; k++) hn[k] = xv[e][k] * rinv * wi[e][k];
        o = hn;
        if (conv)
        {
            #pragma unroll
            for (int k = 0; k < 4; k++)
            {
                float acc = 0.0f;
                #pragma unroll
                for (int j = 0; j < SW_MAX_TAPS; j++)
                    if (j < a.taps) acc = fmaf(cw[e][k][j], j == a.taps - 1 ? hn[k] : tl[e][j < SW_MAX_TAPS - 1 ? j : 0][k], acc);
                o[k] = hn[k] + acc;
            }
            // the tail moves up by one row: entry j takes entry j + 1, the newest takes this row
            #pragma unroll
            for (int j = 0; j < SW_MAX_TAPS - 1; j++)
                if (j < a.taps - 1)
                    *(f32x4*)(tail + (long long)j * a.width + i) = j == a.taps - 2 ? hn : tl[e][j + 1 < SW_MAX_TAPS - 1 ? j + 1 : 0];
        }
        if (a.out_f32) *(f32x4*)((float*)a.out + (long long)r * a.width + i) = o;
        else *(u32x2*)((u16*)a.out + (long long)r * a.width + i) =
                 (u32x2){(u32)f32_to_bf16(o[0]) | ((u32)f32_to_bf16(o[1]) << 16), (u32)f32_to_bf16(o[2]) | ((u32)f32_to_bf16(o[3]) << 16)};
    }
}

// ---- token embedding + hashed token-pair embedding + norm ------------------------------------------------------------------------
// x = n_g(table[t] * scale + pair[(t' mul_prev + t mul_cur) mod buckets]) w, t' = the sequence's previous token: the row in front
// when that belongs to the same sequence, else what the slot keeps (prev_tok int32 [slots]); row `buckets` of the pair table at
// position 0.  fused (single-row spans): the slot takes the row's token here, otherwise token_state_kernel does after the launch.

struct EmbedPairArgs
{
    const void* table; const void* pair; const void* w;         // pair, w nullable
    const int* ids; int* prev_tok; const int* row_seq; const int* row_pos;
    float* x;
    int width, vocab, buckets, mul_prev, mul_cur, groups, fused; float scale, eps;
};

template <typename T>
KERNEL void __launch_bounds__(256) embed_pair_kernel(const EmbedPairArgs a)
{
    DYN_SMEM(smem);
    SHARED float part[4];
    float* v = (float*)smem;
    const int r = bid_x();
    const int id = min(max(a.ids[r], 0), a.vocab - 1);
    const int sq = a.row_seq[r], pos = a.row_pos[r];
    long long prow = a.buckets;
    if (a.pair && pos > 0)
    {
        const int pt = (!a.fused && r > 0 && a.row_seq[r - 1] == sq) ? a.ids[r - 1] : a.prev_tok[sq];
        const long long hsh = ((long long)pt * a.mul_prev + (long long)id * a.mul_cur) % a.buckets;
        prow = hsh < 0 ? hsh + a.buckets : hsh;
    }
    const T* src = (const T*)a.table + (long long)id * a.width;
    const T* psrc = a.pair ? (const T*)a.pair + prow * a.width : nullptr;
    float* xr = a.x + (long long)r * a.width;
    for (int i = tid(); i < a.width; i += 256)
    {
        float t = ro_ld<T>(src + i) * a.scale;
        if (psrc) t += ro_ld<T>(psrc + i);
        v[i] = t;
        if (!a.w) xr[i] = t;
    }
    if (a.w)
    {
        const int gs = a.width / a.groups;
        for (int g = 0; g < a.groups; g++)
        {
            float ss = 0.0f;
            for (int i = g * gs + tid(); i < (g + 1) * gs; i += 256) ss = fmaf(v[i], v[i], ss);
            ss = block_sum_256(ss, part);
            const float rinv = 1.0f / sqrtf(ss / (float)gs + a.eps);
            for (int i = g * gs + tid(); i < (g + 1) * gs; i += 256) xr[i] = v[i] * rinv * ro_ld<T>((const T*)a.w + i);
        }
    }
    else block_sync();
    if (a.fused && tid() == 0) a.prev_tok[sq] = id;             // behind a barrier: every thread has read the slot
}

KERNEL void __launch_bounds__(64) token_state_kernel(const int* ids, int* prev_tok, const int* span_row0, const int* span_rows,
                                                      const int* row_seq, int spans, int vocab)
{
    const int s = bid_x() * 64 + tid();
    if (s >= spans) return;
    const int last = span_row0[s] + span_rows[s] - 1;
    prev_tok[row_seq[last]] = min(max(ids[last], 0), vocab - 1);
}

// ---- router -----------------------------------------------------------------------------------------------------------------
// One wave per token.  logits fp32 [rows, n_total]; scores = softmax over all n_total; the `top` largest (score + correction) win
// (first index on a tie); weight = score / (sum of the chosen scores + 1e-20) * scale.  sigmoid_scores: scores = sigmoid(logits),
// each on its own, and the weights are the chosen scores times scale (no renormalisation).  Rows of ids / wts are `ld` values apart;
// extra_id >= 0: column `top` of every row names that expert with weight 1 (an expert every token uses, run with the chosen ones).

#define ROUTE_MAX_PER_LANE 8

KERNEL void __launch_bounds__(64) moe_route_kernel(const float* logits, const float* correction, int* ids, float* wts,
                                                    int n_total, int top, float scale, int sigmoid_scores, int ld, int extra_id)
{
    const int r = bid_x();
    const int lane = lane_id();
    float s[ROUTE_MAX_PER_LANE], c[ROUTE_MAX_PER_LANE];
    float mx = -INFINITY;
    #pragma unroll
    for (int i = 0; i < ROUTE_MAX_PER_LANE; i++)
    {
        const int e = lane + 64 * i;
        s[i] = e < n_total ? logits[(long long)r * n_total + e] : -INFINITY;
        mx = fmaxf(mx, s[i]);
    }
    mx = wave_allreduce_max(mx);
    float sum = 0.0f;
    #pragma unroll
    for (int i = 0; i < ROUTE_MAX_PER_LANE; i++)
    {
        const int e = lane + 64 * i;
        if (sigmoid_scores) s[i] = e < n_total ? 1.0f / (1.0f + expf(-s[i])) : 0.0f;
        else s[i] = e < n_total ? expf(s[i] - mx) : 0.0f;
        sum += s[i];
    }
    sum = sigmoid_scores ? 1.0f : wave_allreduce_add(sum);
    #pragma unroll
    for (int i = 0; i < ROUTE_MAX_PER_LANE; i++)
    {
        const int e = lane + 64 * i;
        s[i] = s[i] / sum;
        c[i] = e < n_total ? s[i] + (correction ? correction[e] : 0.0f) : -INFINITY;
    }
    float chosen_sum = 0.0f;
    float my_w = 0.0f; int my_id = 0;                    // lane k keeps the k-th choice (top <= 64)
    for (int k = 0; k < top; k++)
    {
        float best = -INFINITY; int best_e = 0x7fffffff;
        #pragma unroll
        for (int i = 0; i < ROUTE_MAX_PER_LANE; i++)
        {
            const int e = lane + 64 * i;
            if (c[i] > best) { best = c[i]; best_e = e; }          // ascending e within a lane: the first maximum stays
        }
        const float wbest = wave_allreduce_max(best);
        int cand = best == wbest ? best_e : 0x7fffffff;
        #pragma unroll
        for (int m = 1; m < 64; m <<= 1) cand = min(cand, (int)shfl_xor_u32((u32)cand, m));
        // the owner hands out the score and retires the expert
        float sc = 0.0f;
        #pragma unroll
        for (int i = 0; i < ROUTE_MAX_PER_LANE; i++)
            if (lane + 64 * i == cand) { sc = s[i]; c[i] = -INFINITY; }
        sc = wave_allreduce_add(sc);
        chosen_sum += sc;
        if (lane == k) { my_w = sc; my_id = cand; }
    }
    if (lane < top)
    {
        ids[r * ld + lane] = my_id;
        wts[r * ld + lane] = sigmoid_scores ? my_w * scale : my_w / (chosen_sum + 1e-20f) * scale;
    }
    if (extra_id >= 0 && lane == 0) { ids[r * ld + top] = extra_id; wts[r * ld + top] = 1.0f; }
}

// per-expert row lists for the grouped linear, in pair order.  Two launches of one workgroup per expert: counts (256 threads, ballot +
// popcount), then offsets (sum of the counts in front) and an ordered compaction by one wave.
KERNEL void __launch_bounds__(256) moe_count_kernel(const int* ids, int pairs, int* count)
{
    SHARED int part[4];
    const int e = bid_x();
    int c = 0;
    for (int base = 0; base < pairs; base += 256)
    {
        const int p = base + tid();
        c += __builtin_popcountll(wave_ballot(p < pairs && ids[p] == e));
    }
    if (lane_id() == 0) part[wave_id()] = c;
    block_sync();
    if (tid() == 0) count[e] = part[0] + part[1] + part[2] + part[3];
}

KERNEL void __launch_bounds__(64) moe_fill_kernel(const int* ids, int pairs, const int* count, int* offset, int* rows)
{
    const int e = bid_x();
    const int lane = lane_id();
    int off = 0;
    for (int i = 0; i < e; i++) off += count[i];
    if (lane == 0) offset[e] = off;
    for (int base = 0; base < pairs; base += 64)
    {
        const int p = base + lane;
        const bool hit = p < pairs && ids[p] == e;
        const u64 mask = wave_ballot(hit);
        if (hit) rows[off + __builtin_popcountll(mask & ((1ull << lane) - 1ull))] = p;
        off += __builtin_popcountll(mask);
    }
}

// ---- C ABI --------------------------------------------------------------------------------------------------------------------

extern "C" int exl2_embed_scale(const void* table, const int* ids, float* x32, void* xh, int dtype, int rows, int width, int vocab,
                                float scale, void* stream)
{
    EXL2_REQUIRE(table && ids && x32, "embed_scale: null operand");
    EXL2_REQUIRE(dtype == 0 || dtype == 1, "embed_scale: dtype must be 0 (bfloat16) or 1 (float32)");
    if (rows <= 0) return EXL2_OK;
    if (dtype == 0) LAUNCH(embed_scale_kernel<u16>, dim3(rows), dim3(256), 0, stream, (const u16*)table, ids, x32, (u16*)xh, width, vocab, scale);
    else LAUNCH(embed_scale_kernel<float>, dim3(rows), dim3(256), 0, stream, (const float*)table, ids, x32, (float*)xh, width, vocab, scale);
    HIP_TRY(hipGetLastError());
    return EXL2_OK;
}

extern "C" int exl2_rms_rows(const float* x, int ldx, const void* w, int one_plus, void* y, int ldy, int y_f32, const int* row_idx,
                             int dtype, int rows, int dim, float eps, void* stream)
{
    EXL2_REQUIRE(x && w && y, "rms_rows: null operand");
    EXL2_REQUIRE(dtype == 0 || dtype == 1, "rms_rows: dtype must be 0 (bfloat16) or 1 (float32)");
    EXL2_REQUIRE(dim > 0 && ldx >= dim && ldy >= dim, "rms_rows: bad shape");
    if (rows <= 0) return EXL2_OK;
    if (dtype == 0) LAUNCH(rms_rows_kernel<u16>, dim3(rows), dim3(256), 0, stream, x, ldx, (const u16*)w, one_plus, y, ldy, y_f32, row_idx, dim, eps);
    else LAUNCH(rms_rows_kernel<float>, dim3(rows), dim3(256), 0, stream, x, ldx, (const float*)w, one_plus, y, ldy, 1, row_idx, dim, eps);
    HIP_TRY(hipGetLastError());
    return EXL2_OK;
}

extern "C" int exl2_post_norm(float* x, void* xh, const float* y, const void* w, int dtype, int rows, int width, float alpha, float eps,
                              const float* moe_y, const int* moe_ids, const float* moe_w, int top, int n_real, void* stream)
{
    EXL2_REQUIRE(x && w, "post_norm: null operand");
    EXL2_REQUIRE(dtype == 0 || dtype == 1, "post_norm: dtype must be 0 (bfloat16) or 1 (float32)");
    EXL2_REQUIRE(y || (moe_ids && moe_w && top > 0), "post_norm: neither a sublayer output nor an expert mixture");
    EXL2_REQUIRE(y || moe_y || n_real == 0, "post_norm: expert outputs missing");
    EXL2_REQUIRE(width > 0 && (size_t)width * 4 <= 160 * 1024 - 64, "post_norm: row of %d values does not fit the LDS", width);
    if (rows <= 0) return EXL2_OK;
    PostNormArgs a;
    a.x = x; a.xh = xh; a.y = y; a.w = w; a.width = width; a.alpha = alpha; a.eps = eps;
    a.moe_y = moe_y; a.moe_ids = moe_ids; a.moe_w = moe_w; a.top = top; a.n_real = n_real;
    const size_t smem = (size_t)width * 4;
    if (smem > 48 * 1024)
    {
        static bool attr_done[EXL2_MAX_DEVICES];
        if (exl2_first_on_device(attr_done))
        {
            (void)hipFuncSetAttribute((const void*)post_norm_kernel<u16>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
            (void)hipFuncSetAttribute((const void*)post_norm_kernel<float>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        }
    }
    if (dtype == 0) LAUNCH(post_norm_kernel<u16>, dim3(rows), dim3(256), smem, stream, a);
    else LAUNCH(post_norm_kernel<float>, dim3(rows), dim3(256), smem, stream, a);
    HIP_TRY(hipGetLastError());
    return EXL2_OK;
}

extern "C" int exl2_add_layer_norm(float* x, const float* y, const void* w, const void* b, void* out, int out_f32, const int* row_idx,
                                   int dtype, int rows, int width, float eps, void* stream)
{
    EXL2_REQUIRE(x, "add_layer_norm: null stream");
    EXL2_REQUIRE(dtype == 0 || dtype == 1, "add_layer_norm: dtype must be 0 (bfloat16) or 1 (float32)");
    EXL2_REQUIRE(!w || out, "add_layer_norm: a norm needs an output");
    EXL2_REQUIRE(w || y, "add_layer_norm: neither an addition nor a norm");
    EXL2_REQUIRE(!(row_idx && y), "add_layer_norm: gathered rows take no addition");
    EXL2_REQUIRE(width > 0 && (size_t)width * 4 <= 160 * 1024 - 64, "add_layer_norm: row of %d values does not fit the LDS", width);
    if (rows <= 0) return EXL2_OK;
    LayerNormArgs a;
    a.x = x; a.y = y; a.w = w; a.b = b; a.out = out; a.out_f32 = out_f32 || dtype == 1; a.row_idx = row_idx; a.width = width; a.eps = eps;
    const bool aligned = ((uintptr_t)x % 16) == 0 && (!y || ((uintptr_t)y % 16) == 0) && (!w || ((uintptr_t)w % 16) == 0)
                         && (!b || ((uintptr_t)b % 16) == 0) && (!out || ((uintptr_t)out % 16) == 0);
    if (width % 4 == 0 && width <= 256 * 4 * LN_VPT && aligned)
    {
        if (dtype == 0) LAUNCH(add_layer_norm_vec_kernel<u16>, dim3(rows), dim3(256), 0, stream, a);
        else LAUNCH(add_layer_norm_vec_kernel<float>, dim3(rows), dim3(256), 0, stream, a);
        HIP_TRY(hipGetLastError());
        return EXL2_OK;
    }
    const size_t smem = (size_t)width * 4;
    if (smem > 48 * 1024)
    {
        static bool attr_done[EXL2_MAX_DEVICES];
        if (exl2_first_on_device(attr_done))
        {
            (void)hipFuncSetAttribute((const void*)add_layer_norm_kernel<u16>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
            (void)hipFuncSetAttribute((const void*)add_layer_norm_kernel<float>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        }
    }
    if (dtype == 0) LAUNCH(add_layer_norm_kernel<u16>, dim3(rows), dim3(256), smem, stream, a);
    else LAUNCH(add_layer_norm_kernel<float>, dim3(rows), dim3(256), smem, stream, a);
    HIP_TRY(hipGetLastError());
    return EXL2_OK;
}

static int moe_route_any(const float* logits, const float* correction, int* ids, float* wts, int rows, int n_total, int top,
                         float scale, int n_real, int* grp_count, int* grp_offset, int* grp_rows, int sigmoid_scores, int shared_slot,
                         void* stream);

extern "C" int exl2_moe_route_scored(const float* logits, const float* correction, int* ids, float* wts, int rows, int n_total, int top,
                                     float scale, int n_real, int* grp_count, int* grp_offset, int* grp_rows, void* stream)
{
    return moe_route_any(logits, correction, ids, wts, rows, n_total, top, scale, n_real, grp_count, grp_offset, grp_rows, 0, 0, stream);
}

extern "C" int exl2_moe_route_sigmoid(const float* logits, int* ids, float* wts, int rows, int n_total, int top, float scale,
                                      int shared_slot, int* grp_count, int* grp_offset, int* grp_rows, void* stream)
{
    return moe_route_any(logits, nullptr, ids, wts, rows, n_total, top, scale, n_total + (shared_slot ? 1 : 0), grp_count, grp_offset,
                         grp_rows, 1, shared_slot, stream);
}

static int moe_route_any(const float* logits, const float* correction, int* ids, float* wts, int rows, int n_total, int top,
                         float scale, int n_real, int* grp_count, int* grp_offset, int* grp_rows, int sigmoid_scores, int shared_slot,
                         void* stream)
{
    const int ld = top + (shared_slot ? 1 : 0);                  // values per row of ids / wts
    EXL2_REQUIRE(logits && ids && wts, "moe_route_scored: null operand");
    EXL2_REQUIRE(n_total > 0 && n_total <= 64 * ROUTE_MAX_PER_LANE, "moe_route_scored: %d experts (at most %d)", n_total, 64 * ROUTE_MAX_PER_LANE);
    EXL2_REQUIRE(top > 0 && top <= 64 && top <= n_total, "moe_route_scored: top %d of %d", top, n_total);
    EXL2_REQUIRE(n_real >= 0 && n_real <= n_total + (shared_slot ? 1 : 0), "moe_route_scored: %d experts with weights of %d", n_real, n_total);
    if (rows <= 0) return EXL2_OK;
    LAUNCH(moe_route_kernel, dim3(rows), dim3(64), 0, stream, logits, correction, ids, wts, n_total, top, scale, sigmoid_scores, ld,
           shared_slot ? n_total : -1);
    if (grp_count)
    {
        EXL2_REQUIRE(grp_offset && grp_rows, "moe_route_scored: grouped lists need offsets and rows");
        if (n_real > 0)
        {
            LAUNCH(moe_count_kernel, dim3(n_real), dim3(256), 0, stream, (const int*)ids, rows * ld, grp_count);
            LAUNCH(moe_fill_kernel, dim3(n_real), dim3(64), 0, stream, (const int*)ids, rows * ld, (const int*)grp_count, grp_offset, grp_rows);
        }
    }
    HIP_TRY(hipGetLastError());
    return EXL2_OK;
}

extern "C" int exl2_add_rms_shift(float* x, const float* y, const float* moe_y, int top, float gain, float eps, const void* shift,
                                  float* prev, float* hn, void* out, int out_f32, const int* row_seq, const int* row_pos,
                                  const int* row_idx, const int* span_row0, const int* span_rows, int spans, int max_span_rows,
                                  int dtype, int rows, int width, void* stream)
{
    EXL2_REQUIRE(x, "add_rms_shift: null stream");
    EXL2_REQUIRE(dtype == 0 || dtype == 1, "add_rms_shift: dtype must be 0 (bfloat16) or 1 (float32)");
    EXL2_REQUIRE(!moe_y || top > 0, "add_rms_shift: expert outputs need their count per row");
    EXL2_REQUIRE(out || y || moe_y, "add_rms_shift: neither an addition nor a norm");
    EXL2_REQUIRE(!(row_idx && (y || moe_y || shift)), "add_rms_shift: gathered rows take no addition and no shift");
    EXL2_REQUIRE(!shift || (out && prev && row_seq && row_pos && span_row0 && span_rows && spans > 0 && max_span_rows > 0),
                 "add_rms_shift: a shift needs an output, the slots' rows and the step's spans");
    EXL2_REQUIRE(!shift || max_span_rows == 1 || hn, "add_rms_shift: spans of several rows need the buffer of normed rows");
    EXL2_REQUIRE(width > 0 && (size_t)width * 4 <= 160 * 1024 - 64, "add_rms_shift: row of %d values does not fit the LDS", width);
    if (rows <= 0) return EXL2_OK;
    RmsShiftArgs a;
    a.x = x; a.y = y; a.moe_y = moe_y; a.top = top; a.hn = shift && max_span_rows > 1 ? hn : nullptr; a.out = out;
    a.out_f32 = out_f32 || dtype == 1; a.shift = shift; a.prev = prev; a.row_seq = row_seq; a.row_pos = row_pos; a.row_idx = row_idx;
    a.width = width; a.gain = gain; a.eps = eps; a.fused = shift && max_span_rows == 1;
    const size_t smem = (size_t)width * 4;
    if (smem > 48 * 1024)
    {
        static bool attr_done[EXL2_MAX_DEVICES];
        if (exl2_first_on_device(attr_done))
        {
            (void)hipFuncSetAttribute((const void*)add_rms_shift_kernel<u16>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
            (void)hipFuncSetAttribute((const void*)add_rms_shift_kernel<float>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        }
    }
    if (dtype == 0) LAUNCH(add_rms_shift_kernel<u16>, dim3(rows), dim3(256), smem, stream, a);
    else LAUNCH(add_rms_shift_kernel<float>, dim3(rows), dim3(256), smem, stream, a);
    if (shift && !a.fused)
    {
        const dim3 grid(rows, (width + 255) / 256);
        if (dtype == 0) LAUNCH(token_shift_kernel<u16>, grid, dim3(256), 0, stream, a);
        else LAUNCH(token_shift_kernel<float>, grid, dim3(256), 0, stream, a);
        LAUNCH(span_last_row_kernel, dim3(spans, (width + 255) / 256), dim3(256), 0, stream, (const float*)hn, width, prev, width, span_row0,
               span_rows, row_seq);
    }
    HIP_TRY(hipGetLastError());
    return EXL2_OK;
}

extern "C" int exl2_span_last_rows(const float* src, int ld, float* slot_rows, int width, const int* span_row0, const int* span_rows,
                                   int spans, const int* row_seq, void* stream)
{
    EXL2_REQUIRE(src && slot_rows && span_row0 && span_rows && row_seq && width > 0 && ld >= width, "span_last_rows: bad operand");
    if (spans <= 0) return EXL2_OK;
    LAUNCH(span_last_row_kernel, dim3(spans, (width + 255) / 256), dim3(256), 0, stream, src, ld, slot_rows, width, span_row0, span_rows, row_seq);
    HIP_TRY(hipGetLastError());
    return EXL2_OK;
}

extern "C" int exl2_sandwich_norm(float* x, const float* y, float ya, const float* y2, float yb, const float* moe_y, int top,
                                  const void* w_out, float mult, const void* w_in, void* out, int out_f32, const int* row_idx,
                                  const void* conv_w, float* tail, const int* row_seq, const int* row_pos, int taps, int dtype, int rows,
                                  int width, int groups, float eps, void* stream)
{
    EXL2_REQUIRE(x, "sandwich_norm: null stream");
    EXL2_REQUIRE(dtype == 0 || dtype == 1, "sandwich_norm: dtype must be 0 (bfloat16) or 1 (float32)");
    const bool pending = y || y2 || moe_y;
    EXL2_REQUIRE(!pending || w_out, "sandwich_norm: a sublayer's output needs the weight of the norm behind it");
    EXL2_REQUIRE(!moe_y || top > 0, "sandwich_norm: expert outputs need their count per row");
    EXL2_REQUIRE(pending || out, "sandwich_norm: neither an addition nor a norm");
    EXL2_REQUIRE(!out || w_in, "sandwich_norm: an output needs the weight of the norm in front of it");
    EXL2_REQUIRE(!(row_idx && (pending || conv_w)), "sandwich_norm: gathered rows take no addition and no convolution");
    EXL2_REQUIRE(!conv_w || (out && taps >= 1 && (taps == 1 || (tail && row_seq && row_pos))), "sandwich_norm: the convolution needs an output, the slots' tails and the rows' places");
    EXL2_REQUIRE(groups > 0 && width > 0 && width % groups == 0, "sandwich_norm: %d values in %d groups", width, groups);
    EXL2_REQUIRE((size_t)width * 4 <= 160 * 1024 - 64, "sandwich_norm: row of %d values does not fit the LDS", width);
    if (rows <= 0) return EXL2_OK;
    SandwichArgs a;
    a.x = x; a.y = y; a.ya = ya; a.y2 = y2; a.yb = yb; a.moe_y = moe_y; a.top = top; a.w_out = w_out; a.mult = mult; a.w_in = w_in;
    a.out = out; a.out_f32 = out_f32 || dtype == 1; a.row_idx = row_idx; a.conv_w = conv_w; a.tail = tail; a.row_seq = row_seq;
    a.row_pos = row_pos; a.taps = taps; a.width = width; a.groups = groups; a.eps = eps;
    const auto al16 = [](const void* p) { return ((uintptr_t)p % 16) == 0; };
    const bool vec = width % 4 == 0 && width <= 256 * 4 * 4 && (width / groups) % 4 == 0 && groups <= SW_MAX_GROUPS && taps <= SW_MAX_TAPS
                     && al16(x) && al16(y) && al16(y2) && al16(moe_y) && al16(w_out) && al16(w_in) && al16(out) && al16(tail) && al16(conv_w);
    if (vec)
    {
        const int nc = width <= 1024 ? 1 : width <= 2048 ? 2 : 4;
        if (dtype == 0)
        {
            if (nc == 1) LAUNCH((sandwich_norm_vec_kernel<u16, 1>), dim3(rows), dim3(256), 0, stream, a);
            else if (nc == 2) LAUNCH((sandwich_norm_vec_kernel<u16, 2>), dim3(rows), dim3(256), 0, stream, a);
            else LAUNCH((sandwich_norm_vec_kernel<u16, 4>), dim3(rows), dim3(256), 0, stream, a);
        }
        else
        {
            if (nc == 1) LAUNCH((sandwich_norm_vec_kernel<float, 1>), dim3(rows), dim3(256), 0, stream, a);
            else if (nc == 2) LAUNCH((sandwich_norm_vec_kernel<float, 2>), dim3(rows), dim3(256), 0, stream, a);
            else LAUNCH((sandwich_norm_vec_kernel<float, 4>), dim3(rows), dim3(256), 0, stream, a);
        }
        HIP_TRY(hipGetLastError());
        return EXL2_OK;
    }
    const size_t smem = (size_t)width * 4;
    if (smem > 48 * 1024)
    {
        static bool attr_done[EXL2_MAX_DEVICES];
        if (exl2_first_on_device(attr_done))
        {
            (void)hipFuncSetAttribute((const void*)sandwich_norm_kernel<u16>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
            (void)hipFuncSetAttribute((const void*)sandwich_norm_kernel<float>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        }
    }
    if (dtype == 0) LAUNCH(sandwich_norm_kernel<u16>, dim3(rows), dim3(256), smem, stream, a);
    else LAUNCH(sandwich_norm_kernel<float>, dim3(rows), dim3(256), smem, stream, a);
    HIP_TRY(hipGetLastError());
    return EXL2_OK;
}

extern "C" int exl2_embed_pair(const void* table, const void* pair, const void* w, const int* ids, int* prev_tok, const int* row_seq,
                               const int* row_pos, const int* span_row0, const int* span_rows, int spans, int max_span_rows, float* x,
                               int dtype, int rows, int width, int vocab, int buckets, int mul_prev, int mul_cur, float scale, int groups,
                               float eps, void* stream)
{
    EXL2_REQUIRE(table && ids && x && row_seq && row_pos, "embed_pair: null operand");
    EXL2_REQUIRE(dtype == 0 || dtype == 1, "embed_pair: dtype must be 0 (bfloat16) or 1 (float32)");
    EXL2_REQUIRE(!pair || (prev_tok && buckets > 0 && span_row0 && span_rows && spans > 0 && max_span_rows > 0),
                 "embed_pair: the pair table needs its size, the slots' tokens and the step's spans");
    EXL2_REQUIRE(width > 0 && vocab > 0 && (!w || (groups > 0 && width % groups == 0)), "embed_pair: bad shape");
    EXL2_REQUIRE((size_t)width * 4 <= 160 * 1024 - 64, "embed_pair: row of %d values does not fit the LDS", width);
    if (rows <= 0) return EXL2_OK;
    EmbedPairArgs a;
    a.table = table; a.pair = pair; a.w = w; a.ids = ids; a.prev_tok = prev_tok; a.row_seq = row_seq; a.row_pos = row_pos; a.x = x;
    a.width = width; a.vocab = vocab; a.buckets = buckets; a.mul_prev = mul_prev; a.mul_cur = mul_cur; a.groups = groups > 0 ? groups : 1;
    a.fused = pair && max_span_rows == 1; a.scale = scale; a.eps = eps;
    const size_t smem = (size_t)width * 4;
    if (smem > 48 * 1024)
    {
        static bool attr_done[EXL2_MAX_DEVICES];
        if (exl2_first_on_device(attr_done))
        {
            (void)hipFuncSetAttribute((const void*)embed_pair_kernel<u16>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
            (void)hipFuncSetAttribute((const void*)embed_pair_kernel<float>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        }
    }
    if (dtype == 0) LAUNCH(embed_pair_kernel<u16>, dim3(rows), dim3(256), smem, stream, a);
    else LAUNCH(embed_pair_kernel<float>, dim3(rows), dim3(256), smem, stream, a);
    if (pair && !a.fused) LAUNCH(token_state_kernel, dim3((spans + 63) / 64), dim3(64), 0, stream, ids, prev_tok, span_row0, span_rows, row_seq, spans, vocab);
    HIP_TRY(hipGetLastError());
    return EXL2_OK;
}
