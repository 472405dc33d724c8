// window_attn.hip -- grouped-head softmax attention over a paged cache with a sliding window, POOLED blocks behind the window, a
// per-head sink in the softmax denominator and rotated values, for gfx950, + its C ABI.
//
// A position p of a sequence attends to
//   * the tokens j with 0 <= p - j < window, and
//   * one pooled key / value for every block of `pool` consecutive tokens [b pool, b pool + pool) that lies wholly in front of the
//     window (b pool + pool - 1 <= p - window): the mean of the block's cached keys and the mean of its cached values,
// in one softmax whose denominator also holds exp(sink[head]).  Tokens that have left the window and whose block is not complete
// behind it are not seen.  Keys and queries are rotated over their first rot_dims values, values over all of theirs (the head's
// output is turned back by its own position), so the cache holds rotated keys AND rotated values.
//
// Cache: keys [pages, page, kv_heads, dim], values [pages, page, kv_heads, vdim] reached through a per-sequence block table;
// pooled rows [pages, ceil(page / pool), kv_heads, dim | vdim]: block b's row sits in the page of its first token at index
// ((b pool) % page) / pool (consecutive blocks that start in one page are `pool` tokens apart, so the indices are distinct).
// Rows of a step are a flat list (row r = position row_pos[r] of sequence row_seq[r]); a row's result depends only on its own
// (sequence, position).  Scores, softmax, sums, angles and rotations are fp32.
// Rotary layouts: halves (value i pairs with i + n / 2) or interleaved (2i with 2i + 1); angle p * freq[i], cos and sin times `amp`.
// Variants a design may ask for (the *_ex entry points): a CHUNKED mask instead of the window -- p sees j <= p with
// floor(j / chunk) == floor(p / chunk), chunks counted from the sequence's start --, a soft cap  c tanh(s / c)  on the scores, ONE gate
// value per head instead of one per output value, and rows that bring queries only (a layer that attends over another layer's
// cached keys and values).
#include "hw.h"
#include "errors.h"
#include <stdint.h>

template <typename T> DEV float wa_ld(const T* p);
template <> DEV float wa_ld<u16>(const u16* p) { return bf16_to_f32(*p); }
template <> DEV float wa_ld<float>(const float* p) { return *p; }
template <typename T> DEV void wa_st(T* p, float v);
template <> DEV void wa_st<u16>(u16* p, float v) { *p = f32_to_bf16(v); }
template <> DEV void wa_st<float>(float* p, float v) { *p = v; }

DEV float wa_block_sum(float v, float* part)
{
    v = wave_allreduce_add(v);
    block_sync();
    if (lane_id() == 0) part[wave_id()] = v;
    block_sync();
    return part[0] + part[1] + part[2] + part[3];
}
DEV float wa_block_max(float v, float* part)
{
    v = wave_allreduce_max(v);
    block_sync();
    if (lane_id() == 0) part[wave_id()] = v;
    block_sync();
    return fmaxf(fmaxf(part[0], part[1]), fmaxf(part[2], part[3]));
}

// the pair partner layout: element indices (a, b) of pair i among n rotated values
DEV void wa_pair(int i, int n, int interleaved, int& ia, int& ib)
{
    if (interleaved) { ia = 2 * i; ib = 2 * i + 1; } else { ia = i; ib = i + n / 2; }
}

// ---- new rows: rotate q (scaled per head) / k / v, append k and v to the cache ---------------------------------------------------

struct RotAppendArgs
{
    const float* f; int ld;                  // [rows, ld] fp32: q at q_off (H x dim), k at k_off (G x dim), v at v_off (G x vdim)
    int q_off, k_off, v_off;
    void* q_out;                             // [rows, H x dim] operand dtype: rotated, times q_scale[h]
    const float* q_scale;                    // [H]
    void* k_cache; void* v_cache;
    const float* freq; float amp; int rot_dims;          // q / k rotation
    const float* vfreq; int v_rot;           // value rotation over all vdim (0: values are stored as they are)
    int interleaved;
    const int* row_seq; const int* row_pos; const int* block_table; int bt_stride, page;
    int H, G, dim, vdim;
};

// grid (rows): the row's H query heads, G key heads and G value heads
template <typename T>
KERNEL void __launch_bounds__(256) rot_append_kernel(const RotAppendArgs a)
{
    const int r = bid_x(), t = tid();
    const float* src = a.f + (long long)r * a.ld;
    const int pos = a.row_pos[r];
    const float fpos = (float)pos;
    const int pg = a.block_table[(long long)a.row_seq[r] * a.bt_stride + pos / a.page];
    const long long slot = (long long)pg * a.page + pos % a.page;
    const int half = a.rot_dims / 2;
    // queries and keys: (H + G) heads of `dim` values; pairs first, then the values past rot_dims
    const int per = half + (a.dim - a.rot_dims);
    const int kv_heads = a.k_cache ? a.G : 0;                    // no cache: the rows bring queries only
    for (int i = t; i < (a.H + kv_heads) * per; i += 256)
    {
        const int hd = i / per, e = i % per;
        const bool is_q = hd < a.H;
        const float* s = is_q ? src + a.q_off + hd * a.dim : src + a.k_off + (hd - a.H) * a.dim;
        T* d = is_q ? (T*)a.q_out + ((long long)r * a.H + hd) * a.dim : (T*)a.k_cache + (slot * a.G + (hd - a.H)) * a.dim;
        const float mul = is_q ? a.q_scale[hd] : 1.0f;
        if (e < half)
        {
            int ia, ib;
            wa_pair(e, a.rot_dims, a.interleaved, ia, ib);
            const float ang = fpos * a.freq[e];
            const float c = cosf(ang) * a.amp, sn = sinf(ang) * a.amp;
            const float u = s[ia], v = s[ib];
            wa_st<T>(d + ia, (u * c - v * sn) * mul);
            wa_st<T>(d + ib, (v * c + u * sn) * mul);
        }
        else
        {
            const int j = a.rot_dims + (e - half);
            wa_st<T>(d + j, s[j] * mul);
        }
    }
    const int vhalf = a.vdim / 2;
    if (!a.k_cache) return;
    for (int i = t; i < a.G * vhalf; i += 256)
    {
        const int g = i / vhalf, e = i % vhalf;
        const float* s = src + a.v_off + g * a.vdim;
        T* d = (T*)a.v_cache + (slot * a.G + g) * a.vdim;
        int ia, ib;
        wa_pair(e, a.vdim, a.interleaved, ia, ib);
        const float u = s[ia], v = s[ib];
        if (a.v_rot)
        {
            const float ang = fpos * a.vfreq[e];
            const float c = cosf(ang), sn = sinf(ang);
            wa_st<T>(d + ia, u * c - v * sn);
            wa_st<T>(d + ib, v * c + u * sn);
        }
        else { wa_st<T>(d + ia, u); wa_st<T>(d + ib, v); }
    }
    if ((a.vdim & 1) && t == 0)
        for (int g = 0; g < a.G; g++)
            wa_st<T>((T*)a.v_cache + (slot * a.G + g) * a.vdim + a.vdim - 1, src[a.v_off + g * a.vdim + a.vdim - 1]);
}

// ---- pooled rows ----------------------------------------------------------------------------------------------------------------

struct PoolArgs
{
    const void* k_cache; const void* v_cache; void* k_pool; void* v_pool;
    const int* row_seq; const int* row_pos; const int* block_table; int bt_stride, page, pool, per_page;
    int kw, vw;                              // values per token: G x dim, G x vdim
};

// 16 bytes of T as floats
template <typename T> struct WaVec;
template <> struct WaVec<u16>
{
    static constexpr int N = 8;
    static DEV void load(const u16* p, float* f)
    {
        const u32x4 v = *(const u32x4*)p;
        #pragma unroll
        for (int i = 0; i < 4; i++) { f[2 * i] = as_f32(v[i] << 16); f[2 * i + 1] = as_f32(v[i] & 0xffff0000u); }
    }
};
template <> struct WaVec<float>
{
    static constexpr int N = 4;
    static DEV void load(const float* p, float* f)
    {
        const f32x4 v = *(const f32x4*)p;
        #pragma unroll
        for (int i = 0; i < 4; i++) f[i] = v[i];
    }
};

// grid (rows, pieces): a row whose position completes a block (pos % pool == pool - 1) writes that block's mean key and value row,
// read back from the cache as it holds them; other rows leave at once.  VEC: a workgroup takes 64 16-byte pieces of the
// [keys | values] row, wave w sums the block's tokens w, w + 4, .. and the four partial sums meet in LDS; otherwise one value per
// thread over all tokens (sizes that are not whole 16-byte pieces).
template <typename T, bool VEC>
KERNEL void __launch_bounds__(256) pool_blocks_kernel(const PoolArgs a)
{
    constexpr int VN = WaVec<T>::N;
    SHARED float part[4][64][VN];
    const int r = bid_x(), t = tid();
    const int pos = a.row_pos[r];
    if (pos % a.pool != a.pool - 1) return;
    const int* bt = a.block_table + (long long)a.row_seq[r] * a.bt_stride;
    const int p0 = pos - (a.pool - 1);
    const long long dst = (long long)bt[p0 / a.page] * a.per_page + (p0 % a.page) / a.pool;
    const float inv = 1.0f / (float)a.pool;
    if (VEC)
    {
        const int w = wave_id(), lane = lane_id();
        const int piece = bid_y() * 64 + lane, e0 = piece * VN;
        const bool live = e0 < a.kw + a.vw;
        const bool is_k = e0 < a.kw;
        const int e = is_k ? e0 : e0 - a.kw, wd = is_k ? a.kw : a.vw;
        const T* c = (const T*)(is_k ? a.k_cache : a.v_cache);
        float acc[VN];
        #pragma unroll
        for (int i = 0; i < VN; i++) acc[i] = 0.0f;
        if (live)
            for (int j = p0 + w; j <= pos; j += 4)
            {
                float f[VN];
                WaVec<T>::load(c + ((long long)bt[j / a.page] * a.page + j % a.page) * wd + e, f);
                #pragma unroll
                for (int i = 0; i < VN; i++) acc[i] += f[i];
            }
        #pragma unroll
        for (int i = 0; i < VN; i++) part[w][lane][i] = acc[i];
        block_sync();
        if (w == 0 && live)
        {
            T* d = (T*)(is_k ? a.k_pool : a.v_pool) + dst * wd + e;
            #pragma unroll
            for (int i = 0; i < VN; i++) wa_st<T>(d + i, (part[0][lane][i] + part[1][lane][i] + part[2][lane][i] + part[3][lane][i]) * inv);
        }
        return;
    }
    for (int i = t; i < a.kw + a.vw; i += 256)
    {
        const bool is_k = i < a.kw;
        const int e = is_k ? i : i - a.kw, w = is_k ? a.kw : a.vw;
        const T* c = (const T*)(is_k ? a.k_cache : a.v_cache);
        float s = 0.0f;
        for (int j = p0; j <= pos; j++) s += wa_ld<T>(c + ((long long)bt[j / a.page] * a.page + j % a.page) * w + e);
        wa_st<T>((T*)(is_k ? a.k_pool : a.v_pool) + dst * w + e, s * inv);
    }
}

// ---- attention --------------------------------------------------------------------------------------------------------------------

struct WinAttnArgs
{
    const void* q;                           // [rows, H, dim] rotated, scaled
    const void* k_cache; const void* v_cache; const void* k_pool; const void* v_pool;
    const float* sink;                       // [H] (nullable: no sink)
    const float* gate; int ldg;              // fp32 [rows, ldg], value e of head h at h * vdim + e: the output is multiplied by its sigmoid (nullable)
    const float* vfreq; int v_rot, interleaved;
    const int* row_seq; const int* row_pos; const int* block_table; int bt_stride, page, pool, per_page;
    void* out;                               // [rows, H, vdim]
    int H, G, dim, vdim, window;
    int page_shift, pool_shift;              // log2 of page / pool where they are powers of two, else -1 (tile kernels: no divisions)
    int chunk;                               // > 0: chunked mask (the window is not used, no pooled blocks)
    float softcap;                           // > 0: score <- softcap * tanh(score / softcap)
    int gate_head;                           // gate holds one value per head (at h) instead of one per output value (at h * vdim + e)
};

// first token position `pos` sees (window form: may be negative)
DEV int wa_first_key(int pos, int window, int chunk) { return chunk > 0 ? pos - pos % chunk : pos - window + 1; }
DEV float wa_soft_cap(float s, float cap) { return cap > 0.0f ? cap * tanhf(s / cap) : s; }

DEV int wa_div(int x, int d, int shift) { return shift >= 0 ? x >> shift : x / d; }
DEV int wa_mod(int x, int d, int shift) { return shift >= 0 ? x & (d - 1) : x % d; }

#define WA_MAX_V_PER_THREAD 4

// number of pooled blocks position `pos` sees
DEV int wa_blocks_seen(int pos, int window, int pool)
{
    const int behind = pos - window + 1;     // tokens in front of the window
    return pool > 0 && behind > 0 ? behind / pool : 0;
}

// Workgroup = one (row, head); general and fp32 form.  The key list is [pooled blocks | window tokens], taken 256 at a time:
// thread t scores entry t of the chunk, the chunk joins the running softmax (which starts from the sink: maximum = sink, sum = 1),
// then thread t owns values t, t + 256, .. of the weighted sum.  The output is turned back by the row's position and gated.
template <typename T>
KERNEL void __launch_bounds__(256) window_attn_kernel(const WinAttnArgs a)
{
    DYN_SMEM(smem);
    SHARED float part[4];
    SHARED float prob[256];
    SHARED long long voff[256];
    float* qv = (float*)smem;                                // [dim]
    float* ov = qv + a.dim;                                  // [vdim]
    const int r = bid_x(), h = bid_y(), t = tid();
    const int g = h / (a.H / a.G);
    const int pos = a.row_pos[r];
    const int* bt = a.block_table + (long long)a.row_seq[r] * a.bt_stride;
    const T* qr = (const T*)a.q + ((long long)r * a.H + h) * a.dim;
    for (int i = t; i < a.dim; i += 256) qv[i] = wa_ld<T>(qr + i);
    block_sync();
    const int nb = wa_blocks_seen(pos, a.window, a.pool);
    const int j_lo = max(0, wa_first_key(pos, a.window, a.chunk));
    const int nkeys = nb + (pos - j_lo + 1);
    float m_run = a.sink ? a.sink[h] : -INFINITY, l_run = a.sink ? 1.0f : 0.0f;
    float acc[WA_MAX_V_PER_THREAD];
    #pragma unroll
    for (int e = 0; e < WA_MAX_V_PER_THREAD; e++) acc[e] = 0.0f;
    for (int c0 = 0; c0 < nkeys; c0 += 256)
    {
        const int nc = min(256, nkeys - c0);
        float s = -INFINITY;
        if (t < nc)
        {
            const int e = c0 + t;
            const T* kr;
            if (e < nb)
            {
                const int p0 = e * a.pool;
                const long long row = (long long)bt[p0 / a.page] * a.per_page + (p0 % a.page) / a.pool;
                kr = (const T*)a.k_pool + (row * a.G + g) * a.dim;
                voff[t] = -1 - (row * a.G + g) * (long long)a.vdim;              // negative: a pooled row
            }
            else
            {
                const int j = j_lo + (e - nb);
                const long long row = (long long)bt[j / a.page] * a.page + j % a.page;
                kr = (const T*)a.k_cache + (row * a.G + g) * a.dim;
                voff[t] = (row * a.G + g) * (long long)a.vdim;
            }
            float d = 0.0f;
            for (int i = 0; i < a.dim; i++) d = fmaf(qv[i], wa_ld<T>(kr + i), d);
            s = wa_soft_cap(d, a.softcap);
        }
        const float m_new = fmaxf(m_run, wa_block_max(s, part));
        const float p = t < nc ? expf(s - m_new) : 0.0f;
        prob[t] = p;
        const float corr = expf(m_run - m_new);
        l_run = l_run * corr + wa_block_sum(p, part);        // (its barriers also publish prob and voff)
        m_run = m_new;
        #pragma unroll
        for (int e = 0; e < WA_MAX_V_PER_THREAD; e++)
        {
            const int i = t + 256 * e;
            if (i >= a.vdim) break;
            float o = acc[e] * corr;
            for (int jj = 0; jj < nc; jj++)
            {
                const long long off = voff[jj];
                const float v = off >= 0 ? wa_ld<T>((const T*)a.v_cache + off + i) : wa_ld<T>((const T*)a.v_pool + (-1 - off) + i);
                o = fmaf(prob[jj], v, o);
            }
            acc[e] = o;
        }
        block_sync();                                        // prob / voff are rewritten by the next chunk
    }
    #pragma unroll
    for (int e = 0; e < WA_MAX_V_PER_THREAD; e++)
    {
        const int i = t + 256 * e;
        if (i < a.vdim) ov[i] = acc[e] / l_run;
    }
    block_sync();
    T* out = (T*)a.out + ((long long)r * a.H + h) * a.vdim;
    const float* gt = a.gate && !a.gate_head ? a.gate + (long long)r * a.ldg + h * a.vdim : nullptr;
    const float hg = a.gate && a.gate_head ? 1.0f / (1.0f + expf(-a.gate[(long long)r * a.ldg + h])) : 1.0f;
    const float fpos = (float)pos;
    const int vhalf = a.vdim / 2;
    for (int i = t; i < vhalf; i += 256)
    {
        int ia, ib;
        wa_pair(i, a.vdim, a.interleaved, ia, ib);
        float u = ov[ia], v = ov[ib];
        if (a.v_rot)
        {
            const float ang = fpos * a.vfreq[i];
            const float c = cosf(ang), sn = sinf(ang);
            const float u2 = u * c + v * sn, v2 = v * c - u * sn;           // turned by -ang
            u = u2; v = v2;
        }
        if (gt) { u *= 1.0f / (1.0f + expf(-gt[ia])); v *= 1.0f / (1.0f + expf(-gt[ib])); }
        wa_st<T>(out + ia, u * hg);
        wa_st<T>(out + ib, v * hg);
    }
    if ((a.vdim & 1) && t == 0)
    {
        float u = ov[a.vdim - 1];
        if (gt) u *= 1.0f / (1.0f + expf(-gt[a.vdim - 1]));
        wa_st<T>(out + a.vdim - 1, u * hg);
    }
}

// ---- bfloat16 on the matrix cores ---------------------------------------------------------------------------------------------------
// Workgroup = one tile of <= 64 RPW consecutive positions of one sequence x one head; wave w owns RPW blocks of 16 query rows.
// The tile's key list is [pooled blocks 0 .. NB) | tokens j_lo .. last position], NB and j_lo taken for the tile as a whole and
// masked per query row; it goes by in steps of 64 entries whose key and value rows are staged row-major in LDS (each entry's row is
// looked up through the block table -- pooled rows in the pooled tensors -- one step ahead of its loads, two steps ahead of its use).
// Scores are computed transposed, S^T = K Q^T (A = key rows from LDS, B = the wave's query rows held in registers), so that the
// accumulator layout of S^T (lane (q, g) holds keys 4g .. 4g + 3 of a 16-key block for query q) is the B-operand layout of
// O^T += V^T P^T with the 32 keys of a product taken in the order {4g .. 4g + 3 of block 0, of block 1}: probabilities stay in
// registers, and V^T's A operand comes from the row-major value tile by transposing LDS reads.  Softmax statistics per query =
// per accumulator column (running maximum starts at the sink, the sum at 1), fp32; P rounded to bfloat16 for the product.
// The epilogue turns the head's output back by the row's position, applies the gate and stores bfloat16.

struct WinMfmaArgs
{
    WinAttnArgs w;
    const int* tile_row0; const int* tile_rows;
    // decoded tokens, nsplit > 1: the steps of a row's key list are dealt to nsplit workgroups; partial results go to
    // part_o fp32 [rows, H, nsplit, vdim] (sums relative to the partial maximum) and part_ml fp32 [rows, H, nsplit, 2] (maximum, sum)
    float* part_o; float* part_ml; int nsplit;
};

#define WM_BK 64
#define WM_NEG_BIG (-1.0e30f)

DEV u32 wm_pack2(float lo, float hi) { return (u32)f32_to_bf16(lo) | ((u32)f32_to_bf16(hi) << 16); }

template <int DIM, int VDIM, int RPW>
KERNEL void __launch_bounds__(256, 2) window_attn_mfma_kernel(const WinMfmaArgs m)
{
    DYN_SMEM(smem);
    const WinAttnArgs& a = m.w;
    constexpr int KSTR = DIM + 8, VSTR = VDIM + 16;              // row strides (values): conflict-free 16-byte and transposing reads
    constexpr int KK = DIM / 32, DB = VDIM / 16, NBLK = WM_BK / 16;
    constexpr int KP = WM_BK * DIM / 8, VP = WM_BK * VDIM / 8;   // 16-byte pieces of a key / value tile
    constexpr int KPT = (KP + 255) / 256, VPT = (VP + 255) / 256;
    u16* k_lds = (u16*)smem;
    u16* v_lds = k_lds + WM_BK * KSTR;

    const int t = tid(), lane = lane_id(), wv = wave_id();
    const int qi = lane & 15, g = lane >> 4;
    const int tile_i = bid_x(), h = bid_y();
    const int kh = h / (a.H / a.G);
    const int r0 = m.tile_row0[tile_i], n_rows = m.tile_rows[tile_i];
    const int p0 = a.row_pos[r0], p_last = p0 + n_rows - 1;
    const int* bt = a.block_table + (long long)a.row_seq[r0] * a.bt_stride;
    const int NB = wa_blocks_seen(p_last, a.window, a.pool);
    const int j_lo = max(0, wa_first_key(p0, a.window, a.chunk));
    const int total = NB + (p_last - j_lo + 1);
    const int n_tiles = (total + WM_BK - 1) / WM_BK;
    const u16* kc = (const u16*)a.k_cache; const u16* vc = (const u16*)a.v_cache;
    const u16* kp = (const u16*)a.k_pool; const u16* vp = (const u16*)a.v_pool;

    // entry e of the key list -> its row in the cache (>= 0) or in the pooled tensors (-1 - row)
    auto entry_row = [&](int e) -> long long {
        e = min(e, total - 1);
        if (e < NB)
        {
            const int b0 = e * a.pool;
            return -1 - ((long long)bt[wa_div(b0, a.page, a.page_shift)] * a.per_page
                         + wa_div(wa_mod(b0, a.page, a.page_shift), a.pool, a.pool_shift));
        }
        const int j = j_lo + (e - NB);
        return (long long)bt[wa_div(j, a.page, a.page_shift)] * a.page + wa_mod(j, a.page, a.page_shift);
    };

    // this wave's RPW x 16 query rows as B operands: lane (qi, g) holds Q[row 16 n + qi][32 kk + 8 g .. + 8] of block n; every key
    // and value fragment read from LDS feeds RPW products
    int my_row[RPW], qrow[RPW], qpos[RPW], my_nb[RPW], my_lo[RPW];
    u32x4 qb[RPW][KK];
    #pragma unroll
    for (int n = 0; n < RPW; n++)
    {
        my_row[n] = (wv * RPW + n) * 16 + qi;
        qrow[n] = r0 + min(my_row[n], n_rows - 1);
        qpos[n] = p0 + min(my_row[n], n_rows - 1);
        const u16* qp = (const u16*)a.q + ((long long)qrow[n] * a.H + h) * DIM + 8 * g;
        #pragma unroll
        for (int kk = 0; kk < KK; kk++) qb[n][kk] = *(const u32x4*)(qp + 32 * kk);
        my_nb[n] = wa_blocks_seen(qpos[n], a.window, a.pool);
        my_lo[n] = wa_first_key(qpos[n], a.window, a.chunk);    // first token this query sees (may be negative)
    }
    const bool wave_live = wv * RPW * 16 < n_rows;
    // what the wave as a whole can see: blocks below wave_nb, tokens wave_lo .. wave_hi
    const int wp0 = p0 + min(wv * RPW * 16, n_rows - 1), wp1 = p0 + min(wv * RPW * 16 + RPW * 16 - 1, n_rows - 1);
    const int wave_nb = wa_blocks_seen(wp1, a.window, a.pool), wave_lo = wa_first_key(wp0, a.window, a.chunk), wave_hi = wp1;

    f32x4 ot[RPW][DB];
    float m_run[RPW], l_run[RPW];
    #pragma unroll
    for (int n = 0; n < RPW; n++)
    {
        #pragma unroll
        for (int d = 0; d < DB; d++) ot[n][d] = (f32x4){0.0f, 0.0f, 0.0f, 0.0f};
        m_run[n] = a.sink ? a.sink[h] : WM_NEG_BIG; l_run[n] = a.sink ? 1.0f : 0.0f;
    }

    long long krow[KPT], vrow[VPT];                             // rows of the NEXT step's pieces
    u32x4 kreg[KPT], vreg[VPT];
    auto lookup = [&](int step) {
        const int k0 = step * WM_BK;
        #pragma unroll
        for (int i = 0; i < KPT; i++) krow[i] = entry_row(k0 + (t + i * 256) / (DIM / 8));
        #pragma unroll
        for (int i = 0; i < VPT; i++) vrow[i] = DIM == VDIM ? krow[i] : entry_row(k0 + (t + i * 256) / (VDIM / 8));
    };
    auto fetch = [&]() {
        #pragma unroll
        for (int i = 0; i < KPT; i++)
        {
            const int c = t + i * 256;
            if (KP % 256 != 0 && c >= KP) break;
            const long long row = krow[i];
            const u16* src = row >= 0 ? kc + (row * a.G + kh) * DIM : kp + ((-1 - row) * a.G + kh) * DIM;
            kreg[i] = *(const u32x4*)(src + (c % (DIM / 8)) * 8);
        }
        #pragma unroll
        for (int i = 0; i < VPT; i++)
        {
            const int c = t + i * 256;
            if (VP % 256 != 0 && c >= VP) break;
            const long long row = vrow[i];
            const u16* src = row >= 0 ? vc + (row * a.G + kh) * VDIM : vp + ((-1 - row) * a.G + kh) * VDIM;
            vreg[i] = *(const u32x4*)(src + (c % (VDIM / 8)) * 8);
        }
    };
    auto stage = [&]() {
        #pragma unroll
        for (int i = 0; i < KPT; i++)
        {
            const int c = t + i * 256;
            if (KP % 256 != 0 && c >= KP) break;
            *(u32x4*)(k_lds + (c / (DIM / 8)) * KSTR + (c % (DIM / 8)) * 8) = kreg[i];
        }
        #pragma unroll
        for (int i = 0; i < VPT; i++)
        {
            const int c = t + i * 256;
            if (VP % 256 != 0 && c >= VP) break;
            *(u32x4*)(v_lds + (c / (VDIM / 8)) * VSTR + (c % (VDIM / 8)) * 8) = vreg[i];
        }
    };

    lookup(0);
    fetch();
    if (n_tiles > 1) lookup(1);
    for (int step = 0; step < n_tiles; step++)
    {
        block_sync();                                            // everybody is done with the previous step's tiles
        stage();
        block_sync();
        if (step + 1 < n_tiles)
        {
            fetch();                                             // in flight during the products below
            if (step + 2 < n_tiles) lookup(step + 2);
        }
        const int k0 = step * WM_BK;
        // nothing in this step for the wave's rows?
        {
            const int e_hi = min(k0 + WM_BK, total) - 1;
            bool any = false;
            if (k0 < NB) any = k0 < wave_nb;
            if (e_hi >= NB)
            {
                const int ja = j_lo + max(k0 - NB, 0), jb = j_lo + (e_hi - NB);
                any = any || (ja <= wave_hi && jb >= wave_lo);
            }
            if (!wave_live || !any) continue;
        }
        f32x4 st[RPW][NBLK];
        #pragma unroll
        for (int blk = 0; blk < NBLK; blk++)
        {
            #pragma unroll
            for (int n = 0; n < RPW; n++) st[n][blk] = (f32x4){0.0f, 0.0f, 0.0f, 0.0f};
            const u16* kf = k_lds + (16 * blk + qi) * KSTR + 8 * g;
            #pragma unroll
            for (int kk = 0; kk < KK; kk++)
            {
                const u32x4 kv = *(const u32x4*)(kf + 32 * kk);
                #pragma unroll
                for (int n = 0; n < RPW; n++) st[n][blk] = mfma_16x16x32_bf16(kv, qb[n][kk], st[n][blk]);
            }
        }
        u32x4 pb[RPW][NBLK / 2];
        float alpha[RPW];
        #pragma unroll
        for (int n = 0; n < RPW; n++)
        {
            float sc[4 * NBLK];
            float m_loc = WM_NEG_BIG;
            #pragma unroll
            for (int blk = 0; blk < NBLK; blk++)
                #pragma unroll
                for (int r = 0; r < 4; r++)
                {
                    const int e = k0 + 16 * blk + 4 * g + r;
                    const int j = j_lo + (e - NB);
                    const bool valid = e < total && (e < NB ? e < my_nb[n] : (j <= qpos[n] && j >= my_lo[n]));
                    const float v = valid ? wa_soft_cap(st[n][blk][r], a.softcap) : WM_NEG_BIG;
                    sc[blk * 4 + r] = v;
                    m_loc = fmaxf(m_loc, v);
                }
            m_loc = fmaxf(m_loc, shfl_xor_f32(m_loc, 16));
            m_loc = fmaxf(m_loc, shfl_xor_f32(m_loc, 32));
            const float m_new = fmaxf(m_run[n], m_loc);
            alpha[n] = expf(m_run[n] - m_new);
            float p_sum = 0.0f;
            #pragma unroll
            for (int e2 = 0; e2 < 2 * NBLK; e2++)
            {
                const float pa = sc[2 * e2] > 0.5f * WM_NEG_BIG ? expf(sc[2 * e2] - m_new) : 0.0f;
                const float pc = sc[2 * e2 + 1] > 0.5f * WM_NEG_BIG ? expf(sc[2 * e2 + 1] - m_new) : 0.0f;
                p_sum += pa + pc;
                pb[n][e2 / 4][e2 % 4] = wm_pack2(pa, pc);
            }
            p_sum += shfl_xor_f32(p_sum, 16);
            p_sum += shfl_xor_f32(p_sum, 32);
            l_run[n] = l_run[n] * alpha[n] + p_sum;
            m_run[n] = m_new;
        }
        // O^T = alpha O^T + V^T P^T: this lane points at value row 4 g + qi / 4, features 16 d + 4 (qi % 4) .. + 3
        const u16* vbase = v_lds + (4 * g + (qi >> 2)) * VSTR + 4 * (qi & 3);
        #pragma unroll
        for (int d = 0; d < DB; d++)
        {
            #pragma unroll
            for (int n = 0; n < RPW; n++) { ot[n][d][0] *= alpha[n]; ot[n][d][1] *= alpha[n]; ot[n][d][2] *= alpha[n]; ot[n][d][3] *= alpha[n]; }
            #pragma unroll
            for (int m2 = 0; m2 < NBLK / 2; m2++)
            {
                const f16x4 lo = lds_read_tr16_b64((const f16*)(vbase + (32 * m2) * VSTR + 16 * d));
                const f16x4 hi = lds_read_tr16_b64((const f16*)(vbase + (32 * m2 + 16) * VSTR + 16 * d));
                const u32x2 l2 = __builtin_bit_cast(u32x2, lo), h2 = __builtin_bit_cast(u32x2, hi);
                const u32x4 va = {l2[0], l2[1], h2[0], h2[1]};
                #pragma unroll
                for (int n = 0; n < RPW; n++) ot[n][d] = mfma_16x16x32_bf16(va, pb[n][m2], ot[n][d]);
            }
        }
    }

    // O^T[feature 16 d + 4 g + r][query qi] / l, turned back by the row's position, gated -> out[row][head][feature]
    #pragma unroll
    for (int n = 0; n < RPW; n++)
    {
        if (my_row[n] >= n_rows) continue;
        const float inv = l_run[n] > 0.0f ? 1.0f / l_run[n] : 0.0f;
        #pragma unroll
        for (int d = 0; d < DB; d++) { ot[n][d][0] *= inv; ot[n][d][1] *= inv; ot[n][d][2] *= inv; ot[n][d][3] *= inv; }
        if (a.v_rot)
        {
            const float fpos = (float)qpos[n];
            if (a.interleaved)
            {
                #pragma unroll
                for (int d = 0; d < DB; d++)
                    #pragma unroll
                    for (int r = 0; r < 4; r += 2)
                    {
                        const float ang = fpos * a.vfreq[(16 * d + 4 * g + r) / 2];
                        const float c = cosf(ang), sn = sinf(ang);
                        const float u = ot[n][d][r], v = ot[n][d][r + 1];
                        ot[n][d][r] = u * c + v * sn; ot[n][d][r + 1] = v * c - u * sn;
                    }
            }
            else
            {
                #pragma unroll
                for (int d = 0; d < DB / 2; d++)
                    #pragma unroll
                    for (int r = 0; r < 4; r++)
                    {
                        const float ang = fpos * a.vfreq[16 * d + 4 * g + r];
                        const float c = cosf(ang), sn = sinf(ang);
                        const float u = ot[n][d][r], v = ot[n][d + DB / 2][r];
                        ot[n][d][r] = u * c + v * sn; ot[n][d + DB / 2][r] = v * c - u * sn;
                    }
            }
        }
        u16* op = (u16*)a.out + ((long long)qrow[n] * a.H + h) * VDIM + 4 * g;
        const float* gt = a.gate && !a.gate_head ? a.gate + (long long)qrow[n] * a.ldg + h * VDIM + 4 * g : nullptr;
        const float hg = a.gate && a.gate_head ? 1.0f / (1.0f + expf(-a.gate[(long long)qrow[n] * a.ldg + h])) : 1.0f;
        #pragma unroll
        for (int d = 0; d < DB; d++)
        {
            f32x4 y = ot[n][d] * hg;
            if (gt)
            {
                const f32x4 gv = *(const f32x4*)(gt + 16 * d);
                #pragma unroll
                for (int r = 0; r < 4; r++) y[r] *= 1.0f / (1.0f + expf(-gv[r]));
            }
            *(u32x2*)(op + 16 * d) = (u32x2){wm_pack2(y[0], y[1]), wm_pack2(y[2], y[3])};
        }
    }
}

static int wa_log2_exact(int x) { int sh = 0; while ((1 << sh) < x) sh++; return x > 0 && (1 << sh) == x ? sh : -1; }

template <int DIM, int VDIM>
static void wm_launch(const WinMfmaArgs& m, int tiles, hipStream_t s)
{
    // RPW = 1.  (RPW = 2 -- tiles of 128 positions, every LDS fragment feeding two products -- was built and measured slower at
    // head size 128: 217 against 107 us at 2048 rows x 16 heads; its 233 registers left arrays in scratch memory.)
    static bool attr_done[EXL2_MAX_DEVICES];
    const size_t lds = ((size_t)WM_BK * (DIM + 8) + (size_t)WM_BK * (VDIM + 16)) * 2;
    if (exl2_first_on_device(attr_done))
        (void)hipFuncSetAttribute((const void*)window_attn_mfma_kernel<DIM, VDIM, 1>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    LAUNCH((window_attn_mfma_kernel<DIM, VDIM, 1>), dim3(tiles, m.w.H), dim3(256), lds, s, m);
}

// Decoded tokens: workgroup = one row x one key / value head.  The 16 query columns of the products are the query heads that
// share the key head (at most 16 per workgroup; blockIdx.z walks further sixteens), all at the row's position, so the key list
// [pooled blocks | window tokens] needs no mask beyond its length.  It goes by in steps of 128 entries staged by all four waves;
// wave w takes entries 32 w .. 32 w + 31 of every step with its own running (maximum, sum, O^T) -- the sink counts in wave 0 --
// and the four partial results meet in LDS at the end.  One pass over the keys serves all heads of the group.

#define WD_BK 128

template <int DIM, int VDIM>
KERNEL void __launch_bounds__(256) window_attn_decode_kernel(const WinMfmaArgs m)
{
    DYN_SMEM(smem);
    const WinAttnArgs& a = m.w;
    constexpr int KSTR = DIM + 8, VSTR = VDIM + 16;
    constexpr int KK = DIM / 32, DB = VDIM / 16;
    constexpr int KP = WD_BK * DIM / 8, VP = WD_BK * VDIM / 8;
    constexpr int KPT = (KP + 255) / 256, VPT = (VP + 255) / 256;
    u16* k_lds = (u16*)smem;
    u16* v_lds = k_lds + WD_BK * KSTR;

    const int t = tid(), lane = lane_id(), wv = wave_id();
    const int qi = lane & 15, g = lane >> 4;
    const int kh = bid_y();
    const int split = bid_z() % m.nsplit;
    const int hpg = a.H / a.G, h0 = (bid_z() / m.nsplit) * 16, nh = min(16, hpg - h0);      // this workgroup's heads: kh * hpg + h0 .. + nh
    const int r = m.tile_row0[bid_x()];
    const int pos = a.row_pos[r];
    const int* bt = a.block_table + (long long)a.row_seq[r] * a.bt_stride;
    const int NB = wa_blocks_seen(pos, a.window, a.pool);
    const int j_lo = max(0, wa_first_key(pos, a.window, a.chunk));
    const int total = NB + (pos - j_lo + 1);
    const int all_steps = (total + WD_BK - 1) / WD_BK;
    const int per_split = (all_steps + m.nsplit - 1) / m.nsplit;
    const int step_lo = split * per_split, n_steps = min(all_steps, step_lo + per_split);      // this workgroup's steps: step_lo .. n_steps
    const u16* kc = (const u16*)a.k_cache; const u16* vc = (const u16*)a.v_cache;
    const u16* kp = (const u16*)a.k_pool; const u16* vp = (const u16*)a.v_pool;
    auto entry_row = [&](int e) -> long long {
        e = min(e, total - 1);
        if (e < NB)
        {
            const int b0 = e * a.pool;
            return -1 - ((long long)bt[wa_div(b0, a.page, a.page_shift)] * a.per_page
                         + wa_div(wa_mod(b0, a.page, a.page_shift), a.pool, a.pool_shift));
        }
        const int j = j_lo + (e - NB);
        return (long long)bt[wa_div(j, a.page, a.page_shift)] * a.page + wa_mod(j, a.page, a.page_shift);
    };
    const int head = kh * hpg + h0 + min(qi, nh - 1);
    u32x4 qb[KK];
    {
        const u16* qp = (const u16*)a.q + ((long long)r * a.H + head) * DIM + 8 * g;
        #pragma unroll
        for (int kk = 0; kk < KK; kk++) qb[kk] = *(const u32x4*)(qp + 32 * kk);
    }
    f32x4 ot[DB];
    #pragma unroll
    for (int d = 0; d < DB; d++) ot[d] = (f32x4){0.0f, 0.0f, 0.0f, 0.0f};
    const bool with_sink = a.sink && wv == 0 && split == 0;      // the sink counts once
    float m_run = with_sink ? a.sink[head] : WM_NEG_BIG, l_run = with_sink ? 1.0f : 0.0f;

    long long krow[KPT], vrow[VPT];
    u32x4 kreg[KPT], vreg[VPT];
    auto lookup = [&](int step) {
        const int k0 = step * WD_BK;
        #pragma unroll
        for (int i = 0; i < KPT; i++) krow[i] = entry_row(k0 + (t + i * 256) / (DIM / 8));
        #pragma unroll
        for (int i = 0; i < VPT; i++) vrow[i] = DIM == VDIM ? krow[i] : entry_row(k0 + (t + i * 256) / (VDIM / 8));
    };
    auto fetch = [&]() {
        #pragma unroll
        for (int i = 0; i < KPT; i++)
        {
            const int c = t + i * 256;
            const long long row = krow[i];
            const u16* src = row >= 0 ? kc + (row * a.G + kh) * DIM : kp + ((-1 - row) * a.G + kh) * DIM;
            kreg[i] = *(const u32x4*)(src + (c % (DIM / 8)) * 8);
        }
        #pragma unroll
        for (int i = 0; i < VPT; i++)
        {
            const int c = t + i * 256;
            const long long row = vrow[i];
            const u16* src = row >= 0 ? vc + (row * a.G + kh) * VDIM : vp + ((-1 - row) * a.G + kh) * VDIM;
            vreg[i] = *(const u32x4*)(src + (c % (VDIM / 8)) * 8);
        }
    };
    auto stage = [&]() {
        #pragma unroll
        for (int i = 0; i < KPT; i++)
        {
            const int c = t + i * 256;
            *(u32x4*)(k_lds + (c / (DIM / 8)) * KSTR + (c % (DIM / 8)) * 8) = kreg[i];
        }
        #pragma unroll
        for (int i = 0; i < VPT; i++)
        {
            const int c = t + i * 256;
            *(u32x4*)(v_lds + (c / (VDIM / 8)) * VSTR + (c % (VDIM / 8)) * 8) = vreg[i];
        }
    };
    static_assert(KP % 256 == 0 && VP % 256 == 0, "a step is a whole number of 16-byte pieces per thread");

    if (step_lo < n_steps)
    {
        lookup(step_lo);
        fetch();
        if (step_lo + 1 < n_steps) lookup(step_lo + 1);
    }
    for (int step = step_lo; step < n_steps; step++)
    {
        block_sync();
        stage();
        block_sync();
        if (step + 1 < n_steps)
        {
            fetch();
            if (step + 2 < n_steps) lookup(step + 2);
        }
        const int k0 = step * WD_BK + 32 * wv;                  // this wave's 32 entries
        if (k0 >= total) continue;
        f32x4 st[2];
        #pragma unroll
        for (int blk = 0; blk < 2; blk++)
        {
            st[blk] = (f32x4){0.0f, 0.0f, 0.0f, 0.0f};
            const u16* kf = k_lds + (32 * wv + 16 * blk + qi) * KSTR + 8 * g;
            #pragma unroll
            for (int kk = 0; kk < KK; kk++) st[blk] = mfma_16x16x32_bf16(*(const u32x4*)(kf + 32 * kk), qb[kk], st[blk]);
        }
        float sc[8];
        float m_loc = WM_NEG_BIG;
        #pragma unroll
        for (int blk = 0; blk < 2; blk++)
            #pragma unroll
            for (int rr = 0; rr < 4; rr++)
            {
                const float v = k0 + 16 * blk + 4 * g + rr < total ? wa_soft_cap(st[blk][rr], a.softcap) : WM_NEG_BIG;
                sc[blk * 4 + rr] = v;
                m_loc = fmaxf(m_loc, v);
            }
        m_loc = fmaxf(m_loc, shfl_xor_f32(m_loc, 16));
        m_loc = fmaxf(m_loc, shfl_xor_f32(m_loc, 32));
        const float m_new = fmaxf(m_run, m_loc);
        const float alpha = expf(m_run - m_new);
        float p_sum = 0.0f;
        u32x4 pb;
        #pragma unroll
        for (int e2 = 0; e2 < 4; e2++)
        {
            const float pa = sc[2 * e2] > 0.5f * WM_NEG_BIG ? expf(sc[2 * e2] - m_new) : 0.0f;
            const float pc = sc[2 * e2 + 1] > 0.5f * WM_NEG_BIG ? expf(sc[2 * e2 + 1] - m_new) : 0.0f;
            p_sum += pa + pc;
            pb[e2] = wm_pack2(pa, pc);
        }
        p_sum += shfl_xor_f32(p_sum, 16);
        p_sum += shfl_xor_f32(p_sum, 32);
        l_run = l_run * alpha + p_sum;
        m_run = m_new;
        const u16* vbase = v_lds + (32 * wv + 4 * g + (qi >> 2)) * VSTR + 4 * (qi & 3);
        #pragma unroll
        for (int d = 0; d < DB; d++)
        {
            ot[d][0] *= alpha; ot[d][1] *= alpha; ot[d][2] *= alpha; ot[d][3] *= alpha;
            const f16x4 lo = lds_read_tr16_b64((const f16*)(vbase + 16 * d));
            const f16x4 hi = lds_read_tr16_b64((const f16*)(vbase + 16 * VSTR + 16 * d));
            const u32x2 l2 = __builtin_bit_cast(u32x2, lo), h2 = __builtin_bit_cast(u32x2, hi);
            ot[d] = mfma_16x16x32_bf16((u32x4){l2[0], l2[1], h2[0], h2[1]}, pb, ot[d]);
        }
    }

    // the four waves' partial results -> LDS (over the tiles): [wave][16 queries] (m, l), [wave][VDIM][16] O^T
    block_sync();
    float* s_ml = (float*)smem;                                  // [4][16][2]
    float* s_o = s_ml + 4 * 16 * 2;                              // [4][VDIM][16]
    if (g == 0) { s_ml[(wv * 16 + qi) * 2] = m_run; s_ml[(wv * 16 + qi) * 2 + 1] = l_run; }
    #pragma unroll
    for (int d = 0; d < DB; d++)
        #pragma unroll
        for (int rr = 0; rr < 4; rr++) s_o[(wv * VDIM + 16 * d + 4 * g + rr) * 16 + qi] = ot[d][rr];
    block_sync();
    // thread = (query column, pair of values): merge, turn back, gate, store
    const float fpos = (float)pos;
    for (int i = t; i < 16 * (VDIM / 2); i += 256)
    {
        const int q = i % 16, pr = i / 16;
        if (q >= nh) continue;
        int ia, ib;
        wa_pair(pr, VDIM, a.interleaved, ia, ib);
        float mx = WM_NEG_BIG;
        #pragma unroll
        for (int w = 0; w < 4; w++) mx = fmaxf(mx, s_ml[(w * 16 + q) * 2]);
        float l = 0.0f, u = 0.0f, v = 0.0f;
        #pragma unroll
        for (int w = 0; w < 4; w++)
        {
            const float mw = s_ml[(w * 16 + q) * 2];
            const float sc2 = mw > 0.5f * WM_NEG_BIG ? expf(mw - mx) : 0.0f;
            l = fmaf(s_ml[(w * 16 + q) * 2 + 1], sc2, l);
            u = fmaf(s_o[(w * VDIM + ia) * 16 + q], sc2, u);
            v = fmaf(s_o[(w * VDIM + ib) * 16 + q], sc2, v);
        }
        const int hd = kh * hpg + h0 + q;
        if (m.nsplit > 1)                                        // partial result: the merge kernel finishes the row
        {
            const long long pi = ((long long)r * a.H + hd) * m.nsplit + split;
            m.part_o[pi * VDIM + ia] = u; m.part_o[pi * VDIM + ib] = v;
            if (pr == 0) { m.part_ml[pi * 2] = mx; m.part_ml[pi * 2 + 1] = l; }
            continue;
        }
        const float inv = l > 0.0f ? 1.0f / l : 0.0f;
        u *= inv; v *= inv;
        if (a.v_rot)
        {
            const float ang = fpos * a.vfreq[pr];
            const float c = cosf(ang), sn = sinf(ang);
            const float u2 = u * c + v * sn, v2 = v * c - u * sn;
            u = u2; v = v2;
        }
        if (a.gate && a.gate_head)
        {
            const float hg = 1.0f / (1.0f + expf(-a.gate[(long long)r * a.ldg + hd]));
            u *= hg; v *= hg;
        }
        else if (a.gate)
        {
            const float* gt = a.gate + (long long)r * a.ldg + hd * VDIM;
            u *= 1.0f / (1.0f + expf(-gt[ia])); v *= 1.0f / (1.0f + expf(-gt[ib]));
        }
        u16* op = (u16*)a.out + ((long long)r * a.H + hd) * VDIM;
        op[ia] = f32_to_bf16(u); op[ib] = f32_to_bf16(v);
    }
}

// grid (decoded rows, heads): joins the nsplit partial results of a row's head, turns the output back, gates and stores it
KERNEL void __launch_bounds__(64) window_attn_merge_kernel(const WinMfmaArgs m)
{
    const WinAttnArgs& a = m.w;
    const int r = m.tile_row0[bid_x()], hd = bid_y();
    const long long p0 = ((long long)r * a.H + hd) * m.nsplit;
    float mx = WM_NEG_BIG;
    for (int sp = 0; sp < m.nsplit; sp++) mx = fmaxf(mx, m.part_ml[(p0 + sp) * 2]);
    float l = 0.0f;
    for (int sp = 0; sp < m.nsplit; sp++)
    {
        const float ms = m.part_ml[(p0 + sp) * 2];
        if (ms > 0.5f * WM_NEG_BIG) l = fmaf(m.part_ml[(p0 + sp) * 2 + 1], expf(ms - mx), l);
    }
    const float inv = l > 0.0f ? 1.0f / l : 0.0f;
    const float fpos = (float)a.row_pos[r];
    const float* gt = a.gate && !a.gate_head ? a.gate + (long long)r * a.ldg + hd * a.vdim : nullptr;
    const float hg = a.gate && a.gate_head ? 1.0f / (1.0f + expf(-a.gate[(long long)r * a.ldg + hd])) : 1.0f;
    u16* op = (u16*)a.out + ((long long)r * a.H + hd) * a.vdim;
    for (int pr = tid(); pr < a.vdim / 2; pr += 64)
    {
        int ia, ib;
        wa_pair(pr, a.vdim, a.interleaved, ia, ib);
        float u = 0.0f, v = 0.0f;
        for (int sp = 0; sp < m.nsplit; sp++)
        {
            const float ms = m.part_ml[(p0 + sp) * 2];
            if (ms <= 0.5f * WM_NEG_BIG) continue;
            const float sc = expf(ms - mx);
            u = fmaf(m.part_o[(p0 + sp) * a.vdim + ia], sc, u);
            v = fmaf(m.part_o[(p0 + sp) * a.vdim + ib], sc, v);
        }
        u *= inv; v *= inv;
        if (a.v_rot)
        {
            const float ang = fpos * a.vfreq[pr];
            const float c = cosf(ang), sn = sinf(ang);
            const float u2 = u * c + v * sn, v2 = v * c - u * sn;
            u = u2; v = v2;
        }
        if (gt) { u *= 1.0f / (1.0f + expf(-gt[ia])); v *= 1.0f / (1.0f + expf(-gt[ib])); }
        op[ia] = f32_to_bf16(u * hg); op[ib] = f32_to_bf16(v * hg);
    }
}

template <int DIM, int VDIM>
static void wd_launch(const WinMfmaArgs& m, int tiles, hipStream_t s)
{
    static bool attr_done[EXL2_MAX_DEVICES];
    size_t lds = ((size_t)WD_BK * (DIM + 8) + (size_t)WD_BK * (VDIM + 16)) * 2;
    const size_t merge = sizeof(float) * (4 * 16 * 2 + (size_t)4 * VDIM * 16);
    if (merge > lds) lds = merge;
    if (exl2_first_on_device(attr_done))
        (void)hipFuncSetAttribute((const void*)window_attn_decode_kernel<DIM, VDIM>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    const int hpg = m.w.H / m.w.G;
    LAUNCH((window_attn_decode_kernel<DIM, VDIM>), dim3(tiles, m.w.G, m.nsplit * ((hpg + 15) / 16)), dim3(256), lds, s, m);
    if (m.nsplit > 1) LAUNCH(window_attn_merge_kernel, dim3(tiles, m.w.H), dim3(64), 0, s, m);
}

// ---- C ABI ----------------------------------------------------------------------------------------------------------------------

extern "C" int exl2_kv_rot_append_ex(const float* f, int ld, int q_off, int k_off, int v_off, void* q_out, const float* q_scale,
                                     void* k_cache, void* v_cache, void* k_pool, void* v_pool, const float* freq, float amp, int rot_dims,
                                     const float* vfreq, int v_rot, int interleaved, const int* row_seq, const int* row_pos,
                                     const int* block_table, int bt_stride, int page, int pool, int dtype, int rows, int heads,
                                     int kv_heads, int dim, int vdim, void* stream);
extern "C" int exl2_window_attn_ex(const void* q, const void* k_cache, const void* v_cache, const void* k_pool, const void* v_pool,
                                   const float* sink, const float* gate, int ldg, const float* vfreq, int v_rot, int interleaved,
                                   const int* row_seq, const int* row_pos, const int* block_table, int bt_stride, int page, int pool,
                                   void* out, int dtype, int rows, int heads, int kv_heads, int dim, int vdim, int window, int chunk,
                                   float softcap, int gate_head, void* stream);
extern "C" int exl2_window_attn_tiles_ex(const void* q, const void* k_cache, const void* v_cache, const void* k_pool, const void* v_pool,
                                         const float* sink, const float* gate, int ldg, const float* vfreq, int v_rot, int interleaved,
                                         const int* row_seq, const int* row_pos, const int* block_table, int bt_stride, int page, int pool,
                                         void* out, const int* tile_row0, const int* tile_rows, int tiles, int tile_mode, float* part_o,
                                         float* part_ml, int nsplit, int heads, int kv_heads, int dim, int vdim, int window, int chunk,
                                         float softcap, int gate_head, void* stream);

extern "C" int exl2_kv_rot_append(const float* f, int ld, int q_off, int k_off, int v_off, void* q_out, const float* q_scale,
                                  void* k_cache, void* v_cache, void* k_pool, void* v_pool, const float* freq, float amp, int rot_dims,
                                  const float* vfreq, int v_rot, int interleaved, const int* row_seq, const int* row_pos,
                                  const int* block_table, int bt_stride, int page, int pool, int dtype, int rows, int heads,
                                  int kv_heads, int dim, int vdim, void* stream)
{
    EXL2_REQUIRE(k_cache && v_cache, "kv_rot_append: null operand");
    return exl2_kv_rot_append_ex(f, ld, q_off, k_off, v_off, q_out, q_scale, k_cache, v_cache, k_pool, v_pool, freq, amp, rot_dims, vfreq,
                                 v_rot, interleaved, row_seq, row_pos, block_table, bt_stride, page, pool, dtype, rows, heads, kv_heads,
                                 dim, vdim, stream);
}

extern "C" int exl2_kv_rot_append_ex(const float* f, int ld, int q_off, int k_off, int v_off, void* q_out, const float* q_scale,
                                     void* k_cache, void* v_cache, void* k_pool, void* v_pool, const float* freq, float amp, int rot_dims,
                                     const float* vfreq, int v_rot, int interleaved, const int* row_seq, const int* row_pos,
                                     const int* block_table, int bt_stride, int page, int pool, int dtype, int rows, int heads,
                                     int kv_heads, int dim, int vdim, void* stream)
{
    EXL2_REQUIRE(f && q_out && q_scale && freq && row_seq && row_pos && block_table, "kv_rot_append: null operand");
    EXL2_REQUIRE((k_cache == nullptr) == (v_cache == nullptr), "kv_rot_append: keys and values go to the cache together");
    EXL2_REQUIRE(k_cache || pool == 0, "kv_rot_append: rows that bring queries only write no pooled blocks");
    EXL2_REQUIRE(dtype == 0 || dtype == 1, "kv_rot_append: dtype must be 0 (bfloat16) or 1 (float32)");
    EXL2_REQUIRE(heads > 0 && kv_heads > 0 && heads % kv_heads == 0 && dim > 0 && vdim > 0, "kv_rot_append: bad head shape");
    EXL2_REQUIRE(rot_dims >= 0 && rot_dims <= dim && rot_dims % 2 == 0, "kv_rot_append: %d rotated of %d values", rot_dims, dim);
    EXL2_REQUIRE(!v_rot || (vfreq && vdim % 2 == 0), "kv_rot_append: rotated values need an even size and their frequencies");
    EXL2_REQUIRE(page > 0 && pool >= 0 && (pool == 0 || (k_pool && v_pool)), "kv_rot_append: bad paging (page %d, pool %d)", page, pool);
    if (rows <= 0) return EXL2_OK;
    RotAppendArgs a;
    a.f = f; a.ld = ld; a.q_off = q_off; a.k_off = k_off; a.v_off = v_off; a.q_out = q_out; a.q_scale = q_scale; a.k_cache = k_cache;
    a.v_cache = v_cache; a.freq = freq; a.amp = amp; a.rot_dims = rot_dims; a.vfreq = vfreq; a.v_rot = v_rot; a.interleaved = interleaved;
    a.row_seq = row_seq; a.row_pos = row_pos; a.block_table = block_table; a.bt_stride = bt_stride; a.page = page;
    a.H = heads; a.G = kv_heads; a.dim = dim; a.vdim = vdim;
    if (dtype == 0) LAUNCH(rot_append_kernel<u16>, dim3(rows), dim3(256), 0, stream, a);
    else LAUNCH(rot_append_kernel<float>, dim3(rows), dim3(256), 0, stream, a);
    if (pool > 0)
    {
        PoolArgs p;
        p.k_cache = k_cache; p.v_cache = v_cache; p.k_pool = k_pool; p.v_pool = v_pool; p.row_seq = row_seq; p.row_pos = row_pos;
        p.block_table = block_table; p.bt_stride = bt_stride; p.page = page; p.pool = pool; p.per_page = (page + pool - 1) / pool;
        p.kw = kv_heads * dim; p.vw = kv_heads * vdim;
        const int vn = dtype == 0 ? 8 : 4;
        const bool vec = p.kw % vn == 0 && p.vw % vn == 0 && ((uintptr_t)k_cache % 16) == 0 && ((uintptr_t)v_cache % 16) == 0;
        const dim3 grid(rows, vec ? ((p.kw + p.vw) / vn + 63) / 64 : 1);
        if (dtype == 0) { if (vec) LAUNCH((pool_blocks_kernel<u16, true>), grid, dim3(256), 0, stream, p); else LAUNCH((pool_blocks_kernel<u16, false>), grid, dim3(256), 0, stream, p); }
        else { if (vec) LAUNCH((pool_blocks_kernel<float, true>), grid, dim3(256), 0, stream, p); else LAUNCH((pool_blocks_kernel<float, false>), grid, dim3(256), 0, stream, p); }
    }
    HIP_TRY(hipGetLastError());
    return EXL2_OK;
}

extern "C" int exl2_window_attn(const void* q, const void* k_cache, const void* v_cache, const void* k_pool, const void* v_pool,
                                const float* sink, const float* gate, int ldg, const float* vfreq, int v_rot, int interleaved,
                                const int* row_seq, const int* row_pos, const int* block_table, int bt_stride, int page, int pool,
                                void* out, int dtype, int rows, int heads, int kv_heads, int dim, int vdim, int window, void* stream)
{
    return exl2_window_attn_ex(q, k_cache, v_cache, k_pool, v_pool, sink, gate, ldg, vfreq, v_rot, interleaved, row_seq, row_pos,
                               block_table, bt_stride, page, pool, out, dtype, rows, heads, kv_heads, dim, vdim, window, 0, 0.0f, 0, stream);
}

extern "C" int exl2_window_attn_ex(const void* q, const void* k_cache, const void* v_cache, const void* k_pool, const void* v_pool,
                                   const float* sink, const float* gate, int ldg, const float* vfreq, int v_rot, int interleaved,
                                   const int* row_seq, const int* row_pos, const int* block_table, int bt_stride, int page, int pool,
                                   void* out, int dtype, int rows, int heads, int kv_heads, int dim, int vdim, int window, int chunk,
                                   float softcap, int gate_head, void* stream)
{
    EXL2_REQUIRE(chunk >= 0 && (chunk == 0 || pool == 0), "window_attn: a chunked mask has no pooled blocks");
    EXL2_REQUIRE(softcap >= 0.0f, "window_attn: negative soft cap");
    EXL2_REQUIRE(q && k_cache && v_cache && row_seq && row_pos && block_table && out, "window_attn: null operand");
    EXL2_REQUIRE(dtype == 0 || dtype == 1, "window_attn: dtype must be 0 (bfloat16) or 1 (float32)");
    EXL2_REQUIRE(heads > 0 && kv_heads > 0 && heads % kv_heads == 0 && dim > 0, "window_attn: bad head shape");
    EXL2_REQUIRE(vdim > 0 && vdim <= 256 * WA_MAX_V_PER_THREAD, "window_attn: vdim %d (at most %d)", vdim, 256 * WA_MAX_V_PER_THREAD);
    EXL2_REQUIRE(page > 0 && window > 0 && pool >= 0 && (pool == 0 || (k_pool && v_pool)), "window_attn: bad window / paging");
    EXL2_REQUIRE(!v_rot || (vfreq && vdim % 2 == 0), "window_attn: rotated values need an even size and their frequencies");
    if (rows <= 0) return EXL2_OK;
    WinAttnArgs a;
    a.q = q; a.k_cache = k_cache; a.v_cache = v_cache; a.k_pool = k_pool; a.v_pool = v_pool; a.sink = sink; a.gate = gate; a.ldg = ldg;
    a.vfreq = vfreq; a.v_rot = v_rot; a.interleaved = interleaved; a.row_seq = row_seq; a.row_pos = row_pos; a.block_table = block_table;
    a.bt_stride = bt_stride; a.page = page; a.pool = pool; a.per_page = pool > 0 ? (page + pool - 1) / pool : 0; a.out = out;
    a.H = heads; a.G = kv_heads; a.dim = dim; a.vdim = vdim; a.window = window; a.page_shift = a.pool_shift = -1;
    a.chunk = chunk; a.softcap = softcap; a.gate_head = gate_head;
    const size_t smem = (size_t)(dim + vdim) * 4;
    if (dtype == 0) LAUNCH(window_attn_kernel<u16>, dim3(rows, heads), dim3(256), smem, stream, a);
    else LAUNCH(window_attn_kernel<float>, dim3(rows, heads), dim3(256), smem, stream, a);
    HIP_TRY(hipGetLastError());
    return EXL2_OK;
}

/* 1 if exl2_window_attn_tiles takes these head sizes */
extern "C" int exl2_window_attn_tiles_supported(int dim, int vdim)
{
    return (dim == vdim && (dim == 32 || dim == 64 || dim == 96 || dim == 128 || dim == 256)) || (dim == 192 && vdim == 128)
           || (dim == 128 && vdim == 64) || (dim == 64 && vdim == 128);
}

/* exl2_window_attn on the matrix cores (bfloat16, head sizes of exl2_window_attn_tiles_supported; gate rows and offsets multiples
   of 4 values).  The step's rows come as tiles.  tile_mode 64: tile i = rows tile_row0[i] .. + tile_rows[i], <= 64 consecutive
   positions of ONE sequence (portions of prompts; one head per workgroup).  tile_mode 1: the single rows tile_row0[i] (decoded
   tokens; the heads of a key / value head share one pass over the keys); nsplit > 1 deals the key list's steps of 128 entries to
   nsplit workgroups, part_o fp32 [rows, heads, nsplit, vdim] and part_ml fp32 [rows, heads, nsplit, 2] are scratch indexed by row. */
extern "C" int exl2_window_attn_tiles(const void* q, const void* k_cache, const void* v_cache, const void* k_pool, const void* v_pool,
                                      const float* sink, const float* gate, int ldg, const float* vfreq, int v_rot, int interleaved,
                                      const int* row_seq, const int* row_pos, const int* block_table, int bt_stride, int page, int pool,
                                      void* out, const int* tile_row0, const int* tile_rows, int tiles, int tile_mode, float* part_o,
                                      float* part_ml, int nsplit, int heads, int kv_heads, int dim, int vdim, int window, void* stream)
{
    return exl2_window_attn_tiles_ex(q, k_cache, v_cache, k_pool, v_pool, sink, gate, ldg, vfreq, v_rot, interleaved, row_seq, row_pos,
                                     block_table, bt_stride, page, pool, out, tile_row0, tile_rows, tiles, tile_mode, part_o, part_ml,
                                     nsplit, heads, kv_heads, dim, vdim, window, 0, 0.0f, 0, stream);
}

extern "C" int exl2_window_attn_tiles_ex(const void* q, const void* k_cache, const void* v_cache, const void* k_pool, const void* v_pool,
                                         const float* sink, const float* gate, int ldg, const float* vfreq, int v_rot, int interleaved,
                                         const int* row_seq, const int* row_pos, const int* block_table, int bt_stride, int page, int pool,
                                         void* out, const int* tile_row0, const int* tile_rows, int tiles, int tile_mode, float* part_o,
                                         float* part_ml, int nsplit, int heads, int kv_heads, int dim, int vdim, int window, int chunk,
                                         float softcap, int gate_head, void* stream)
{
    EXL2_REQUIRE(chunk >= 0 && (chunk == 0 || pool == 0), "window_attn_tiles: a chunked mask has no pooled blocks");
    EXL2_REQUIRE(softcap >= 0.0f, "window_attn_tiles: negative soft cap");
    EXL2_REQUIRE(nsplit >= 1 && nsplit <= 64 && (nsplit == 1 || (tile_mode == 1 && part_o && part_ml)),
                 "window_attn_tiles: key splits (1 .. 64) need tile_mode 1 and scratch");
    EXL2_REQUIRE(q && k_cache && v_cache && row_seq && row_pos && block_table && out && tile_row0, "window_attn_tiles: null operand");
    EXL2_REQUIRE(tile_mode == 64 || tile_mode == 1, "window_attn_tiles: tile_mode is 64 or 1");
    EXL2_REQUIRE(tile_mode == 1 || tile_rows, "window_attn_tiles: tile_rows missing");
    EXL2_REQUIRE(heads > 0 && kv_heads > 0 && heads % kv_heads == 0, "window_attn_tiles: bad head shape");
    EXL2_REQUIRE(page > 0 && window > 0 && pool >= 0 && (pool == 0 || (k_pool && v_pool)), "window_attn_tiles: bad window / paging");
    EXL2_REQUIRE(!v_rot || vfreq, "window_attn_tiles: rotated values need their frequencies");
    EXL2_REQUIRE(!gate || gate_head || (ldg % 4 == 0 && ((uintptr_t)gate % 16) == 0), "window_attn_tiles: gate rows must be 16-byte aligned");
    if (!exl2_window_attn_tiles_supported(dim, vdim))
        EXL2_FAIL(EXL2_E_UNSUPPORTED, "window_attn_tiles: head sizes %d / %d outside the matrix-core form", dim, vdim);
    if (tiles <= 0) return EXL2_OK;
    WinMfmaArgs m;
    WinAttnArgs& a = m.w;
    a.q = q; a.k_cache = k_cache; a.v_cache = v_cache; a.k_pool = k_pool; a.v_pool = v_pool; a.sink = sink; a.gate = gate; a.ldg = ldg;
    a.vfreq = vfreq; a.v_rot = v_rot; a.interleaved = interleaved; a.row_seq = row_seq; a.row_pos = row_pos; a.block_table = block_table;
    a.bt_stride = bt_stride; a.page = page; a.pool = pool; a.per_page = pool > 0 ? (page + pool - 1) / pool : 0; a.out = out;
    a.H = heads; a.G = kv_heads; a.dim = dim; a.vdim = vdim; a.window = window;
    a.chunk = chunk; a.softcap = softcap; a.gate_head = gate_head;
    a.page_shift = wa_log2_exact(page); a.pool_shift = pool > 0 ? wa_log2_exact(pool) : -1;
    m.tile_row0 = tile_row0; m.tile_rows = tile_rows; m.part_o = part_o; m.part_ml = part_ml; m.nsplit = nsplit;
    hipStream_t s = (hipStream_t)stream;
    if (tile_mode == 1)
    {
        if (dim == 32 && vdim == 32) wd_launch<32, 32>(m, tiles, s);
        else if (dim == 64 && vdim == 64) wd_launch<64, 64>(m, tiles, s);
        else if (dim == 96 && vdim == 96) wd_launch<96, 96>(m, tiles, s);
        else if (dim == 128 && vdim == 128) wd_launch<128, 128>(m, tiles, s);
        else if (dim == 256 && vdim == 256) wd_launch<256, 256>(m, tiles, s);
        else if (dim == 192 && vdim == 128) wd_launch<192, 128>(m, tiles, s);
        else if (dim == 128 && vdim == 64) wd_launch<128, 64>(m, tiles, s);
        else wd_launch<64, 128>(m, tiles, s);
        HIP_TRY(hipGetLastError());
        return EXL2_OK;
    }
    if (dim == 32 && vdim == 32) wm_launch<32, 32>(m, tiles, s);
    else if (dim == 64 && vdim == 64) wm_launch<64, 64>(m, tiles, s);
    else if (dim == 96 && vdim == 96) wm_launch<96, 96>(m, tiles, s);
    else if (dim == 128 && vdim == 128) wm_launch<128, 128>(m, tiles, s);
    else if (dim == 256 && vdim == 256) wm_launch<256, 256>(m, tiles, s);
    else if (dim == 192 && vdim == 128) wm_launch<192, 128>(m, tiles, s);
    else if (dim == 128 && vdim == 64) wm_launch<128, 64>(m, tiles, s);
    else wm_launch<64, 128>(m, tiles, s);
    HIP_TRY(hipGetLastError());
    return EXL2_OK;
}
