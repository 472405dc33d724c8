// dense.hip -- linears over UNQUANTIZED weights (bfloat16 or fp32, stored [out, in]) for gfx950, + their C ABI.
//
// y[r, n] = epilogue( sum_k x[r, k] * w[n, k] ), fp32 accumulation always.  One entry point, four kernels:
//   * lin_rows_kernel  -- decode-sized calls (<= 16 rows): one wave per output column, the K range split over the 64 lanes with
//                         16-byte loads of the weight row (a [out, in] row is contiguous: one wave streams it once for all rows);
//                         also the sparse-MoE decode form: every row names the weight slab it multiplies (w_sel).
//   * lin_mfma_kernel  -- bfloat16, 17 .. 64 rows: v_mfma_f32_16x16x32_bf16.  Both operands are K-contiguous, so a lane's 8 values of
//                         an A or B fragment are ONE 16-byte load straight from memory into the register the matrix core reads.
//   * lin_mfma_tile_kernel -- bfloat16, more rows: 128 x 128 tiles staged through LDS, two stages deep.
//   * lin_tile_kernel  -- fp32 (true 32-bit FMA, no reduced-precision matrix mode) and every shape the other two decline
//                         (K or a leading dimension that is not a multiple of 8 values): 64 x 64 tiles through LDS.
// A call may be batched over blockIdx.z (per-head projections: element offsets per batch for x, w, y, aux) or GROUPED (sparse MoE
// at many rows: batch z = expert z multiplies the rows listed for it, counts and lists in device memory, no host round trip).
// Epilogues fold the layer's elementwise steps into the producing linear: acc * sigmoid(aux) (output gate), silu(aux) * acc
// (gated MLP), the clamped gated unit min(aux, L) * sigmoid(1.702 min(aux, L)) * (clamp(acc, -L, L) + 1), relu(acc)^2, the soft
// cap L tanh(acc / L), a plain scale L acc, tanh(acc), and relu(aux[row] acc)^2 (an expert whose INPUT carries the router's weight:
// W (s h) = s (W h)), the two halves of a gated unit on such an input -- silu(aux[row] acc) aux[row] from the gate matrix, then
// aux acc from the up matrix --; a bias vector (fp32, one value per output column) is added to the accumulator first.
#include "hw.h"
#include "errors.h"

enum { DENSE_BF16 = 0, DENSE_F32 = 1 };
enum { EPI_NONE = 0, EPI_MUL_SIGMOID_AUX = 1, EPI_SILU_AUX_MUL = 2, EPI_CLAMPED_GLU = 3, EPI_RELU_SQUARED = 4, EPI_SOFT_CAP = 5,
       EPI_SCALE = 6, EPI_TANH = 7, EPI_ROW_SCALED_RELU_SQUARED = 8, EPI_ROW_SCALED_SILU_SCALED = 9, EPI_AUX_MUL = 10, EPI_LAST = 10 };
// aux holds ONE value per row (ldaux apart), not one per output
#define EPI_ROW_AUX(e) ((e) == EPI_ROW_SCALED_RELU_SQUARED || (e) == EPI_ROW_SCALED_SILU_SCALED)
#define EPI_READS_AUX(e) (((e) >= EPI_MUL_SIGMOID_AUX && (e) <= EPI_CLAMPED_GLU) || EPI_ROW_AUX(e) || (e) == EPI_AUX_MUL)
#define EPI_AUX_COL(e, n) (EPI_ROW_AUX(e) ? 0 : (n))

struct LinArgs
{
    const void* x; const void* w; void* y; const float* aux;
    const float* bias;                       // [N] added to the accumulator before the epilogue (nullptr: none)
    int M, N, K;
    int ldx, ldw, ldy, ldaux;
    long long sxb, swb, syb, sauxb;          // element offsets per batch (blockIdx.z)
    const int* w_sel; int n_sel;             // rows kernel: row r multiplies slab w_sel[r] (>= n_sel: the row is skipped)
    const int* grp_count; const int* grp_offset; const int* grp_rows;     // grouped: rows of batch z = grp_rows[grp_offset[z] + i]
    int x_div;                               // x row of logical row p = p / x_div (several output rows per input row)
    int epi; float limit;
};

template <typename T> DEV float ld1(const T* p);
template <> DEV float ld1<u16>(const u16* p) { return bf16_to_f32(*p); }
template <> DEV float ld1<float>(const float* p) { return *p; }
template <typename T> DEV void st1(T* p, float v);
template <> DEV void st1<u16>(u16* p, float v) { *p = f32_to_bf16(v); }
template <> DEV void st1<float>(float* p, float v) { *p = v; }

// 16 bytes of T as floats
template <typename T> struct Vec16;
template <> struct Vec16<u16>
{
    static constexpr int N = 8;
    static DEV void load(const u16* p, float* f)
    {
        const u32x4 v = *(const u32x4*)p;
        #pragma unroll
        for (int i = 0; i < 4; i++) { f[2 * i] = as_f32(v[i] << 16); f[2 * i + 1] = as_f32(v[i] & 0xffff0000u); }
    }
};
template <> struct Vec16<float>
{
    static constexpr int N = 4;
    static DEV void load(const float* p, float* f)
    {
        const f32x4 v = *(const f32x4*)p;
        #pragma unroll
        for (int i = 0; i < 4; i++) f[i] = v[i];
    }
};

DEV float sigmoid_f32(float z) { return 1.0f / (1.0f + expf(-z)); }

DEV float lin_epilogue(int epi, float acc, float aux, float limit)
{
    if (epi == EPI_MUL_SIGMOID_AUX) return acc * sigmoid_f32(aux);
    if (epi == EPI_SILU_AUX_MUL) return aux * sigmoid_f32(aux) * acc;
    if (epi == EPI_CLAMPED_GLU)
    {
        const float g = fminf(aux, limit);
        const float u = fminf(fmaxf(acc, -limit), limit);
        return g * sigmoid_f32(1.702f * g) * (u + 1.0f);
    }
    if (epi == EPI_RELU_SQUARED) { const float r = fmaxf(acc, 0.0f); return r * r; }
    if (epi == EPI_SOFT_CAP) return limit * tanhf(acc / limit);
    if (epi == EPI_SCALE) return acc * limit;
    if (epi == EPI_TANH) return tanhf(acc);
    if (epi == EPI_ROW_SCALED_RELU_SQUARED) { const float r = fmaxf(acc * aux, 0.0f); return r * r; }
    if (epi == EPI_ROW_SCALED_SILU_SCALED) { const float z = acc * aux; return z * sigmoid_f32(z) * aux; }
    if (epi == EPI_AUX_MUL) return acc * aux;
    return acc;
}

// ---- <= 16 rows -------------------------------------------------------------------------------------------------------------

template <typename T, typename TY, int MB, bool VEC>
KERNEL void __launch_bounds__(256) lin_rows_kernel(const LinArgs a)
{
    const int n = bid_x() * 4 + wave_id();
    const int r0 = bid_y() * MB;
    const int z = bid_z();
    const int lane = lane_id();
    if (n >= a.N) return;
    long long slab = (long long)z * a.swb;
    if (a.w_sel)
    {
        const int e = a.w_sel[r0];                       // MB == 1 in this form
        if (e < 0 || e >= a.n_sel) return;
        slab += (long long)e * a.swb;
    }
    const T* wr = (const T*)a.w + slab + (long long)n * a.ldw;
    const T* xr[MB];
    #pragma unroll
    for (int m = 0; m < MB; m++)
    {
        const int r = min(r0 + m, a.M - 1);
        xr[m] = (const T*)a.x + (long long)z * a.sxb + (long long)(r / a.x_div) * a.ldx;
    }
    float acc[MB];
    #pragma unroll
    for (int m = 0; m < MB; m++) acc[m] = 0.0f;
    if (VEC)
    {
        constexpr int V = Vec16<T>::N;
        for (int k = lane * V; k < a.K; k += 64 * V)
        {
            float wv[V];
            Vec16<T>::load(wr + k, wv);
            #pragma unroll
            for (int m = 0; m < MB; m++)
            {
                float xv[V];
                Vec16<T>::load(xr[m] + k, xv);
                #pragma unroll
                for (int i = 0; i < V; i++) acc[m] = fmaf(xv[i], wv[i], acc[m]);
            }
        }
    }
    else
    {
        for (int k = lane; k < a.K; k += 64)
        {
            const float wv = ld1<T>(wr + k);
            #pragma unroll
            for (int m = 0; m < MB; m++) acc[m] = fmaf(ld1<T>(xr[m] + k), wv, acc[m]);
        }
    }
    #pragma unroll
    for (int m = 0; m < MB; m++) acc[m] = wave_allreduce_add(acc[m]);
    if (lane == 0)
    {
        #pragma unroll
        for (int m = 0; m < MB; m++)
        {
            const int r = r0 + m;
            if (r >= a.M) break;
            float aux = 0.0f;
            if (EPI_READS_AUX(a.epi)) aux = a.aux[(long long)z * a.sauxb + (long long)r * a.ldaux + EPI_AUX_COL(a.epi, n)];
            st1<TY>((TY*)a.y + (long long)z * a.syb + (long long)r * a.ldy + n, lin_epilogue(a.epi, acc[m] + (a.bias ? a.bias[n] : 0.0f), aux, a.limit));
        }
    }
}

// ---- 64 x 64 tiles, fp32 FMA ----------------------------------------------------------------------------------------------

template <typename T, typename TY>
KERNEL void __launch_bounds__(256) lin_tile_kernel(const LinArgs a)
{
    SHARED __attribute__((aligned(16))) float As[16][68];
    SHARED __attribute__((aligned(16))) float Bs[16][68];
    SHARED int rowmap[64];
    const int z = bid_z();
    const int m0 = bid_y() * 64, n0 = bid_x() * 64;
    const int M = a.grp_count ? a.grp_count[z] : a.M;
    if (m0 >= M) return;
    const int t = tid();
    if (t < 64)
    {
        const int r = min(m0 + t, M - 1);
        rowmap[t] = a.grp_rows ? a.grp_rows[a.grp_offset[z] + r] : r;
    }
    block_sync();
    const int lr = t >> 2, lk = (t & 3) * 4;                 // this thread stages 4 consecutive k of one row / column
    const T* xp = (const T*)a.x + (long long)z * a.sxb + (long long)(rowmap[lr] / a.x_div) * a.ldx;
    const int nn = min(n0 + lr, a.N - 1);
    const T* wp = (const T*)a.w + (long long)z * a.swb + (long long)nn * a.ldw;
    const int ty = t >> 4, tx = t & 15;
    float acc[4][4];
    #pragma unroll
    for (int i = 0; i < 4; i++)
        #pragma unroll
        for (int j = 0; j < 4; j++) acc[i][j] = 0.0f;
    for (int k0 = 0; k0 < a.K; k0 += 16)
    {
        #pragma unroll
        for (int i = 0; i < 4; i++)
        {
            const int k = k0 + lk + i;
            As[lk + i][lr] = k < a.K ? ld1<T>(xp + k) : 0.0f;
            Bs[lk + i][lr] = k < a.K ? ld1<T>(wp + k) : 0.0f;
        }
        block_sync();
        #pragma unroll
        for (int k = 0; k < 16; k++)
        {
            const f32x4 av = *(const f32x4*)&As[k][ty * 4];
            const f32x4 bv = *(const f32x4*)&Bs[k][tx * 4];
            #pragma unroll
            for (int i = 0; i < 4; i++)
                #pragma unroll
                for (int j = 0; j < 4; j++) acc[i][j] = fmaf(av[i], bv[j], acc[i][j]);
        }
        block_sync();
    }
    #pragma unroll
    for (int i = 0; i < 4; i++)
    {
        const int rl = ty * 4 + i;
        if (m0 + rl >= M) continue;
        const long long r = rowmap[rl];
        #pragma unroll
        for (int j = 0; j < 4; j++)
        {
            const int n = n0 + tx * 4 + j;
            if (n >= a.N) continue;
            float aux = 0.0f;
            if (EPI_READS_AUX(a.epi)) aux = a.aux[(long long)z * a.sauxb + r * a.ldaux + EPI_AUX_COL(a.epi, n)];
            st1<TY>((TY*)a.y + (long long)z * a.syb + r * a.ldy + n, lin_epilogue(a.epi, acc[i][j] + (a.bias ? a.bias[n] : 0.0f), aux, a.limit));
        }
    }
}

// ---- bfloat16 on the matrix cores ------------------------------------------------------------------------------------------
// Workgroup = 4 waves = (16 * RT) rows x 256 columns; a wave owns 64 columns (4 B fragments) and RT row blocks.  Lane l of a
// fragment holds row / column (l & 15), k = 8 (l >> 4) .. + 7 of the 32-wide step: 16 contiguous bytes of a K-contiguous row.
// Rows and columns past the edge are clamped for the loads and dropped at the store; the K tail is masked by lane group.

template <typename TY, int RT>
KERNEL void __launch_bounds__(256) lin_mfma_kernel(const LinArgs a)
{
    SHARED int rowmap[16 * RT];
    const int z = bid_z();
    const int m0 = bid_y() * 16 * RT, n0 = bid_x() * 256 + wave_id() * 64;
    const int M = a.grp_count ? a.grp_count[z] : a.M;
    if (m0 >= M) return;
    const int t = tid(), lane = lane_id();
    if (t < 16 * RT)
    {
        const int r = min(m0 + t, M - 1);
        rowmap[t] = a.grp_rows ? a.grp_rows[a.grp_offset[z] + r] : r;
    }
    block_sync();
    if (n0 >= a.N) return;
    const int li = lane & 15, kg = (lane >> 4) * 8;
    const u16* xp[RT];
    #pragma unroll
    for (int i = 0; i < RT; i++)
        xp[i] = (const u16*)a.x + (long long)z * a.sxb + (long long)(rowmap[16 * i + li] / a.x_div) * a.ldx + kg;
    const u16* wp[4];
    #pragma unroll
    for (int j = 0; j < 4; j++)
        wp[j] = (const u16*)a.w + (long long)z * a.swb + (long long)min(n0 + 16 * j + li, a.N - 1) * a.ldw + kg;
    f32x4 acc[RT][4];
    #pragma unroll
    for (int i = 0; i < RT; i++)
        #pragma unroll
        for (int j = 0; j < 4; j++) acc[i][j] = (f32x4){0.0f, 0.0f, 0.0f, 0.0f};
    const u32x4 zero = {0u, 0u, 0u, 0u};
    for (int k0 = 0; k0 < a.K; k0 += 32)
    {
        const bool live = k0 + kg < a.K;                     // K % 8 == 0: a lane's 8 values are all inside or all outside
        u32x4 af[RT], bf[4];
        #pragma unroll
        for (int i = 0; i < RT; i++) af[i] = live ? *(const u32x4*)(xp[i] + k0) : zero;
        #pragma unroll
        for (int j = 0; j < 4; j++) bf[j] = live ? *(const u32x4*)(wp[j] + k0) : zero;
        #pragma unroll
        for (int i = 0; i < RT; i++)
            #pragma unroll
            for (int j = 0; j < 4; j++) acc[i][j] = mfma_16x16x32_bf16(af[i], bf[j], acc[i][j]);
    }
    // D: column (lane & 15) of the fragment, rows 4 (lane >> 4) + r
    #pragma unroll
    for (int i = 0; i < RT; i++)
        #pragma unroll
        for (int r = 0; r < 4; r++)
        {
            const int rl = 16 * i + 4 * (lane >> 4) + r;
            if (m0 + rl >= M) continue;
            const long long row = rowmap[rl];
            #pragma unroll
            for (int j = 0; j < 4; j++)
            {
                const int n = n0 + 16 * j + li;
                if (n >= a.N) continue;
                float aux = 0.0f;
                if (EPI_READS_AUX(a.epi)) aux = a.aux[(long long)z * a.sauxb + row * a.ldaux + EPI_AUX_COL(a.epi, n)];
                st1<TY>((TY*)a.y + (long long)z * a.syb + row * a.ldy + n, lin_epilogue(a.epi, acc[i][j][r] + (a.bias ? a.bias[n] : 0.0f), aux, a.limit));
            }
        }
}

// ---- bfloat16 on the matrix cores, 128 x 128 tiles through LDS (many rows) ------------------------------------------------------
// Workgroup = 4 waves = 128 rows x 128 columns, a wave owns a 64 x 64 quadrant (4 x 4 fragments).  A K step is 32 values: the
// workgroup stages the 128 x 32 slices of x and w (16 bytes per thread and row, row stride 80 bytes: the 16-lane phases of a
// 16-byte LDS read fall into distinct banks), two stages deep -- the next step's slices are requested from memory before the current
// step's 16 MFMAs and written to the other stage after them.

#define LT_STRIDE 40                                         // values per staged row (32 + 8 of padding)

template <typename TY>
KERNEL void __launch_bounds__(256) lin_mfma_tile_kernel(const LinArgs a)
{
    SHARED __attribute__((aligned(16))) u16 As[2][128 * LT_STRIDE];
    SHARED __attribute__((aligned(16))) u16 Bs[2][128 * LT_STRIDE];
    SHARED int rowmap[128];
    const int z = bid_z();
    const int m0 = bid_y() * 128, n0 = bid_x() * 128;
    const int M = a.grp_count ? a.grp_count[z] : a.M;
    if (m0 >= M) return;
    const int t = tid(), lane = lane_id(), w = wave_id();
    if (t < 128)
    {
        const int r = min(m0 + t, M - 1);
        rowmap[t] = a.grp_rows ? a.grp_rows[a.grp_offset[z] + r] : r;
    }
    block_sync();
    // staging: thread t brings chunk (t & 3) of rows (t >> 2) and (t >> 2) + 64 of both slices
    const int sr = t >> 2, sc = (t & 3) * 8;
    const u16* xp0 = (const u16*)a.x + (long long)z * a.sxb + (long long)(rowmap[sr] / a.x_div) * a.ldx + sc;
    const u16* xp1 = (const u16*)a.x + (long long)z * a.sxb + (long long)(rowmap[sr + 64] / a.x_div) * a.ldx + sc;
    const u16* wp0 = (const u16*)a.w + (long long)z * a.swb + (long long)min(n0 + sr, a.N - 1) * a.ldw + sc;
    const u16* wp1 = (const u16*)a.w + (long long)z * a.swb + (long long)min(n0 + sr + 64, a.N - 1) * a.ldw + sc;
    const u32x4 zero = {0u, 0u, 0u, 0u};
    const int li = lane & 15, kg = (lane >> 4) * 8;
    const int wm = (w >> 1) * 64, wn = (w & 1) * 64;
    f32x4 acc[4][4];
    #pragma unroll
    for (int i = 0; i < 4; i++)
        #pragma unroll
        for (int j = 0; j < 4; j++) acc[i][j] = (f32x4){0.0f, 0.0f, 0.0f, 0.0f};

    u32x4 ra0, ra1, rb0, rb1;
    {
        const bool live = sc < a.K;
        ra0 = live ? *(const u32x4*)xp0 : zero; ra1 = live ? *(const u32x4*)xp1 : zero;
        rb0 = live ? *(const u32x4*)wp0 : zero; rb1 = live ? *(const u32x4*)wp1 : zero;
    }
    *(u32x4*)&As[0][sr * LT_STRIDE + sc] = ra0; *(u32x4*)&As[0][(sr + 64) * LT_STRIDE + sc] = ra1;
    *(u32x4*)&Bs[0][sr * LT_STRIDE + sc] = rb0; *(u32x4*)&Bs[0][(sr + 64) * LT_STRIDE + sc] = rb1;
    block_sync();
    int stage = 0;
    for (int k0 = 0; k0 < a.K; k0 += 32)
    {
        const int kn = k0 + 32;
        if (kn < a.K)
        {
            const bool live = kn + sc < a.K;
            ra0 = live ? *(const u32x4*)(xp0 + kn) : zero; ra1 = live ? *(const u32x4*)(xp1 + kn) : zero;
            rb0 = live ? *(const u32x4*)(wp0 + kn) : zero; rb1 = live ? *(const u32x4*)(wp1 + kn) : zero;
        }
        u32x4 af[4], bf[4];
        #pragma unroll
        for (int i = 0; i < 4; i++) af[i] = *(const u32x4*)&As[stage][(wm + 16 * i + li) * LT_STRIDE + kg];
        #pragma unroll
        for (int j = 0; j < 4; j++) bf[j] = *(const u32x4*)&Bs[stage][(wn + 16 * j + li) * LT_STRIDE + kg];
        #pragma unroll
        for (int i = 0; i < 4; i++)
            #pragma unroll
            for (int j = 0; j < 4; j++) acc[i][j] = mfma_16x16x32_bf16(af[i], bf[j], acc[i][j]);
        if (kn < a.K)
        {
            const int o = stage ^ 1;
            *(u32x4*)&As[o][sr * LT_STRIDE + sc] = ra0; *(u32x4*)&As[o][(sr + 64) * LT_STRIDE + sc] = ra1;
            *(u32x4*)&Bs[o][sr * LT_STRIDE + sc] = rb0; *(u32x4*)&Bs[o][(sr + 64) * LT_STRIDE + sc] = rb1;
        }
        block_sync();
        stage ^= 1;
    }
    #pragma unroll
    for (int i = 0; i < 4; i++)
        #pragma unroll
        for (int r = 0; r < 4; r++)
        {
            const int rl = wm + 16 * i + 4 * (lane >> 4) + r;
            if (m0 + rl >= M) continue;
            const long long row = rowmap[rl];
            #pragma unroll
            for (int j = 0; j < 4; j++)
            {
                const int n = n0 + wn + 16 * j + li;
                if (n >= a.N) continue;
                float aux = 0.0f;
                if (EPI_READS_AUX(a.epi)) aux = a.aux[(long long)z * a.sauxb + row * a.ldaux + EPI_AUX_COL(a.epi, n)];
                st1<TY>((TY*)a.y + (long long)z * a.syb + row * a.ldy + n, lin_epilogue(a.epi, acc[i][j][r] + (a.bias ? a.bias[n] : 0.0f), aux, a.limit));
            }
        }
}

// ---- host -------------------------------------------------------------------------------------------------------------------

template <typename T, typename TY, bool VEC>
static void launch_rows(const LinArgs& a, int batch, hipStream_t s)
{
    if (a.w_sel) { LAUNCH((lin_rows_kernel<T, TY, 1, VEC>), dim3((a.N + 3) / 4, a.M, batch), dim3(256), 0, s, a); return; }
    if (a.M <= 1) LAUNCH((lin_rows_kernel<T, TY, 1, VEC>), dim3((a.N + 3) / 4, 1, batch), dim3(256), 0, s, a);
    else if (a.M <= 2) LAUNCH((lin_rows_kernel<T, TY, 2, VEC>), dim3((a.N + 3) / 4, 1, batch), dim3(256), 0, s, a);
    else if (a.M <= 4) LAUNCH((lin_rows_kernel<T, TY, 4, VEC>), dim3((a.N + 3) / 4, 1, batch), dim3(256), 0, s, a);
    else LAUNCH((lin_rows_kernel<T, TY, 8, VEC>), dim3((a.N + 3) / 4, (a.M + 7) / 8, batch), dim3(256), 0, s, a);
}

template <typename T, typename TY>
static void launch_dense(const LinArgs& a, int batch, bool vec_ok, int max_rows, hipStream_t s)
{
    if (a.w_sel || (!a.grp_count && a.M <= 16))
    {
        if (vec_ok) launch_rows<T, TY, true>(a, batch, s); else launch_rows<T, TY, false>(a, batch, s);
        return;
    }
    if constexpr (sizeof(T) == 2)
    {
        if (vec_ok)
        {
            if (max_rows <= 32) LAUNCH((lin_mfma_kernel<TY, 2>), dim3((a.N + 255) / 256, (max_rows + 31) / 32, batch), dim3(256), 0, s, a);
            else if (max_rows <= 64) LAUNCH((lin_mfma_kernel<TY, 4>), dim3((a.N + 255) / 256, (max_rows + 63) / 64, batch), dim3(256), 0, s, a);
            else LAUNCH((lin_mfma_tile_kernel<TY>), dim3((a.N + 127) / 128, (max_rows + 127) / 128, batch), dim3(256), 0, s, a);
            return;
        }
    }
    LAUNCH((lin_tile_kernel<T, TY>), dim3((a.N + 63) / 64, (max_rows + 63) / 64, batch), dim3(256), 0, s, a);
}

extern "C" int exl2_dense_linear_bias(const void* x, const void* w, const float* bias, void* y, const float* aux, int dtype, int y_f32,
                                      int M, int N, int K, int ldx, int ldw, int ldy, int ldaux,
                                      int batch, long long sxb, long long swb, long long syb, long long sauxb,
                                      const int* w_sel, int n_sel, const int* grp_count, const int* grp_offset, const int* grp_rows,
                                      int x_div, int epi, float limit, void* stream);

extern "C" int exl2_dense_linear(const void* x, const void* w, void* y, const float* aux, int dtype, int y_f32,
                                 int M, int N, int K, int ldx, int ldw, int ldy, int ldaux,
                                 int batch, long long sxb, long long swb, long long syb, long long sauxb,
                                 const int* w_sel, int n_sel, const int* grp_count, const int* grp_offset, const int* grp_rows,
                                 int x_div, int epi, float limit, void* stream)
{
    return exl2_dense_linear_bias(x, w, nullptr, y, aux, dtype, y_f32, M, N, K, ldx, ldw, ldy, ldaux, batch, sxb, swb, syb, sauxb,
                                  w_sel, n_sel, grp_count, grp_offset, grp_rows, x_div, epi, limit, stream);
}

extern "C" int exl2_dense_linear_bias(const void* x, const void* w, const float* bias, void* y, const float* aux, int dtype, int y_f32,
                                      int M, int N, int K, int ldx, int ldw, int ldy, int ldaux,
                                      int batch, long long sxb, long long swb, long long syb, long long sauxb,
                                      const int* w_sel, int n_sel, const int* grp_count, const int* grp_offset, const int* grp_rows,
                                      int x_div, int epi, float limit, void* stream)
{
    EXL2_REQUIRE(x && w && y, "dense_linear: null operand");
    EXL2_REQUIRE(dtype == DENSE_BF16 || dtype == DENSE_F32, "dense_linear: dtype must be 0 (bfloat16) or 1 (float32)");
    EXL2_REQUIRE(M >= 0 && N > 0 && K > 0 && batch > 0 && x_div > 0, "dense_linear: bad shape %d x %d x %d, batch %d", M, N, K, batch);
    EXL2_REQUIRE(ldx >= K || x_div > 0, "dense_linear: ldx"); EXL2_REQUIRE(ldw >= K && ldy > 0, "dense_linear: leading dimensions");
    EXL2_REQUIRE(epi >= EPI_NONE && epi <= EPI_LAST, "dense_linear: unknown epilogue %d", epi);
    EXL2_REQUIRE(!EPI_READS_AUX(epi) || aux, "dense_linear: the epilogue needs aux");
    EXL2_REQUIRE(epi != EPI_SOFT_CAP || limit > 0.0f, "dense_linear: the soft cap needs a positive limit");
    EXL2_REQUIRE(!bias || (batch == 1 && !w_sel && !grp_count), "dense_linear: a bias goes with a plain (one-slab) call");
    EXL2_REQUIRE(!(w_sel && grp_count), "dense_linear: w_sel and groups exclude each other");
    EXL2_REQUIRE(!grp_count || (grp_offset && grp_rows), "dense_linear: grouped call without offsets / row lists");
    EXL2_REQUIRE(dtype == DENSE_BF16 || y_f32, "dense_linear: float32 operands give float32 results");
    if (M == 0) return EXL2_OK;
    LinArgs a;
    a.x = x; a.w = w; a.y = y; a.aux = aux; a.bias = bias; a.M = M; a.N = N; a.K = K; a.ldx = ldx; a.ldw = ldw; a.ldy = ldy; a.ldaux = ldaux;
    a.sxb = sxb; a.swb = swb; a.syb = syb; a.sauxb = sauxb; a.w_sel = w_sel; a.n_sel = n_sel;
    a.grp_count = grp_count; a.grp_offset = grp_offset; a.grp_rows = grp_rows; a.x_div = x_div; a.epi = epi; a.limit = limit;
    const int es = dtype == DENSE_BF16 ? 2 : 4, v = 16 / es;
    // 16-byte loads: every row start and every step must stay aligned
    const bool vec_ok = K % v == 0 && ldx % v == 0 && ldw % v == 0 && sxb % v == 0 && swb % v == 0
                        && ((uintptr_t)x % 16) == 0 && ((uintptr_t)w % 16) == 0;
    hipStream_t s = (hipStream_t)stream;
    if (dtype == DENSE_F32) launch_dense<float, float>(a, batch, vec_ok, M, s);
    else if (y_f32) launch_dense<u16, float>(a, batch, vec_ok, M, s);
    else launch_dense<u16, u16>(a, batch, vec_ok, M, s);
    HIP_TRY(hipGetLastError());
    return EXL2_OK;
}
