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
#include "hw.h"
#include "errors.h"

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
    for (int i = t; i < (a.H + a.G) * per; i += 256)
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

// grid (rows): a row whose position completes a block (pos % pool == pool - 1) writes that block's mean key and value row, read
// back from the cache as it holds them; other rows leave at once.
template <typename T>
KERNEL void __launch_bounds__(256) pool_blocks_kernel(const PoolArgs a)
{
    const int r = bid_x(), t = tid();
    const int pos = a.row_pos[r];
    if (pos % a.pool != a.pool - 1) return;
    const int* bt = a.block_table + (long long)a.row_seq[r] * a.bt_stride;
    const int p0 = pos - (a.pool - 1);
    const long long dst = (long long)bt[p0 / a.page] * a.per_page + (p0 % a.page) / a.pool;
    const float inv = 1.0f / (float)a.pool;
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
};

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
    const int j_lo = max(0, pos - a.window + 1);
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
            s = d;
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
    const float* gt = a.gate ? a.gate + (long long)r * a.ldg + h * a.vdim : nullptr;
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
        wa_st<T>(out + ia, u);
        wa_st<T>(out + ib, v);
    }
    if ((a.vdim & 1) && t == 0)
    {
        float u = ov[a.vdim - 1];
        if (gt) u *= 1.0f / (1.0f + expf(-gt[a.vdim - 1]));
        wa_st<T>(out + a.vdim - 1, u);
    }
}

// ---- C ABI ----------------------------------------------------------------------------------------------------------------------

extern "C" int exl2_kv_rot_append(const float* f, int ld, int q_off, int k_off, int v_off, void* q_out, const float* q_scale,
                                  void* k_cache, void* v_cache, void* k_pool, void* v_pool, const float* freq, float amp, int rot_dims,
                                  const float* vfreq, int v_rot, int interleaved, const int* row_seq, const int* row_pos,
                                  const int* block_table, int bt_stride, int page, int pool, int dtype, int rows, int heads,
                                  int kv_heads, int dim, int vdim, void* stream)
{
    EXL2_REQUIRE(f && q_out && q_scale && k_cache && v_cache && freq && row_seq && row_pos && block_table, "kv_rot_append: null operand");
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
        if (dtype == 0) LAUNCH(pool_blocks_kernel<u16>, dim3(rows), dim3(256), 0, stream, p);
        else LAUNCH(pool_blocks_kernel<float>, dim3(rows), dim3(256), 0, stream, p);
    }
    HIP_TRY(hipGetLastError());
    return EXL2_OK;
}

extern "C" int exl2_window_attn(const void* q, const void* k_cache, const void* v_cache, const void* k_pool, const void* v_pool,
                                const float* sink, const float* gate, int ldg, const float* vfreq, int v_rot, int interleaved,
                                const int* row_seq, const int* row_pos, const int* block_table, int bt_stride, int page, int pool,
                                void* out, int dtype, int rows, int heads, int kv_heads, int dim, int vdim, int window, void* stream)
{
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
    a.H = heads; a.G = kv_heads; a.dim = dim; a.vdim = vdim; a.window = window;
    const size_t smem = (size_t)(dim + vdim) * 4;
    if (dtype == 0) LAUNCH(window_attn_kernel<u16>, dim3(rows, heads), dim3(256), smem, stream, a);
    else LAUNCH(window_attn_kernel<float>, dim3(rows, heads), dim3(256), smem, stream, a);
    HIP_TRY(hipGetLastError());
    return EXL2_OK;
}
