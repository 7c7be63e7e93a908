// latent_attn.hip -- attention over a compressed (latent) KV cache with a sliding window, for gfx950, + its C ABI.
//
// A token's cache row is [c (kv_rank values, RMS-normed) | k_rot (rot values, rotated by the token's position)], shared by all
// heads; rows live in pages of a pool ([pages, page, kv_rank + rot]) reached through a per-sequence block table.  A head's key is
// W_uk c and its value W_uv c, so with q_abs = W_uk^T q_nope (a batched dense linear) the score is
//     s_j = (q_abs . c_j + rot(q_rot, p) . k_rot_j) * scale            over  max(0, p - window + 1) <= j <= p,
// and the head's output in latent space is sum_j softmax(s)_j c_j; W_uv is applied afterwards (another batched linear).  Nothing
// per head is ever materialised for a cached token, in prompts and in decoding alike.
//
// Rows of a step are a flat list: row r belongs to sequence row_seq[r] (a block-table row) at position row_pos[r]; prompt
// portions of several requests and single decoded tokens go through the same launch, and a row's result depends only on its own
// (sequence, position).  Scores, softmax and the weighted sum are fp32; positions and angles are fp32 with the inverse
// frequencies passed in as a table (made in double precision on the host).
// Interleaved rotary layout: dimension 2i is paired with 2i + 1, angle p * inv_freq[i]; dimensions past rot_dims pass unchanged.
#include "hw.h"
#include "errors.h"

template <typename T> DEV float la_ld(const T* p);
template <> DEV float la_ld<u16>(const u16* p) { return bf16_to_f32(*p); }
template <> DEV float la_ld<float>(const float* p) { return *p; }
template <typename T> DEV void la_st(T* p, float v);
template <> DEV void la_st<u16>(u16* p, float v) { *p = f32_to_bf16(v); }
template <> DEV void la_st<float>(float* p, float v) { *p = v; }

DEV float la_block_sum(float v, float* part)
{
    v = wave_allreduce_add(v);
    block_sync();
    if (lane_id() == 0) part[wave_id()] = v;
    block_sync();
    return part[0] + part[1] + part[2] + part[3];
}
DEV float la_block_max(float v, float* part)
{
    v = wave_allreduce_max(v);
    block_sync();
    if (lane_id() == 0) part[wave_id()] = v;
    block_sync();
    return fmaxf(fmaxf(part[0], part[1]), fmaxf(part[2], part[3]));
}

// ---- new rows into the cache: RMS norm of the latent, rotation of the shared key part ----------------------------------------

struct LatAppendArgs
{
    const float* dkv; int ld;                // [rows, ld]: kv_rank latent values then rot key values
    const void* norm_w; float eps;
    int R, rot, rot_dims;
    const float* inv_freq;
    const int* row_seq; const int* row_pos; const int* block_table; int bt_stride, page;
    void* cache;
};

template <typename T>
KERNEL void __launch_bounds__(256) latent_append_kernel(const LatAppendArgs a)
{
    SHARED float part[4];
    const int r = bid_x();
    const float* src = a.dkv + (long long)r * a.ld;
    const int pos = a.row_pos[r];
    const int pg = a.block_table[(long long)a.row_seq[r] * a.bt_stride + pos / a.page];
    T* dst = (T*)a.cache + ((long long)pg * a.page + pos % a.page) * (a.R + a.rot);
    float ss = 0.0f;
    for (int i = tid(); i < a.R; i += 256) { const float v = src[i]; ss = fmaf(v, v, ss); }
    ss = la_block_sum(ss, part);
    const float rinv = 1.0f / sqrtf(ss / (float)a.R + a.eps);
    for (int i = tid(); i < a.R; i += 256) la_st<T>(dst + i, src[i] * rinv * la_ld<T>((const T*)a.norm_w + i));
    const float* ks = src + a.R;
    for (int i = tid(); i < a.rot_dims / 2; i += 256)
    {
        const float ang = (float)pos * a.inv_freq[i];
        const float c = cosf(ang), s = sinf(ang);
        const float u = ks[2 * i], v = ks[2 * i + 1];
        la_st<T>(dst + a.R + 2 * i, u * c - v * s);
        la_st<T>(dst + a.R + 2 * i + 1, v * c + u * s);
    }
    for (int i = a.rot_dims + tid(); i < a.rot; i += 256) la_st<T>(dst + a.R + i, ks[i]);
}

// ---- attention ----------------------------------------------------------------------------------------------------------------

struct LatAttnArgs
{
    const void* q; int ldq, q_head_stride, q_rot_off;      // rotated part of head h of row r: q[r * ldq + h * q_head_stride + q_rot_off ..]
    const float* q_abs;                                     // [rows, H, R]
    const void* cache; int page;
    const int* row_seq; const int* row_pos; const int* block_table; int bt_stride;
    void* out;                                              // [rows, H, R]
    int H, R, rot, rot_dims;
    const float* inv_freq;
    float scale; int window;
};

#define LA_MAX_R_PER_THREAD 4

// Workgroup = one (row, head).  Keys are taken 256 at a time: thread t scores key t of the chunk (a dot product over the whole
// cache row), the chunk joins the running softmax, then thread t owns latent elements t, t + 256, .. of the weighted sum.
template <typename T>
KERNEL void __launch_bounds__(256) latent_attn_kernel(const LatAttnArgs a)
{
    DYN_SMEM(smem);
    SHARED float part[4];
    SHARED float prob[256];
    SHARED long long koff[256];
    float* qv = (float*)smem;                               // [R + rot]
    const int r = bid_x(), h = bid_y();
    const int t = tid();
    const int D = a.R + a.rot;
    const int pos = a.row_pos[r];
    const int* bt = a.block_table + (long long)a.row_seq[r] * a.bt_stride;
    const float* qa = a.q_abs + ((long long)r * a.H + h) * a.R;
    for (int i = t; i < a.R; i += 256) qv[i] = qa[i];
    const T* qr = (const T*)a.q + (long long)r * a.ldq + (long long)h * a.q_head_stride + a.q_rot_off;
    for (int i = t; i < a.rot_dims / 2; i += 256)
    {
        const float ang = (float)pos * a.inv_freq[i];
        const float c = cosf(ang), s = sinf(ang);
        const float u = la_ld<T>(qr + 2 * i), v = la_ld<T>(qr + 2 * i + 1);
        qv[a.R + 2 * i] = u * c - v * s;
        qv[a.R + 2 * i + 1] = v * c + u * s;
    }
    for (int i = a.rot_dims + t; i < a.rot; i += 256) qv[a.R + i] = la_ld<T>(qr + i);
    block_sync();

    const int j_lo = max(0, pos - a.window + 1);
    const int nkeys = pos - j_lo + 1;
    float m_run = -INFINITY, l_run = 0.0f;
    float acc[LA_MAX_R_PER_THREAD];
    #pragma unroll
    for (int e = 0; e < LA_MAX_R_PER_THREAD; e++) acc[e] = 0.0f;
    const T* cache = (const T*)a.cache;
    for (int c0 = 0; c0 < nkeys; c0 += 256)
    {
        const int nc = min(256, nkeys - c0);
        float s = -INFINITY;
        if (t < nc)
        {
            const int j = j_lo + c0 + t;
            const long long off = ((long long)bt[j / a.page] * a.page + j % a.page) * D;
            koff[t] = off;
            const T* kr = cache + off;
            float d = 0.0f;
            for (int i = 0; i < D; i++) d = fmaf(qv[i], la_ld<T>(kr + i), d);
            s = d * a.scale;
        }
        const float m_new = fmaxf(m_run, la_block_max(s, part));
        const float p = t < nc ? expf(s - m_new) : 0.0f;
        prob[t] = p;
        const float corr = expf(m_run - m_new);             // exp(-inf) = 0 on the first chunk
        l_run = l_run * corr + la_block_sum(p, part);       // (its barriers also publish prob and koff)
        m_run = m_new;
        #pragma unroll
        for (int e = 0; e < LA_MAX_R_PER_THREAD; e++)
        {
            const int i = t + 256 * e;
            if (i >= a.R) break;
            float o = acc[e] * corr;
            for (int jj = 0; jj < nc; jj++) o = fmaf(prob[jj], la_ld<T>(cache + koff[jj] + i), o);
            acc[e] = o;
        }
        block_sync();                                       // prob / koff are rewritten by the next chunk
    }
    T* out = (T*)a.out + ((long long)r * a.H + h) * a.R;
    #pragma unroll
    for (int e = 0; e < LA_MAX_R_PER_THREAD; e++)
    {
        const int i = t + 256 * e;
        if (i < a.R) la_st<T>(out + i, acc[e] / l_run);
    }
}

// ---- C ABI --------------------------------------------------------------------------------------------------------------------

extern "C" int exl2_latent_append(const float* dkv, int ld, const void* norm_w, float eps, int dtype, int rows, int kv_rank, int rot,
                                  int rot_dims, const float* inv_freq, const int* row_seq, const int* row_pos, const int* block_table,
                                  int bt_stride, int page, void* cache, void* stream)
{
    EXL2_REQUIRE(dkv && norm_w && inv_freq && row_seq && row_pos && block_table && cache, "latent_append: null operand");
    EXL2_REQUIRE(dtype == 0 || dtype == 1, "latent_append: dtype must be 0 (bfloat16) or 1 (float32)");
    EXL2_REQUIRE(kv_rank > 0 && rot >= 0 && rot_dims >= 0 && rot_dims <= rot && rot_dims % 2 == 0 && ld >= kv_rank + rot && page > 0,
                 "latent_append: bad shape (kv_rank %d, rot %d, rot_dims %d, ld %d, page %d)", kv_rank, rot, rot_dims, ld, page);
    if (rows <= 0) return EXL2_OK;
    LatAppendArgs a;
    a.dkv = dkv; a.ld = ld; a.norm_w = norm_w; a.eps = eps; a.R = kv_rank; a.rot = rot; a.rot_dims = rot_dims; a.inv_freq = inv_freq;
    a.row_seq = row_seq; a.row_pos = row_pos; a.block_table = block_table; a.bt_stride = bt_stride; a.page = page; a.cache = cache;
    if (dtype == 0) LAUNCH(latent_append_kernel<u16>, dim3(rows), dim3(256), 0, stream, a);
    else LAUNCH(latent_append_kernel<float>, dim3(rows), dim3(256), 0, stream, a);
    HIP_TRY(hipGetLastError());
    return EXL2_OK;
}

extern "C" int exl2_latent_attn(const void* q, int ldq, int q_head_stride, int q_rot_off, const float* q_abs, const void* cache, int page,
                                const int* row_seq, const int* row_pos, const int* block_table, int bt_stride, void* out, int dtype,
                                int rows, int heads, int kv_rank, int rot, int rot_dims, const float* inv_freq, float scale, int window,
                                void* stream)
{
    EXL2_REQUIRE(q && q_abs && cache && row_seq && row_pos && block_table && out && inv_freq, "latent_attn: null operand");
    EXL2_REQUIRE(dtype == 0 || dtype == 1, "latent_attn: dtype must be 0 (bfloat16) or 1 (float32)");
    EXL2_REQUIRE(heads > 0 && kv_rank > 0 && kv_rank <= 256 * LA_MAX_R_PER_THREAD, "latent_attn: kv_rank %d (at most %d)", kv_rank, 256 * LA_MAX_R_PER_THREAD);
    EXL2_REQUIRE(rot >= 0 && rot_dims >= 0 && rot_dims <= rot && rot_dims % 2 == 0 && page > 0 && window > 0,
                 "latent_attn: bad shape (rot %d, rot_dims %d, page %d, window %d)", rot, rot_dims, page, window);
    if (rows <= 0) return EXL2_OK;
    LatAttnArgs a;
    a.q = q; a.ldq = ldq; a.q_head_stride = q_head_stride; a.q_rot_off = q_rot_off; a.q_abs = q_abs; a.cache = cache; a.page = page;
    a.row_seq = row_seq; a.row_pos = row_pos; a.block_table = block_table; a.bt_stride = bt_stride; a.out = out;
    a.H = heads; a.R = kv_rank; a.rot = rot; a.rot_dims = rot_dims; a.inv_freq = inv_freq; a.scale = scale; a.window = window;
    const size_t smem = (size_t)(kv_rank + rot) * 4;
    if (dtype == 0) LAUNCH(latent_attn_kernel<u16>, dim3(rows, heads), dim3(256), smem, stream, a);
    else LAUNCH(latent_attn_kernel<float>, dim3(rows, heads), dim3(256), smem, stream, a);
    HIP_TRY(hipGetLastError());
    return EXL2_OK;
}
