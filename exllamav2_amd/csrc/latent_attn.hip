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

// ---- bfloat16 on the matrix cores ----------------------------------------------------------------------------------------------
// A wave owns 16 query vectors that share their keys: TR = 16: sixteen consecutive positions of one sequence x one head (a prompt's
// portion; the four waves of a workgroup take four heads), TR = 1: one position x sixteen heads (a decoded token).  Keys go by in
// steps of 32: the workgroup stages the step's cache rows in LDS twice -- row-major for S = Q C^T (both operands K-contiguous) and
// transposed ([latent element][key]) for O += P C, whose B operand wants 8 consecutive KEYS of one latent element per lane.  The
// scores leave the accumulators through a wave-private LDS tile (laid over the row-major copy once all waves have used it) to become
// the A operand of the second product.  Softmax state
// (running maximum, sum) is per query row = per accumulator row, kept in registers; fp32 throughout, P rounded to bfloat16 for the
// matrix core.  grid.z > 1 splits the key steps over workgroups (decoding against a long window): partial (m, l, O) go to
// scratch and latent_attn_merge_kernel joins them.

struct LatMfmaArgs
{
    const u16* q; int ldq, q_head_stride, q_rot_off;
    const float* q_abs;
    const u16* cache; int page;
    const int* row_seq; const int* row_pos; const int* block_table; int bt_stride;
    const int* tile_row0; const int* tile_rows;
    u16* out;
    float* part_o; float* part_ml; int nsplit;
    int H, R, rot, rot_dims;
    const float* inv_freq;
    float scale; int window;
    int DP;                                                  // kv_rank + rot rounded up to a multiple of 32
};

#define LA_KT 32
#define LA_TS 40                                             // row stride (values) of the transposed and the probability tiles
#define LA_ROT_STEPS 4
#define LA_MAX_SPLIT 32
#define LA_STAGE_IT 10                                       // 16-byte chunks per thread and key step: (512 + 128) / 8 / 8

DEV u32 la_pack2(float lo, float hi) { return (u32)f32_to_bf16(lo) | ((u32)f32_to_bf16(hi) << 16); }

// RS > 0: the EXACT form -- kv_rank == 16 NT and rot == 32 RS are compile-time constants, so every size guard below folds away and the
// unrolled loops become straight-line code the scheduler can reorder (LDS reads of the next fragments ahead of the current matrix
// products).  RS == 0: sizes from the arguments (any kv_rank % 32 == 0, rot % 8 == 0).
template <int NT, int TR, int RS>
KERNEL void __launch_bounds__(256) latent_attn_mfma_kernel(const LatMfmaArgs a)
{
    DYN_SMEM(smem);
    const int tile = bid_x(), hb = bid_y(), split = bid_z();
    const int w = wave_id(), lane = lane_id(), li = lane & 15, g = lane >> 4, t = tid();
    const int r0 = a.tile_row0[tile];
    const int n = TR == 16 ? a.tile_rows[tile] : 1;
    const int p0 = a.row_pos[r0];
    const int* bt = a.block_table + (long long)a.row_seq[r0] * a.bt_stride;
    const int H = a.H;
    const int R = RS > 0 ? NT * 16 : a.R, rot = RS > 0 ? RS * 32 : a.rot;
    const int D = R + rot, DP = RS > 0 ? D : a.DP, CS = DP + 8;
    u16* Cs = (u16*)smem;                                    // [32][CS]
    u16* Ct = Cs + LA_KT * CS;                               // [R][LA_TS]
    u16* Ps = Cs + w * 16 * LA_TS;                           // [16][LA_TS], this wave's: OVER the row-major copy, once every wave is done with it

    // the query vector this lane feeds as A-operand row li
    int qrow, qhead;
    if (TR == 16) { qrow = r0 + min(li, n - 1); qhead = hb * 4 + w; }
    else { qrow = r0; qhead = (hb * 4 + w) * 16 + li; }
    const bool wave_live = (TR == 16 ? hb * 4 + w : (hb * 4 + w) * 16) < H;
    const int qh = min(qhead, H - 1);
    const int qpos = a.row_pos[qrow];

    constexpr int KSC = NT / 2;
    u32x4 qf[KSC + LA_ROT_STEPS];
    {
        // (all loads of a batch of 8 k-steps first, then the conversions: a conversion right behind its load makes every k-step a
        // memory round trip of its own)
        const float* qa = a.q_abs + ((long long)qrow * H + qh) * R;
        #pragma unroll
        for (int k0 = 0; k0 < KSC; k0 += 8)
        {
            f32x4 lo[8], hi[8];
            #pragma unroll
            for (int j = 0; j < 8; j++)
            {
                const int ks = min(k0 + j, KSC - 1);
                const int off = min(ks * 32, R - 32) + 8 * g;          // (clamped: k-steps past kv_rank re-read the last one and are zeroed below)
                lo[j] = *(const f32x4*)(qa + off);
                hi[j] = *(const f32x4*)(qa + off + 4);
            }
            #pragma unroll
            for (int j = 0; j < 8; j++)
            {
                const int ks = k0 + j;
                if (ks >= KSC) continue;
                qf[ks] = ks * 32 < R ? (u32x4){la_pack2(lo[j][0], lo[j][1]), la_pack2(lo[j][2], lo[j][3]), la_pack2(hi[j][0], hi[j][1]), la_pack2(hi[j][2], hi[j][3])}
                                     : (u32x4){0u, 0u, 0u, 0u};
            }
        }
        const u16* qr = a.q + (long long)qrow * a.ldq + (long long)qh * a.q_head_stride + a.q_rot_off;
        #pragma unroll
        for (int ks = 0; ks < LA_ROT_STEPS; ks++)
        {
            u32x4 v = {0u, 0u, 0u, 0u};
            if (ks * 32 < rot)
            {
                #pragma unroll
                for (int e2 = 0; e2 < 4; e2++)
                {
                    const int i0 = ks * 32 + 8 * g + 2 * e2;
                    float x0 = 0.0f, x1 = 0.0f;
                    if (i0 < rot)
                    {
                        x0 = bf16_to_f32(qr[i0]); x1 = bf16_to_f32(qr[i0 + 1]);
                        if (i0 < a.rot_dims)
                        {
                            // (bfloat16 path: two-term reduction of the fp32 angle to [-pi, pi], then the hardware sine / cosine -- the
                            // library functions' large-argument path costs microseconds per call in a prologue that runs once per key split)
                            const float ang = (float)qpos * a.inv_freq[i0 >> 1];
                            const float nrev = rintf(ang * 0.15915494309189535f);
                            const float red = fmaf(-nrev, -1.7484555e-07f, fmaf(-nrev, 6.2831855f, ang));
                            const float c = fast_cos(red), sn = fast_sin(red);
                            const float u = x0, vv = x1;
                            x0 = u * c - vv * sn; x1 = vv * c + u * sn;
                        }
                    }
                    v[e2] = la_pack2(x0, x1);
                }
            }
            qf[KSC + ks] = v;
        }
    }

    f32x4 acc[NT];
    #pragma unroll
    for (int nt = 0; nt < NT; nt++) acc[nt] = (f32x4){0.0f, 0.0f, 0.0f, 0.0f};
    float m_run[4], l_run[4];
    #pragma unroll
    for (int r = 0; r < 4; r++) { m_run[r] = -INFINITY; l_run[r] = 0.0f; }

    const int k_lo = max(0, p0 - a.window + 1), k_hi = p0 + n - 1;
    const int steps = (k_hi - k_lo + 1 + LA_KT - 1) / LA_KT;
    const int per_split = (steps + a.nsplit - 1) / a.nsplit;
    const int s_begin = split * per_split, s_end = min(steps, s_begin + per_split);
    const int chunks_per_row = DP >> 3;
    // Staging, software-pipelined: thread t always brings key (t & 31) of a step -- chunks (t >> 5) + 8 i of that cache row -- so one
    // block-table lookup per thread and step names the row, and the row's 16-byte loads are independent of each other.  The loads
    // of step s + 1 are issued before the matrix products of step s and land in registers meanwhile; the row of step s + 2 is
    // looked up behind them.  (Consecutive threads = consecutive keys: the transposed 2-byte LDS stores of a wave are contiguous.)
    const int skey = t & (LA_KT - 1), sch0 = t >> 5;
    const u32x4 zero4 = {0u, 0u, 0u, 0u};
    u32x4 sv[LA_STAGE_IT];
    // the page of this thread's key in step st (a load) and, separately, the row offset made from it: the load is issued a whole step
    // before its value is consumed, so no wait for it ever sits behind freshly issued row loads
    auto key_page = [&](int st) -> int {
        const int j = min(k_lo + st * LA_KT + skey, k_hi);
        return bt[j / a.page];
    };
    auto key_row = [&](int pg, int st) -> long long {
        const int j = min(k_lo + st * LA_KT + skey, k_hi);
        return ((long long)pg * a.page + j % a.page) * D;
    };
    auto issue = [&](long long rowoff) {
        #pragma unroll
        for (int it = 0; it < LA_STAGE_IT; it++)
        {
            const int ch = sch0 + 8 * it;
            sv[it] = ch * 8 < D ? *(const u32x4*)(a.cache + rowoff + ch * 8) : zero4;
        }
    };
    auto commit = [&]() {
        #pragma unroll
        for (int it = 0; it < LA_STAGE_IT; it++)
        {
            const int ch = sch0 + 8 * it;
            if (ch >= chunks_per_row) continue;
            const u32x4 v = sv[it];
            *(u32x4*)(Cs + skey * CS + ch * 8) = v;
            if (ch * 8 < R)
            {
                #pragma unroll
                for (int e = 0; e < 4; e++)
                {
                    Ct[(ch * 8 + 2 * e) * LA_TS + skey] = (u16)(v[e] & 0xffffu);
                    Ct[(ch * 8 + 2 * e + 1) * LA_TS + skey] = (u16)(v[e] >> 16);
                }
            }
        }
    };
    int pg_next = 0;
    if (s_begin < s_end)
    {
        issue(key_row(key_page(s_begin), s_begin));
        if (s_begin + 1 < s_end) pg_next = key_page(s_begin + 1);
    }

    for (int st = s_begin; st < s_end; st++)
    {
        const int kbase = k_lo + st * LA_KT;
        commit();
        block_sync_lds();                                 // (LDS-only barriers: the loads issued below stay in flight across them)
        if (st + 1 < s_end)
        {
            issue(key_row(pg_next, st + 1));
            if (st + 2 < s_end) pg_next = key_page(st + 2);
        }
        float corr[4], pe0[4], pe1[4];
        if (wave_live)
        {
            f32x4 s0 = {0.0f, 0.0f, 0.0f, 0.0f}, s1 = {0.0f, 0.0f, 0.0f, 0.0f};
            // (operand reads in batches of four k-steps ahead of their products: one wave per SIMD has nobody else to hide LDS latency)
            #pragma unroll
            for (int k0 = 0; k0 < KSC; k0 += 4)
            {
                u32x4 b0[4], b1[4];
                #pragma unroll
                for (int j = 0; j < 4; j++)
                    if (k0 + j < KSC && (k0 + j) * 32 < R)
                    {
                        b0[j] = *(const u32x4*)(Cs + li * CS + (k0 + j) * 32 + 8 * g);
                        b1[j] = *(const u32x4*)(Cs + (16 + li) * CS + (k0 + j) * 32 + 8 * g);
                    }
                #pragma unroll
                for (int j = 0; j < 4; j++)
                    if (k0 + j < KSC && (k0 + j) * 32 < R)
                    {
                        s0 = mfma_16x16x32_bf16(qf[k0 + j], b0[j], s0);
                        s1 = mfma_16x16x32_bf16(qf[k0 + j], b1[j], s1);
                    }
            }
            #pragma unroll
            for (int ks = 0; ks < LA_ROT_STEPS; ks++)
                if (ks * 32 < rot)
                {
                    const u32x4 b0 = *(const u32x4*)(Cs + li * CS + R + ks * 32 + 8 * g);
                    const u32x4 b1 = *(const u32x4*)(Cs + (16 + li) * CS + R + ks * 32 + 8 * g);
                    s0 = mfma_16x16x32_bf16(qf[KSC + ks], b0, s0);
                    s1 = mfma_16x16x32_bf16(qf[KSC + ks], b1, s1);
                }
            #pragma unroll
            for (int r = 0; r < 4; r++)
            {
                const int qi = 4 * g + r;
                const int qp = TR == 16 ? p0 + qi : p0;
                const bool live_q = TR == 16 ? qi < n : true;
                const int j0 = kbase + li, j1 = kbase + 16 + li;
                const float v0 = live_q && j0 <= qp && j0 > qp - a.window ? s0[r] * a.scale : -INFINITY;
                const float v1 = live_q && j1 <= qp && j1 > qp - a.window ? s1[r] * a.scale : -INFINITY;
                const float mx = row16_allreduce_max(fmaxf(v0, v1));
                const float m_new = fmaxf(m_run[r], mx);
                const float m_safe = m_new == -INFINITY ? 0.0f : m_new;
                const float e0 = fast_exp(v0 - m_safe), e1 = fast_exp(v1 - m_safe);     // (bfloat16 path: the hardware exponential)
                corr[r] = fast_exp(m_run[r] - m_safe);
                l_run[r] = l_run[r] * corr[r] + row16_allreduce_add(e0 + e1);
                m_run[r] = m_new;
                pe0[r] = e0; pe1[r] = e1;
            }
        }
        block_sync_lds();                                 // every wave has read its S operands: the probability tiles may overwrite them
        if (wave_live)
        {
            #pragma unroll
            for (int r = 0; r < 4; r++)
            {
                Ps[(4 * g + r) * LA_TS + li] = f32_to_bf16(pe0[r]);
                Ps[(4 * g + r) * LA_TS + 16 + li] = f32_to_bf16(pe1[r]);
            }
        }
        block_sync_lds();
        if (wave_live)
        {
            const u32x4 pa = *(const u32x4*)(Ps + li * LA_TS + 8 * g);
            // the running maxima rarely move once a few steps have gone by: rescale the accumulators only when one did
            const bool moved = wave_ballot(corr[0] != 1.0f || corr[1] != 1.0f || corr[2] != 1.0f || corr[3] != 1.0f) != 0ull;
            if (moved)
            {
                #pragma unroll
                for (int nt = 0; nt < NT; nt++)
                    if (nt * 16 < R)
                    {
                        #pragma unroll
                        for (int r = 0; r < 4; r++) acc[nt][r] *= corr[r];
                    }
            }
            #pragma unroll
            for (int n0 = 0; n0 < NT; n0 += 8)
            {
                u32x4 b[8];
                #pragma unroll
                for (int j = 0; j < 8; j++)
                    if ((n0 + j) * 16 < R) b[j] = *(const u32x4*)(Ct + ((n0 + j) * 16 + li) * LA_TS + 8 * g);
                #pragma unroll
                for (int j = 0; j < 8; j++)
                    if ((n0 + j) * 16 < R) acc[n0 + j] = mfma_16x16x32_bf16(pa, b[j], acc[n0 + j]);
            }
        }
        block_sync_lds();
    }
    if (!wave_live) return;
    #pragma unroll
    for (int r = 0; r < 4; r++)
    {
        const int qi = 4 * g + r;
        int orow, ohead;
        if (TR == 16) { orow = r0 + qi; ohead = hb * 4 + w; if (qi >= n) continue; }
        else { orow = r0; ohead = (hb * 4 + w) * 16 + qi; if (ohead >= H) continue; }
        const long long vec = (long long)orow * H + ohead;
        if (a.nsplit == 1)
        {
            const float inv = 1.0f / l_run[r];
            #pragma unroll
            for (int nt = 0; nt < NT; nt++)
                if (nt * 16 < R) a.out[vec * R + nt * 16 + li] = f32_to_bf16(acc[nt][r] * inv);
        }
        else
        {
            float* po = a.part_o + (vec * a.nsplit + split) * R;
            #pragma unroll
            for (int nt = 0; nt < NT; nt++)
                if (nt * 16 < R) po[nt * 16 + li] = acc[nt][r];
            if (li == 0) { a.part_ml[(vec * a.nsplit + split) * 2] = m_run[r]; a.part_ml[(vec * a.nsplit + split) * 2 + 1] = l_run[r]; }
        }
    }
}

// joins the key splits of one query vector: out = sum_s e^(m_s - M) O_s / sum_s e^(m_s - M) l_s
KERNEL void __launch_bounds__(256) latent_attn_merge_kernel(const float* part_o, const float* part_ml, const int* vec_rows, int rows_h,
                                                             int H, int R, int nsplit, u16* out)
{
    const int v = bid_x();                                   // index into the list of (row * H + head)
    const long long vec = (long long)vec_rows[v / H] * H + v % H;
    // (all loads first, unconditionally: a load under a branch is a round trip of its own)
    float ms[LA_MAX_SPLIT], wt[LA_MAX_SPLIT];
    float M = -INFINITY;
    #pragma unroll
    for (int s = 0; s < LA_MAX_SPLIT; s++) { ms[s] = part_ml[(vec * nsplit + min(s, nsplit - 1)) * 2]; wt[s] = part_ml[(vec * nsplit + min(s, nsplit - 1)) * 2 + 1]; }
    #pragma unroll
    for (int s = 0; s < LA_MAX_SPLIT; s++) if (s < nsplit) M = fmaxf(M, ms[s]);
    float L = 0.0f;
    #pragma unroll
    for (int s = 0; s < LA_MAX_SPLIT; s++)
    {
        const float e = s < nsplit && ms[s] != -INFINITY ? expf(ms[s] - M) : 0.0f;
        L = fmaf(e, wt[s], L);
        wt[s] = e;
    }
    for (int i = tid(); i < R; i += 256)
    {
        float pv[LA_MAX_SPLIT];
        #pragma unroll
        for (int s = 0; s < LA_MAX_SPLIT; s++) pv[s] = part_o[(vec * nsplit + min(s, nsplit - 1)) * R + i];
        float o = 0.0f;
        #pragma unroll
        for (int s = 0; s < LA_MAX_SPLIT; s++) o = fmaf(wt[s], s < nsplit ? pv[s] : 0.0f, o);
        out[vec * R + i] = f32_to_bf16(o / L);
    }
}

template <int NT, int TR, int RS>
static void launch_lat_mfma_one(const LatMfmaArgs& a, int tiles, size_t smem, hipStream_t s)
{
    static bool attr_done[EXL2_MAX_DEVICES];
    if (exl2_first_on_device(attr_done))
        (void)hipFuncSetAttribute((const void*)latent_attn_mfma_kernel<NT, TR, RS>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    LAUNCH((latent_attn_mfma_kernel<NT, TR, RS>), dim3(tiles, TR == 16 ? (a.H + 3) / 4 : (a.H + 63) / 64, a.nsplit), dim3(256), smem, s, a);
}

template <int NT>
static void launch_lat_mfma(const LatMfmaArgs& a, int tiles, int tile_rows, size_t smem, hipStream_t s)
{
    const int rs = a.R == NT * 16 && (a.rot == 32 || a.rot == 64) ? a.rot / 32 : 0;
    if (tile_rows == 16)
    {
        if (rs == 1) launch_lat_mfma_one<NT, 16, 1>(a, tiles, smem, s);
        else if (rs == 2) launch_lat_mfma_one<NT, 16, 2>(a, tiles, smem, s);
        else launch_lat_mfma_one<NT, 16, 0>(a, tiles, smem, s);
    }
    else
    {
        if (rs == 1) launch_lat_mfma_one<NT, 1, 1>(a, tiles, smem, s);
        else if (rs == 2) launch_lat_mfma_one<NT, 1, 2>(a, tiles, smem, s);
        else launch_lat_mfma_one<NT, 1, 0>(a, tiles, smem, s);
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

/* the matrix-core form for bfloat16 (kv_rank a multiple of 32 and <= 512, rot a multiple of 8 and <= 128): the rows of the step are
   given as tiles -- tile i covers rows tile_row0[i] .. + tile_rows[i] (<= 16 consecutive positions of ONE sequence) when
   tile_mode is 16, or the single row tile_row0[i] when tile_mode is 1 (decoded tokens; all heads of the row share one pass over
   the keys).  nsplit > 1 (tile_mode 1 only): the keys are split over workgroups, part_o fp32 [rows, heads, nsplit, kv_rank] and
   part_ml fp32 [rows, heads, nsplit, 2] are scratch.  Returns EXL2_E_UNSUPPORTED for other shapes (use exl2_latent_attn). */
extern "C" int exl2_latent_attn_tiles(const void* q, int ldq, int q_head_stride, int q_rot_off, const float* q_abs, const void* cache,
                                      int page, const int* row_seq, const int* row_pos, const int* block_table, int bt_stride, void* out,
                                      const int* tile_row0, const int* tile_rows, int tiles, int tile_mode, float* part_o, float* part_ml,
                                      int nsplit, int heads, int kv_rank, int rot, int rot_dims, const float* inv_freq, float scale,
                                      int window, void* stream)
{
    EXL2_REQUIRE(q && q_abs && cache && row_seq && row_pos && block_table && out && inv_freq && tile_row0, "latent_attn_tiles: null operand");
    EXL2_REQUIRE(tile_mode == 16 || tile_mode == 1, "latent_attn_tiles: tile_mode is 16 or 1");
    EXL2_REQUIRE(tile_mode == 1 || tile_rows, "latent_attn_tiles: tile_rows missing");
    EXL2_REQUIRE(nsplit <= LA_MAX_SPLIT, "latent_attn_tiles: at most %d key splits", LA_MAX_SPLIT);
    EXL2_REQUIRE(nsplit >= 1 && (nsplit == 1 || (tile_mode == 1 && part_o && part_ml)), "latent_attn_tiles: key splits need tile_mode 1 and scratch");
    EXL2_REQUIRE(heads > 0 && page > 0 && window > 0 && rot_dims >= 0 && rot_dims <= rot && rot_dims % 2 == 0, "latent_attn_tiles: bad shape");
    if (kv_rank % 32 != 0 || kv_rank > 512 || kv_rank <= 0 || rot % 8 != 0 || rot > 32 * LA_ROT_STEPS)
        EXL2_FAIL(EXL2_E_UNSUPPORTED, "latent_attn_tiles: kv_rank %d / rot %d outside the matrix-core form", kv_rank, rot);
    if (tiles <= 0) return EXL2_OK;
    LatMfmaArgs a;
    a.q = (const u16*)q; a.ldq = ldq; a.q_head_stride = q_head_stride; a.q_rot_off = q_rot_off; a.q_abs = q_abs;
    a.cache = (const u16*)cache; a.page = page; a.row_seq = row_seq; a.row_pos = row_pos; a.block_table = block_table; a.bt_stride = bt_stride;
    a.tile_row0 = tile_row0; a.tile_rows = tile_rows; a.out = (u16*)out; a.part_o = part_o; a.part_ml = part_ml; a.nsplit = nsplit;
    a.H = heads; a.R = kv_rank; a.rot = rot; a.rot_dims = rot_dims; a.inv_freq = inv_freq; a.scale = scale; a.window = window;
    a.DP = (kv_rank + rot + 31) / 32 * 32;
    const size_t smem = ((size_t)LA_KT * (a.DP + 8) + (size_t)kv_rank * LA_TS) * 2;      // (<= 78 KB: two workgroups per CU)
    hipStream_t s = (hipStream_t)stream;
    if (kv_rank <= 128) launch_lat_mfma<8>(a, tiles, tile_mode, smem, s);
    else if (kv_rank <= 256) launch_lat_mfma<16>(a, tiles, tile_mode, smem, s);
    else launch_lat_mfma<32>(a, tiles, tile_mode, smem, s);
    if (nsplit > 1)
        LAUNCH(latent_attn_merge_kernel, dim3(tiles * heads), dim3(256), 0, s, (const float*)part_o, (const float*)part_ml, tile_row0, tiles,
               heads, kv_rank, nsplit, (u16*)out);
    HIP_TRY(hipGetLastError());
    return EXL2_OK;
}
