// Kernels of decoders with latent attention, a matrix-memory recurrence and a depth-weighted residual stream:
// an embedding with a hashed bigram table (the token before is a sequence's state), the weighted average of all
// earlier layers' results, the logits' soft cap, the preparation of latent attention (the norm of the latent, the
// rotation of the shared key part and of every head's rotated query part, the write into the paged cache), a small
// product per head (a query taken into the latent space, the latent's mix taken out into a head's values, with an
// optional output gate), the matrix memory's recurrence with its normaliser and running maximum, the norm per
// head with weight and gate behind it, and the activation of experts' hidden rows with the routing weight on the
// expert's input or output.  Every size is a run-time value.  Norms, angles, gates, decays and states are float32
// whatever the type of the matrices.
#include "common.h"

__device__ __forceinline__ float lt_sigmoid(float z) { return 1.f / (1.f + expf(-z)); }
// log(sigmoid(x)) = min(x, 0) - log(1 + exp(-|x|))
__device__ __forceinline__ float lt_logsigmoid(float x) { return fminf(x, 0.f) - log1pf(expf(-fabsf(x))); }

#define DISPATCH_T(dt, CALL)                                     \
    do {                                                         \
        if ((dt) == DT_F32) { typedef float T; CALL; }           \
        else if ((dt) == DT_F16) { typedef f16 T; CALL; }        \
        else if ((dt) == DT_BF16) { typedef bf16 T; CALL; }      \
        else return LI_BAD_ARG;                                  \
    } while (0)

// ---------------------------------------------------------------------------
// x[t] = table[token[t]] * scale + bigram[row],  row = (prev * mul_prev + token * mul_cur) mod buckets with prev the
// token before in the same sequence; a sequence's first token (position 0) takes row `buckets`, the table's last.
// The token before the first one that a sequence brings to a step is the sequence's state `prev_state` [slots];
// last_token_kernel leaves every sequence's last token of the step there.
// ---------------------------------------------------------------------------
template <class T>
__global__ void embed_bigram_kernel(const T* __restrict__ table, const T* __restrict__ bigram,
                                    const int* __restrict__ tokens, const int* __restrict__ pos,
                                    const int* __restrict__ tok_slot, const int* __restrict__ prev_state,
                                    float* __restrict__ out, int d, float scale, int64_t mul_prev, int64_t mul_cur,
                                    int buckets) {
    const int t = blockIdx.x, tok = tokens[t], slot = tok_slot[t];
    int64_t row = buckets;
    if (pos[t] > 0) {
        const int64_t prev = (t > 0 && tok_slot[t - 1] == slot) ? tokens[t - 1] : prev_state[slot];
        row = (prev * mul_prev + (int64_t)tok * mul_cur) % buckets;
        if (row < 0) row += buckets;
    }
    const T* e = table + (int64_t)tok * d;
    const T* b = bigram + row * d;
    for (int i = threadIdx.x; i < d; i += blockDim.x) out[(int64_t)t * d + i] = to_f32(e[i]) * scale + to_f32(b[i]);
}

__global__ void last_token_kernel(const int* __restrict__ tokens, const int* __restrict__ seq_slot,
                                  const int* __restrict__ seq_qstart, const int* __restrict__ seq_qlen,
                                  int* __restrict__ prev_state, int n_seqs) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n_seqs) return;
    const int q0 = seq_qstart ? seq_qstart[i] : i, n = seq_qlen ? seq_qlen[i] : 1;
    if (n > 0) prev_state[seq_slot[i]] = tokens[q0 + n - 1];
}

extern "C" int li_embed_bigram(const void* table, const void* bigram, int dt, const int* tokens, const int* pos,
                               const int* tok_slot, const int* seq_slot, const int* seq_qstart, const int* seq_qlen,
                               int* prev_state, float* out, int n, int n_seqs, int d, float scale, int64_t mul_prev,
                               int64_t mul_cur, int buckets, hipStream_t stream) {
    if (n <= 0) return LI_OK;
    if (d <= 0 || buckets <= 0 || n_seqs <= 0) return LI_BAD_ARG;
    DISPATCH_T(dt, (embed_bigram_kernel<T><<<n, 256, 0, stream>>>((const T*)table, (const T*)bigram, tokens, pos, tok_slot,
                                                                  prev_state, out, d, scale, mul_prev, mul_cur, buckets)));
    last_token_kernel<<<(n_seqs + 255) / 256, 256, 0, stream>>>(tokens, seq_slot, seq_qstart, seq_qlen, prev_state, n_seqs);
    LI_CHECK_LAUNCH();
    return LI_OK;
}

// ---------------------------------------------------------------------------
// out = sum over j < n of w[j] * hist[j]: the weighted average of the residual stream's earlier values, which lie
// `stride` floats apart; `count` floats each.
// ---------------------------------------------------------------------------
template <int V>
__global__ void depth_average_kernel(const float* __restrict__ hist, int64_t stride, const float* __restrict__ w, int n,
                                     float* __restrict__ out, int64_t count) {
    const int64_t i = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * V;
    if (i >= count) return;
    float acc[V];
#pragma unroll
    for (int v = 0; v < V; ++v) acc[v] = 0.f;
    for (int j = 0; j < n; ++j) {
        const float wj = w[j];
        const float* src = hist + j * stride + i;
        if (V == 4) {
            const f32x4 x = *(const f32x4*)src;
#pragma unroll
            for (int v = 0; v < V; ++v) acc[v] += wj * x[v];
        } else {
            acc[0] += wj * src[0];
        }
    }
#pragma unroll
    for (int v = 0; v < V; ++v) out[i + v] = acc[v];
}

extern "C" int li_depth_average(const float* hist, int64_t stride, const float* w, int n, float* out, int64_t count,
                                hipStream_t stream) {
    if (count <= 0) return LI_OK;
    if (n <= 0) return LI_BAD_ARG;
    const bool wide = count % 4 == 0 && stride % 4 == 0 && ((uintptr_t)hist | (uintptr_t)out) % 16 == 0;
    if (wide) depth_average_kernel<4><<<(unsigned)((count / 4 + 255) / 256), 256, 0, stream>>>(hist, stride, w, n, out, count);
    else depth_average_kernel<1><<<(unsigned)((count + 255) / 256), 256, 0, stream>>>(hist, stride, w, n, out, count);
    LI_CHECK_LAUNCH();
    return LI_OK;
}

// ---------------------------------------------------------------------------
// x <- cap * tanh(x / cap), in place on float32.
// ---------------------------------------------------------------------------
__global__ void softcap_kernel(float* __restrict__ x, int64_t n, float cap) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) x[i] = cap * tanhf(x[i] / cap);
}

extern "C" int li_softcap(float* x, int64_t n, float cap, hipStream_t stream) {
    if (n <= 0) return LI_OK;
    if (!(cap > 0.f)) return LI_BAD_ARG;
    softcap_kernel<<<(unsigned)((n + 255) / 256), 256, 0, stream>>>(x, n, cap);
    LI_CHECK_LAUNCH();
    return LI_OK;
}

// ---------------------------------------------------------------------------
// Latent attention keeps, for every token, a latent c of size r shared by all heads and one rotated key part of
// size rd; a head's key is an up-projection of c, its value another.  With the up-projection of the keys taken
// into the query (q' = W_uk^T q_unrotated per head) a score is q' . c + q_rot . k_rot, and with the values' taken
// out of the sum a head's output is W_uv (sum of weights * c): one key [c | k_rot] and one value c for all heads.
// The pages hold them in the matrix instruction's operand order (common.h), keys KW = r + rd rounded up to 16 wide
// with zeros behind, values r wide.
// latent_store_kernel, per token, from the float32 rows of the input product (q heads [d | rd] from column q_col,
// then [latent r | rotated part rd] from column kv_col): c = the latent divided by its root mean square over r,
// times a weight; the rotated parts turned by the token's position (pairs (2i, 2i + 1) of the first `rot` of the
// rd dimensions, angle p * freq[i]; the rest pass); key and value into the page of the token's position; every
// head's rotated query part (and the zeros behind it) into q_out [T, H, KW] from column r on.  The first r columns
// of q_out are the product per head's (head_linear_kernel).
// ---------------------------------------------------------------------------
struct MapPages {
    void* k;
    void* v;
    int64_t page_stride;
    const int* page_table;
    int max_pages;
};

__device__ __forceinline__ float rotated(const float* __restrict__ x, int j, int rot, float p,
                                         const float* __restrict__ freq) {
    if (j >= rot) return x[j];
    const int pair = j >> 1;
    const float a = p * freq[pair], c = cosf(a), s = sinf(a);
    const float u = x[2 * pair], v = x[2 * pair + 1];
    return (j & 1) ? v * c + u * s : u * c - v * s;
}

template <class T>
__global__ void latent_store_kernel(const float* __restrict__ proj, int stride, int q_col, int kv_col,
                                    const float* __restrict__ norm_w, float eps, const float* __restrict__ freq, int rot,
                                    const int* __restrict__ pos, const int* __restrict__ tok_slot, T* __restrict__ q_out,
                                    MapPages pg, int H, int d, int rd, int r, int KW) {
    __shared__ float scratch[16];
    const int t = blockIdx.x, p = pos[t];
    const float* row = proj + (int64_t)t * stride;
    const float* lat = row + kv_col;
    float ss = 0.f;
    for (int i = threadIdx.x; i < r; i += blockDim.x) ss += lat[i] * lat[i];
    const float rr = 1.f / sqrtf(block_sum(ss, scratch) / (float)r + eps);
    const int page = pg.page_table[(int64_t)tok_slot[t] * pg.max_pages + p / PAGE], off = p % PAGE;
    T* kp = (T*)pg.k + (int64_t)page * pg.page_stride;
    T* vp = (T*)pg.v + (int64_t)page * pg.page_stride;
    const float fp = (float)p;
    // (few tokens: the grid's second dimension shares a token's key and heads among several workgroups)
    for (int i = blockIdx.y * blockDim.x + threadIdx.x; i < KW; i += gridDim.y * blockDim.x) {
        float v = 0.f;
        if (i < r) {
            v = lat[i] * rr * norm_w[i];
            vp[v_offset(off, i, r)] = from_f32<T>(v);
        } else if (i < r + rd) {
            v = rotated(lat + r, i - r, rot, fp, freq);
        }
        kp[k_offset(off, i, KW)] = from_f32<T>(v);
    }
    const int tail = KW - r;
    for (int idx = blockIdx.y * blockDim.x + threadIdx.x; idx < H * tail; idx += gridDim.y * blockDim.x) {
        const int h = idx / tail, j = idx - h * tail;
        const float v = j < rd ? rotated(row + q_col + (int64_t)h * (d + rd) + d, j, rot, fp, freq) : 0.f;
        q_out[((int64_t)t * H + h) * KW + r + j] = from_f32<T>(v);
    }
}

extern "C" int li_latent_store(const float* proj, int stride, int q_col, int kv_col, const float* norm_w, float eps,
                               const float* freq, int rot, const int* pos, const int* tok_slot, void* q_out, void* k_pages,
                               void* v_pages, int64_t page_stride, const int* page_table, int max_pages, int dt, int n,
                               int H, int d, int rd, int r, hipStream_t stream) {
    if (n <= 0) return LI_OK;
    if (H <= 0 || d < 0 || rd < 0 || r <= 0 || rot < 0 || rot > rd || rot % 2) return LI_BAD_ARG;
    MapPages pg{k_pages, v_pages, page_stride, page_table, max_pages};
    const int KW = round_up(r + rd, 16);
    dim3 grid(n, n >= 256 ? 1 : min(16, (max(KW, H * (KW - r)) + 255) / 256));
    DISPATCH_T(dt, (latent_store_kernel<T><<<grid, 256, 0, stream>>>(proj, stride, q_col, kv_col, norm_w, eps, freq, rot, pos,
                                                                  tok_slot, (T*)q_out, pg, H, d, rd, r, KW)));
    LI_CHECK_LAUNCH();
    return LI_OK;
}

// ---------------------------------------------------------------------------
// A small product per head: out[t][h][j] = sum over i of W[h][j][i] * in[t][h][i]   (W stored [H, n_out, n_in]), i < n_in,
// j < n_out.  Rows of `in` and `out` are addressed by a
// stride per token and one per head, so that a head's part may lie inside a wider row.  `gate` not null: the result
// is multiplied by sigmoid(gate[t][h * n_out + j]) (float32 rows, `gate_stride` apart).  Sums are float32.
// head_linear_kernel (float32 models): a workgroup takes 16 tokens of one head,
// their inputs wait in LDS and every thread owns outputs j.  head_linear_mfma_kernel (16-bit models): a wave owns 32
// outputs x up to 128 tokens of one head (a fragment of W serves four tiles of 32 tokens), W^T as operand A and the tokens' inputs (rounded to the 16-bit type where they
// come in float32, as the sum of two such numbers) as operand B of the 32x32x16 matrix instruction, both read straight from memory, 16 bytes a lane
// where n_in and the rows allow; the four waves of a workgroup take four blocks of outputs for the same tokens.
// ---------------------------------------------------------------------------
#define HL_TOK 16

template <class TI, class TW, class TO>
__global__ __launch_bounds__(256) void head_linear_kernel(const TI* __restrict__ in, int64_t in_st, int in_sh,
                                                          const TW* __restrict__ W, TO* __restrict__ out, int64_t out_st,
                                                          int out_sh, const float* __restrict__ gate, int64_t gate_st,
                                                          int n_tokens, int n_in, int n_out) {
    extern __shared__ float xs[];                       // [HL_TOK][n_in]
    const int t0 = blockIdx.x * HL_TOK, h = blockIdx.y;
    const int nt = min(HL_TOK, n_tokens - t0);
    for (int e = threadIdx.x; e < HL_TOK * n_in; e += blockDim.x) {
        const int k = e / n_in, i = e - k * n_in;
        xs[e] = k < nt ? to_f32(in[(int64_t)(t0 + k) * in_st + (int64_t)h * in_sh + i]) : 0.f;
    }
    __syncthreads();
    const TW* Wh = W + (int64_t)h * n_in * n_out;
    for (int j = threadIdx.x; j < n_out; j += blockDim.x) {
        float acc[HL_TOK];
#pragma unroll
        for (int k = 0; k < HL_TOK; ++k) acc[k] = 0.f;
        for (int i = 0; i < n_in; ++i) {
            const float w = to_f32(Wh[(int64_t)j * n_in + i]);
#pragma unroll
            for (int k = 0; k < HL_TOK; ++k) acc[k] += w * xs[k * n_in + i];
        }
#pragma unroll
        for (int k = 0; k < HL_TOK; ++k) {
            if (k < nt) {
                float v = acc[k];
                if (gate) v *= lt_sigmoid(gate[(int64_t)(t0 + k) * gate_st + (int64_t)h * n_out + j]);
                out[(int64_t)(t0 + k) * out_st + (int64_t)h * out_sh + j] = from_f32<TO>(v);
            }
        }
    }
}

#define HLM_TT 4            // tiles of 32 tokens that a wave multiplies with one fragment of W

template <class TI, class T>
__global__ __launch_bounds__(256) void head_linear_mfma_kernel(const TI* __restrict__ in, int64_t in_st, int in_sh,
                                                               const T* __restrict__ W, T* __restrict__ out, int64_t out_st,
                                                               int out_sh, const float* __restrict__ gate, int64_t gate_st,
                                                               int n_tokens, int n_in, int n_out, int vec) {
    typedef typename Vec<T>::v8 v8;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, col = lane & 31, half = lane >> 5;
    const int tb = blockIdx.x * 32 * HLM_TT, h = blockIdx.y, j0 = (blockIdx.z * 4 + wave) * 32;
    if (j0 >= n_out) return;
    const bool j_ok = j0 + col < n_out;
    const T* wrow = W + ((int64_t)h * n_out + (j_ok ? j0 + col : 0)) * n_in;
    const int tiles = min(HLM_TT, (n_tokens - tb + 31) / 32);            // the same for all lanes
    const TI* xrow[HLM_TT];
#pragma unroll
    for (int u = 0; u < HLM_TT; ++u) xrow[u] = in + (int64_t)min(tb + 32 * u + col, n_tokens - 1) * in_st + (int64_t)h * in_sh;
    f32x16 acc[HLM_TT];
#pragma unroll
    for (int u = 0; u < HLM_TT; ++u)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[u][r] = 0.f;
    for (int k0 = 0; k0 < n_in; k0 += 16) {
        const int i0 = k0 + 8 * half;
        const bool whole = vec && i0 + 8 <= n_in;
        v8 a;
        if (whole) a = *(const v8*)(wrow + i0);
        else {
#pragma unroll
            for (int e = 0; e < 8; ++e) a[e] = i0 + e < n_in ? wrow[i0 + e] : from_f32<T>(0.f);
        }
        if (!j_ok) {
#pragma unroll
            for (int e = 0; e < 8; ++e) a[e] = from_f32<T>(0.f);
        }
#pragma unroll
        for (int u = 0; u < HLM_TT; ++u) {
            if (u >= tiles) break;
            v8 b, b2;                    // b2: what the rounding of a float32 input leaves, so that the product sees 16 bits of it
            float xf[8];
            if (whole) {
                if (sizeof(TI) == 4) {
                    const f32x4 lo = *(const f32x4*)((const float*)xrow[u] + i0), hi = *(const f32x4*)((const float*)xrow[u] + i0 + 4);
#pragma unroll
                    for (int e = 0; e < 4; ++e) { xf[e] = lo[e]; xf[4 + e] = hi[e]; }
                } else {
                    b = *(const v8*)((const T*)xrow[u] + i0);
                }
            } else {
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    xf[e] = i0 + e < n_in ? to_f32(xrow[u][i0 + e]) : 0.f;
                    if (sizeof(TI) != 4) b[e] = from_f32<T>(xf[e]);
                }
            }
            if (sizeof(TI) == 4) {
#pragma unroll
                for (int e = 0; e < 8; ++e) { b[e] = from_f32<T>(xf[e]); b2[e] = from_f32<T>(xf[e] - to_f32(b[e])); }
            }
            acc[u] = mfma32(a, b, acc[u]);
            if (sizeof(TI) == 4) acc[u] = mfma32(a, b2, acc[u]);
        }
    }
#pragma unroll
    for (int u = 0; u < HLM_TT; ++u) {
        const int t = tb + 32 * u + col;
        if (u >= tiles || t >= n_tokens) continue;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int j = j0 + 8 * (r >> 2) + 4 * half + (r & 3);
            if (j < n_out) {
                float v = acc[u][r];
                if (gate) v *= lt_sigmoid(gate[(int64_t)t * gate_st + (int64_t)h * n_out + j]);
                out[(int64_t)t * out_st + (int64_t)h * out_sh + j] = from_f32<T>(v);
            }
        }
    }
}

extern "C" int li_head_linear(const void* in, int in_dt, int64_t in_st, int in_sh, const void* W, int w_dt, void* out,
                              int64_t out_st, int out_sh, const float* gate, int64_t gate_st, int n_tokens, int H, int n_in,
                              int n_out, hipStream_t stream) {
    if (n_tokens <= 0) return LI_OK;
    if (H <= 0 || n_in <= 0 || n_out <= 0) return LI_BAD_ARG;
    if (w_dt == DT_F16 || w_dt == DT_BF16) {
        // 16 bytes a lane where every fragment begins at a multiple of 16 bytes
        const int isz = in_dt == DT_F32 ? 4 : 2;
        const int vec = n_in % 8 == 0 && (uintptr_t)W % 16 == 0 && (uintptr_t)in % 16 == 0 && (in_st * isz) % 16 == 0 &&
                        ((int64_t)in_sh * isz) % 16 == 0;
        dim3 grid((n_tokens + 32 * HLM_TT - 1) / (32 * HLM_TT), H, (n_out + 127) / 128);
#define GOM(TI, T) head_linear_mfma_kernel<TI, T><<<grid, 256, 0, stream>>>((const TI*)in, in_st, in_sh, (const T*)W, (T*)out, out_st, \
                                                                           out_sh, gate, gate_st, n_tokens, n_in, n_out, vec)
        if (in_dt == DT_F32) { if (w_dt == DT_F16) GOM(float, f16); else GOM(float, bf16); }
        else if (in_dt == w_dt) { if (w_dt == DT_F16) GOM(f16, f16); else GOM(bf16, bf16); }
        else return LI_BAD_ARG;
#undef GOM
        LI_CHECK_LAUNCH();
        return LI_OK;
    }
    const size_t lds = (size_t)HL_TOK * n_in * sizeof(float);
    if (lds > 64000) return LI_UNSUPPORTED;
    dim3 grid((n_tokens + HL_TOK - 1) / HL_TOK, H);
    // the weights and the output have the model's type; the input is float32 (rows of a product) or of that type
#define GO(TI, T) head_linear_kernel<TI, T, T><<<grid, 256, lds, stream>>>((const TI*)in, in_st, in_sh, (const T*)W, (T*)out, \
                                                                           out_st, out_sh, gate, gate_st, n_tokens, n_in, n_out)
    if (in_dt == DT_F32) DISPATCH_T(w_dt, GO(float, T));
    else if (in_dt == w_dt) DISPATCH_T(w_dt, GO(T, T));
    else return LI_BAD_ARG;
#undef GO
    LI_CHECK_LAUNCH();
    return LI_OK;
}

// ---------------------------------------------------------------------------
// The matrix memory (mLSTM) recurrence.  Per sequence and head, with q_t, k_t [d] and v_t [dv] from the float32 rows
// `proj` (q is multiplied by qscale), the raw gates gi, gf from two more columns, cap > 0:
//   i = cap tanh((gi + bi[h]) / cap),   f = logsigmoid(cap tanh((gf + bf[h]) / cap))
//   m_t = max(f + m_{t-1}, i);   a_t = exp(f + m_{t-1} - m_t),  b_t = exp(i - m_t)
//   S_t = a_t S_{t-1} + b_t k_t v_t^T;   n_t = a_t n_{t-1} + b_t k_t;   y_t = S_t^T q_t / (max(|n_t . q_t|, exp(-m_t)) + 1e-6)
// S [d, dv], n [d] and m are float32 state of every sequence (`S_state` [slots, H, d, dv]; `nm_state` [slots, H, d + 1]
// with m behind n), zero when it starts (so m_0 = 0).
// Two kernels come first.  mlstm_gates_kernel, a thread per (token, head): i and f into `coef` [T, H, 3].
// mlstm_max_kernel, a wave per (sequence, head), walks the sequence's tokens with the one dependent chain there is,
// m_t, and leaves (a_t, b_t, exp(-m_t)) in `coef` and the last m in the state.  With a_t and b_t known the
// recurrence of S and n is linear, with one decay for all of a head's elements.
// mlstm_scan_kernel, one wave per (sequence or segment, head, 64 columns of dv): a lane keeps its column of S in
// registers for all the tokens of its stretch; q_t, k_t and n lie across the lanes and reach every lane by lane reads.
// PASS 0 walks a sequence's tokens in order from the state and leaves the state up to date (the waves of a head all
// begin from the n that the step found, so the new one goes to `nm_new` [sequences, H, d + 1] first and
// mlstm_commit_kernel puts it into the state once every wave has ended).  A prompt may also be walked in segments
// side by side (ScanSegments): PASS 1 runs every segment from zero and leaves what it adds to S and n and the product
// of its a_t; seg_combine_kernel walks a sequence's segments in order, X <- A_seg X + D_seg, leaving the value
// before every segment where its contribution was; PASS 3 runs every segment again from there and writes y.
// y float32 [T, H * dv].
// ---------------------------------------------------------------------------
__global__ void mlstm_gates_kernel(const float* __restrict__ proj, int stride, int i_col, int f_col,
                                   const float* __restrict__ i_bias, const float* __restrict__ f_bias, float cap,
                                   float* __restrict__ coef, int n_tokens, int H) {
    const int e = blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= n_tokens * H) return;
    const int t = e / H, h = e - t * H;
    const float gi = proj[(int64_t)t * stride + i_col + h] + (i_bias ? i_bias[h] : 0.f);
    const float gf = proj[(int64_t)t * stride + f_col + h] + (f_bias ? f_bias[h] : 0.f);
    coef[(int64_t)e * 3] = cap * tanhf(gi / cap);
    coef[(int64_t)e * 3 + 1] = lt_logsigmoid(cap * tanhf(gf / cap));
}

__global__ __launch_bounds__(64) void mlstm_max_kernel(float* __restrict__ coef, float* __restrict__ nm_state,
                                                       const int* __restrict__ seq_slot, const int* __restrict__ seq_qstart,
                                                       const int* __restrict__ seq_qlen, int H, int d) {
    // one wave per (sequence, head), 64 tokens at a time: every lane fetches its token's i and f, the chain runs over
    // lane reads (no memory in it), each lane keeps the maximum before and after its own token and finishes it alone
    const int seq = blockIdx.x / H, h = blockIdx.x - seq * H, lane = threadIdx.x;
    const int q0 = seq_qstart ? seq_qstart[seq] : seq, n = seq_qlen ? seq_qlen[seq] : 1;
    if (n <= 0) return;
    float* mp = nm_state + ((int64_t)seq_slot[seq] * H + h) * (d + 1) + d;
    float m = *mp;
    for (int base = 0; base < n; base += 64) {
        const int t = base + lane, cnt = min(64, n - base);
        float* c = coef + ((int64_t)(q0 + min(t, n - 1)) * H + h) * 3;
        const float ig = c[0], fg = c[1];
        float before = 0.f, after = 0.f;
        for (int j = 0; j < cnt; ++j) {
            const float fj = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(fg), j));
            const float ij = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(ig), j));
            const float mn = fmaxf(fj + m, ij);
            if (lane == j) { before = m; after = mn; }
            m = mn;
        }
        if (t < n) {
            c[0] = expf(fg + before - after);
            c[1] = expf(ig - after);
            c[2] = expf(-after);
        }
    }
    if (lane == 0) *mp = m;
}

struct ScanSegments {
    const int* seg_seq;         // [segments] the sequence of a segment
    const int* seg_t0;          // [segments] its first token among the sequence's tokens of this step
    const int* seg_n;           // [segments] its tokens
    float* seg_S;               // [segments, H, d, dv]
    float* seg_nrm;             // [segments, H, d]
    float* seg_decay;           // [segments, H]
};

// A head whose keys are more than 128 wide is shared by two waves a column block, 128 rows of S each (a lane's 256
// registers of state would leave one wave a SIMD): RSPLIT = 2, and the two add their halves of y into rows that the
// caller has cleared (two addends: the sum does not depend on their order).
template <int NMAX, int NV, int RSPLIT, int PASS>
__global__ __launch_bounds__(64) void mlstm_scan_kernel(
    const float* __restrict__ proj, int stride, int q_col, int k_col, int v_col, const float* __restrict__ coef,
    float qscale, float* __restrict__ S_state, const float* __restrict__ nm_state, float* __restrict__ nm_new,
    const int* __restrict__ seq_slot, const int* __restrict__ seq_qstart, const int* __restrict__ seq_qlen,
    float* __restrict__ y, int H, int d, int dv, ScanSegments sg) {
    const int h = blockIdx.y, lane = threadIdx.x, col = (blockIdx.z / RSPLIT) * 64 + lane;
    const int r0 = (blockIdx.z % RSPLIT) * NMAX;             // this wave's first row of S
    const bool live = col < dv;
    int q0, n;
    float* S;
    const float* nsrc;
    if (PASS == 0) {
        const int seq = blockIdx.x;
        q0 = seq_qstart ? seq_qstart[seq] : seq;
        n = seq_qlen ? seq_qlen[seq] : 1;
        S = S_state + (((int64_t)seq_slot[seq] * H + h) * d) * dv + col;
        nsrc = nm_state + ((int64_t)seq_slot[seq] * H + h) * (d + 1);
    } else {
        const int seg = blockIdx.x;
        q0 = seq_qstart[sg.seg_seq[seg]] + sg.seg_t0[seg];
        n = sg.seg_n[seg];
        S = sg.seg_S + (((int64_t)seg * H + h) * d) * dv + col;
        nsrc = sg.seg_nrm + ((int64_t)seg * H + h) * d;
    }
    if (n <= 0) return;
    float s[NMAX], nl[NV];
#pragma unroll
    for (int i = 0; i < NMAX; ++i) s[i] = (PASS != 1 && live && r0 + i < d) ? S[(int64_t)(r0 + i) * dv] : 0.f;
#pragma unroll
    for (int v = 0; v < NV; ++v) nl[v] = (PASS != 1 && v * 64 + lane < d) ? nsrc[v * 64 + lane] : 0.f;
    float qv[NV], kv[NV], x = 0.f, ca = 0.f, cb = 0.f, cm = 0.f, decay = 1.f;
    auto fetch = [&](int t) {
        const float* __restrict__ row = proj + (int64_t)(q0 + t) * stride;
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            const int i = v * 64 + lane;
            if (PASS != 1) qv[v] = i < d ? row[q_col + h * d + i] * qscale : 0.f;
            kv[v] = i < d ? row[k_col + h * d + i] : 0.f;
        }
        x = live ? row[v_col + h * dv + col] : 0.f;
        const float* c = coef + ((int64_t)(q0 + t) * H + h) * 3;
        ca = c[0]; cb = c[1]; cm = c[2];
    };
    fetch(0);
    for (int t = 0; t < n; ++t) {
        float qt[NV], kt[NV];
#pragma unroll
        for (int v = 0; v < NV; ++v) { qt[v] = PASS != 1 ? qv[v] : 0.f; kt[v] = kv[v]; }
        const float a = ca, b = cb, em = cm, bx = cb * x;
        if (t + 1 < n) fetch(t + 1);
        decay *= a;
        float nq = 0.f;
#pragma unroll
        for (int v = 0; v < NV; ++v) { nl[v] = a * nl[v] + b * kt[v]; nq += nl[v] * qt[v]; }
        if (PASS != 1) nq = wave_sum(nq);
        // the registers that hold this wave's rows of k_t and q_t (the second half of them where the rows are shared)
        constexpr int NH = (NMAX + 63) / 64;
        float kh[NH], qh[NH];
#pragma unroll
        for (int v = 0; v < NH; ++v) {
            kh[v] = (RSPLIT > 1 && r0) ? kt[(NV - NH + v) % NV] : kt[v];
            qh[v] = (RSPLIT > 1 && r0) ? qt[(NV - NH + v) % NV] : qt[v];
        }
        float acc = 0.f;
#pragma unroll
        for (int i = 0; i < NMAX; ++i) {
            const float kk = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(kh[i >> 6]), i & 63));
            float qq = 0.f;
            if (PASS != 1) qq = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(qh[i >> 6]), i & 63));
            s[i] = a * s[i] + kk * bx;
            if (PASS != 1) acc += s[i] * qq;
        }
        if (PASS != 1 && live) {
            float* to = y + (int64_t)(q0 + t) * H * dv + h * dv + col;
            const float v = acc / (fmaxf(fabsf(nq), em) + 1e-6f);
            if (RSPLIT > 1) atomicAdd(to, v); else *to = v;
        }
    }
    if (PASS == 3) return;
    if (live) {
#pragma unroll
        for (int i = 0; i < NMAX; ++i) if (r0 + i < d) S[(int64_t)(r0 + i) * dv] = s[i];
    }
    if (blockIdx.z == 0) {
        float* to = PASS == 0 ? nm_new + ((int64_t)blockIdx.x * H + h) * (d + 1) : sg.seg_nrm + ((int64_t)blockIdx.x * H + h) * d;
#pragma unroll
        for (int v = 0; v < NV; ++v) if (v * 64 + lane < d) to[v * 64 + lane] = nl[v];
        if (PASS == 1 && lane == 0) sg.seg_decay[(int64_t)blockIdx.x * H + h] = decay;
    }
}

// n of every (sequence, head) from the scratch memory into the state (m, behind it, is mlstm_max_kernel's).
__global__ void mlstm_commit_kernel(const float* __restrict__ nm_new, float* __restrict__ nm_state,
                                    const int* __restrict__ seq_slot, const int* __restrict__ seq_qlen, int H, int d) {
    const int seq = blockIdx.x, h = blockIdx.y;
    if (seq_qlen && seq_qlen[seq] <= 0) return;
    const float* from = nm_new + ((int64_t)seq * H + h) * (d + 1);
    float* to = nm_state + ((int64_t)seq_slot[seq] * H + h) * (d + 1);
    for (int i = threadIdx.x; i < d; i += blockDim.x) to[i] = from[i];
}

// One thread per element of a head's state (`per_head` of them, `state_stride` floats from head to head in the
// state): walks the sequence's segments in order.
__global__ void seg_combine_kernel(float* __restrict__ state, int64_t state_stride, const int* __restrict__ seq_slot,
                                   const int* __restrict__ seq_seg0, const int* __restrict__ seq_nseg,
                                   float* __restrict__ seg_buf, const float* __restrict__ seg_decay, int H, int64_t per_head) {
    const int seq = blockIdx.x, h = blockIdx.y;
    const int c0 = seq_seg0[seq], nc = seq_nseg[seq];
    for (int64_t e = (int64_t)blockIdx.z * blockDim.x + threadIdx.x; e < per_head; e += (int64_t)gridDim.z * blockDim.x) {
        float* X = state + ((int64_t)seq_slot[seq] * H + h) * state_stride + e;
        float x = *X;
        for (int c = c0; c < c0 + nc; ++c) {
            float* L = seg_buf + ((int64_t)c * H + h) * per_head + e;
            const float own = *L;
            *L = x;
            x = seg_decay[(int64_t)c * H + h] * x + own;
        }
        *X = x;
    }
}

#define MLSTM_GO(NM, NV, RS, PASS, GRID) mlstm_scan_kernel<NM, NV, RS, PASS><<<GRID, 64, 0, stream>>>(proj, stride, q_col, k_col, v_col, \
        coef, qscale, S_state, nm_state, nm_new, seq_slot, seq_qstart, seq_qlen, y, H, d, dv, sg)
#define MLSTM_LAUNCH(PASS, GRID)                                                                                       \
    do {                                                                                                               \
        if (d <= 16) MLSTM_GO(16, 1, 1, PASS, GRID); else if (d <= 32) MLSTM_GO(32, 1, 1, PASS, GRID);                 \
        else if (d <= 64) MLSTM_GO(64, 1, 1, PASS, GRID); else if (d <= 128) MLSTM_GO(128, 2, 1, PASS, GRID);          \
        else MLSTM_GO(128, 4, 2, PASS, GRID);                                                                          \
    } while (0)

// y must be cleared where d > 128 (two waves add their halves into it).  coef: scratch float32 [T, H, 3]; nm_new: scratch float32 [sequences, H, d + 1].  n_segs > 0 (with the segment lists and
// scratch seg_S [segments, H, d, dv], seg_nrm [segments, H, d], seg_decay [segments, H]): the tokens run in segments.
extern "C" int li_mlstm_scan(const float* proj, int stride, int q_col, int k_col, int v_col, int i_col, int f_col,
                             const float* i_bias, const float* f_bias, float cap, float qscale, float* S_state,
                             float* nm_state, float* nm_new, float* coef, const int* seq_slot, const int* seq_qstart,
                             const int* seq_qlen, float* y, int n_tokens, int n_seqs, int H, int d, int dv,
                             const int* seg_seq, const int* seg_t0, const int* seg_n, const int* seq_seg0,
                             const int* seq_nseg, int n_segs, float* seg_S, float* seg_nrm, float* seg_decay,
                             hipStream_t stream) {
    if (n_seqs <= 0 || n_tokens <= 0) return LI_OK;
    if (H <= 0 || d <= 0 || dv <= 0 || !(cap > 0.f) || !coef) return LI_BAD_ARG;
    if (d > 256) return LI_UNSUPPORTED;
    mlstm_gates_kernel<<<(n_tokens * H + 255) / 256, 256, 0, stream>>>(proj, stride, i_col, f_col, i_bias, f_bias, cap, coef,
                                                                       n_tokens, H);
    mlstm_max_kernel<<<n_seqs * H, 64, 0, stream>>>(coef, nm_state, seq_slot, seq_qstart, seq_qlen, H, d);
    ScanSegments sg{seg_seq, seg_t0, seg_n, seg_S, seg_nrm, seg_decay};
    if (n_segs <= 0) {
        if (!nm_new) return LI_BAD_ARG;
        dim3 grid(n_seqs, H, (dv + 63) / 64 * (d > 128 ? 2 : 1));
        MLSTM_LAUNCH(0, grid);
        mlstm_commit_kernel<<<dim3(n_seqs, H), 64, 0, stream>>>(nm_new, nm_state, seq_slot, seq_qlen, H, d);
    } else {
        if (!seq_qstart || !seq_qlen || !seg_seq || !seg_t0 || !seg_n || !seq_seg0 || !seq_nseg || !seg_S || !seg_nrm || !seg_decay)
            return LI_BAD_ARG;
        dim3 grid(n_segs, H, (dv + 63) / 64 * (d > 128 ? 2 : 1));
        MLSTM_LAUNCH(1, grid);
        const int64_t per_head = (int64_t)d * dv;
        seg_combine_kernel<<<dim3(n_seqs, H, (unsigned)((per_head + 255) / 256)), 256, 0, stream>>>(
            S_state, per_head, seq_slot, seq_seg0, seq_nseg, seg_S, seg_decay, H, per_head);
        seg_combine_kernel<<<dim3(n_seqs, H, 1), 256, 0, stream>>>(nm_state, d + 1, seq_slot, seq_seg0, seq_nseg, seg_nrm,
                                                                    seg_decay, H, d);
        MLSTM_LAUNCH(3, grid);
    }
    LI_CHECK_LAUNCH();
    return LI_OK;
}

// ---------------------------------------------------------------------------
// out[t][h][j] = y[t][h][j] / sqrt(mean over j of y[t][h]^2 + eps) * w[h * dv + j] * sigmoid(gate[t][h * dv + j]):
// every head's part of a row divided by its own root mean square, then a weight over all heads and a gate
// (float32 rows `gate_stride` apart; null: none).  One wave per (token, head).
// ---------------------------------------------------------------------------
template <class T>
__global__ __launch_bounds__(256) void gated_head_norm_kernel(const float* __restrict__ y, const float* __restrict__ w,
                                                              const float* __restrict__ gate, int64_t gate_stride,
                                                              T* __restrict__ out, int n_units, int H, int dv, float eps) {
    const int unit = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    if (unit >= n_units) return;
    const int t = unit / H, h = unit - t * H;
    const float* yr = y + (int64_t)unit * dv;
    float ss = 0.f;
    for (int i = lane; i < dv; i += 64) ss += yr[i] * yr[i];
    const float r = 1.f / sqrtf(wave_sum(ss) / (float)dv + eps);
    for (int i = lane; i < dv; i += 64) {
        float v = yr[i] * r * (w ? w[h * dv + i] : 1.f);
        if (gate) v *= lt_sigmoid(gate[(int64_t)t * gate_stride + h * dv + i]);
        out[(int64_t)unit * dv + i] = from_f32<T>(v);
    }
}

extern "C" int li_gated_head_norm(const float* y, const float* w, const float* gate, int64_t gate_stride, void* out, int dt,
                                  int n_rows, int H, int dv, float eps, hipStream_t stream) {
    if (n_rows <= 0) return LI_OK;
    if (H <= 0 || dv <= 0) return LI_BAD_ARG;
    const int units = n_rows * H;
    DISPATCH_T(dt, (gated_head_norm_kernel<T><<<(units + 3) / 4, 256, 0, stream>>>(y, w, gate, gate_stride, (T*)out, units, H, dv, eps)));
    LI_CHECK_LAUNCH();
    return LI_OK;
}

// ---------------------------------------------------------------------------
// The hidden rows of experts side by side, z float32 [rows, n_blocks * ff + tail] (the sums of the up products),
// through the activation with the routing weight: block e of a row takes weight wgt[r][e] (the tail, an expert that
// every token uses, wgt[r][n_blocks]), r = idx[row] (idx null: the row itself); `col` >= 0: every block takes
// wgt[r][col] (the rows of one expert).  on_input: out = act(weight * z), the weight on the expert's input (its up
// product is linear); else out = weight * act(z).  A weight of zero gives zero.  act: 0 gelu (erf), 1 gelu (tanh),
// 2 silu, 3 the square of relu.
// ---------------------------------------------------------------------------
__device__ __forceinline__ float lt_act(float z, int act) {
    if (act == 3) { const float r = fmaxf(z, 0.f); return r * r; }
    if (act == 2) return z / (1.f + expf(-z));
    if (act == 1) return gate_activation(z, true);
    return 0.5f * z * (1.f + erff(z * 0.70710678118654752f));
}

template <class T>
__global__ void expert_act_kernel(const float* __restrict__ z, const float* __restrict__ wgt, int wcols,
                                  const int* __restrict__ idx, int col, T* __restrict__ out, int n_blocks, int ff, int tail,
                                  int act, int on_input) {
    const int64_t row = blockIdx.x;
    const int64_t r = idx ? idx[row] : row;
    const int cols = n_blocks * ff + tail;
    for (int i = blockIdx.y * blockDim.x + threadIdx.x; i < cols; i += gridDim.y * blockDim.x) {
        const int e = col >= 0 ? col : (i < n_blocks * ff ? i / ff : n_blocks);
        const float w = wgt ? wgt[r * wcols + e] : 1.f;
        const float v = z[row * cols + i];
        out[row * cols + i] = from_f32<T>(w == 0.f ? 0.f : (on_input ? lt_act(w * v, act) : w * lt_act(v, act)));
    }
}

extern "C" int li_expert_act(const float* z, const float* wgt, int wcols, const int* idx, int col, void* out, int dt, int n,
                             int n_blocks, int ff, int tail, int act, int on_input, hipStream_t stream) {
    if (n <= 0) return LI_OK;
    if (n_blocks < 0 || ff < 0 || tail < 0 || act < 0 || act > 3 || (wgt && col >= wcols)) return LI_BAD_ARG;
    const int cols = n_blocks * ff + tail;
    if (cols <= 0) return LI_OK;
    dim3 grid(n, n >= 1024 ? 1 : (cols + 1023) / 1024);
    DISPATCH_T(dt, (expert_act_kernel<T><<<grid, 256, 0, stream>>>(z, wgt, wcols, idx, col, (T*)out, n_blocks, ff, tail, act, on_input)));
    LI_CHECK_LAUNCH();
    return LI_OK;
}
