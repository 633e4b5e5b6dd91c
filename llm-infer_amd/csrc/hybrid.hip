// Kernels of hybrid decoders that alternate attention with a state-space mixer and route tokens to experts:
// a scaled embedding with sinusoidal positions, the per-head RMS norm of q and k with the write into the paged
// cache, differential attention over blocks of positions (two softmax maps over the same values, combined and
// normed per head), the short causal convolution with its per-sequence history, the selective state-space
// recurrence with a float32 state per sequence (token by token, or a prompt in segments side by side), the gated
// norm in groups behind it, plain activations, the router of a mixture of experts (logits, choice, weights), the
// weighting of the experts' hidden rows, and the lists of tokens by expert with the gather and scatter of their rows.
// The 16-bit attention on the matrix cores is diff_attention.hip.  Every size is a run-time value.
// Whatever a norm, a score, an attention weight, a decay, a step size or a recurrent state is made of is float32
// here, whatever the type of the matrices.
#include "common.h"

__device__ __forceinline__ float sigmoidf_(float z) { return 1.f / (1.f + expf(-z)); }
__device__ __forceinline__ float siluf_(float z) { return z / (1.f + expf(-z)); }
__device__ __forceinline__ float softplusf_(float z) { return z > 20.f ? z : log1pf(expf(z)); }
__device__ __forceinline__ float gelu_erff_(float z) { return 0.5f * z * (1.f + erff(z * 0.70710678118654752f)); }

#define DISPATCH_T(dt, CALL)                                     \
    do {                                                         \
        if ((dt) == DT_F32) { typedef float T; CALL; }           \
        else if ((dt) == DT_F16) { typedef f16 T; CALL; }        \
        else if ((dt) == DT_BF16) { typedef bf16 T; CALL; }      \
        else return LI_BAD_ARG;                                  \
    } while (0)

// ---------------------------------------------------------------------------
// x[t] = table[token[t]] * scale + P(pos[t]),  P(p)[2i] = sin(p f_i),  P(p)[2i+1] = cos(p f_i);  the
// frequencies f_i come from the host (float32, one for every pair).  `freq` null: no positions are added.
// ---------------------------------------------------------------------------
template <class T>
__global__ void embed_pos_kernel(const T* __restrict__ table, const int* __restrict__ tokens,
                                 const int* __restrict__ pos, const float* __restrict__ freq, float* __restrict__ out,
                                 int d, float scale) {
    const int t = blockIdx.x;
    const T* row = table + (int64_t)tokens[t] * d;
    const float p = pos ? (float)pos[t] : 0.f;
    for (int i = threadIdx.x; i < d; i += blockDim.x) {
        float v = to_f32(row[i]) * scale;
        if (freq) {
            const float a = p * freq[i >> 1];
            v += (i & 1) ? cosf(a) : sinf(a);
        }
        out[(int64_t)t * d + i] = v;
    }
}

extern "C" int li_embed_pos(const void* table, int dt, const int* tokens, const int* pos, const float* freq, float* out,
                            int n, int d, float scale, hipStream_t stream) {
    if (n <= 0) return LI_OK;
    if (d <= 0) return LI_BAD_ARG;
    DISPATCH_T(dt, (embed_pos_kernel<T><<<n, 256, 0, stream>>>((const T*)table, tokens, pos, freq, out, d, scale)));
    LI_CHECK_LAUNCH();
    return LI_OK;
}

// ---------------------------------------------------------------------------
// out[t] = [a[t] | b[t]] in type T (a, b float32 rows of width d): the input of a product over both.
// ---------------------------------------------------------------------------
template <class T>
__global__ void concat_cast_kernel(const float* __restrict__ a, const float* __restrict__ b, T* __restrict__ out, int d) {
    const int64_t t = blockIdx.x;
    for (int i = threadIdx.x; i < d; i += blockDim.x) {
        out[t * 2 * d + i] = from_f32<T>(a[t * d + i]);
        out[t * 2 * d + d + i] = from_f32<T>(b[t * d + i]);
    }
}

extern "C" int li_concat_cast(const float* a, const float* b, void* out, int dt, int n, int d, hipStream_t stream) {
    if (n <= 0) return LI_OK;
    DISPATCH_T(dt, (concat_cast_kernel<T><<<n, 256, 0, stream>>>(a, b, (T*)out, d)));
    LI_CHECK_LAUNCH();
    return LI_OK;
}

// ---------------------------------------------------------------------------
// out = act(in), float32 in, type T out.  act: 0 gelu (erf), 1 gelu (tanh), 2 silu, 3 the square of relu.
// ---------------------------------------------------------------------------
template <class T>
__global__ void activation_kernel(const float* __restrict__ in, T* __restrict__ out, int64_t n, int act) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const float z = in[i];
    const float r = fmaxf(z, 0.f);
    out[i] = from_f32<T>(act == 0 ? gelu_erff_(z) : (act == 1 ? gate_activation(z, true) : (act == 2 ? siluf_(z) : r * r)));
}

extern "C" int li_activation(const float* in, void* out, int dt, int64_t n, int act, hipStream_t stream) {
    if (n <= 0) return LI_OK;
    if (act < 0 || act > 3) return LI_BAD_ARG;
    DISPATCH_T(dt, (activation_kernel<T><<<(unsigned)((n + 255) / 256), 256, 0, stream>>>(in, (T*)out, n, act)));
    LI_CHECK_LAUNCH();
    return LI_OK;
}

// ---------------------------------------------------------------------------
// The cache of an attention whose keys are several maps wide.  A key of a token and KV head is its maps side by
// side, each padded with zeros to DP = d rounded up to 16: KW = maps * DP.  Inside a page keys and values lie in
// the order of the matrix instruction's operands (common.h, k_offset / v_offset with head size KW for the keys).
// qk_norm_store: per token, from the float32 rows of the q/k/v product (columns q | k | v from `col0` on):
// every map of every q and k head is divided by its root mean square over d and multiplied by a weight of size
// d (null: none; eps < 0: no norm at all); q goes to `q_out` [T, H, KW] in the cache's type (padded likewise), k
// and v into the page of the token's position.
// ---------------------------------------------------------------------------
struct MapPages {
    void* k;
    void* v;
    int64_t page_stride;
    const int* page_table;
    int max_pages;
};

template <class T>
__global__ void qk_norm_store_kernel(const float* __restrict__ qkv, int stride, int col0, const float* __restrict__ qw,
                                     const float* __restrict__ kw, float eps, const int* __restrict__ pos,
                                     const int* __restrict__ tok_slot, T* __restrict__ q_out, MapPages pg, int H,
                                     int G, int maps, int d, int dv) {
    const int t = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
    const float* row = qkv + (int64_t)t * stride + col0;
    const int DP = round_up(d, 16), KW = maps * DP, p = pos[t];
    const int page = pg.page_table[(int64_t)tok_slot[t] * pg.max_pages + p / PAGE], off = p % PAGE;
    T* kp = (T*)pg.k + (int64_t)page * pg.page_stride;
    T* vp = (T*)pg.v + (int64_t)page * pg.page_stride;
    const int n_units = (H + G) * maps;                   // one wave a (head, map), the units over the grid's second dimension
    for (int u = blockIdx.y * nw + wave; u < n_units; u += gridDim.y * nw) {
        const bool is_q = u < H * maps;
        const float* src = row + (int64_t)u * d;          // q heads then k heads, each maps * d wide
        float ss = 0.f;
        for (int i = lane; i < d; i += 64) ss += src[i] * src[i];
        const float r = eps >= 0.f ? 1.f / sqrtf(wave_sum(ss) / (float)d + eps) : 1.f;
        const float* w = is_q ? qw : kw;
        for (int i = lane; i < DP; i += 64) {
            const float v = i < d ? src[i] * r * (w ? w[i] : 1.f) : 0.f;
            if (is_q) q_out[(int64_t)t * H * KW + (int64_t)u * DP + i] = from_f32<T>(v);
            else {
                const int ku = u - H * maps, g = ku / maps, m = ku - g * maps;
                kp[g * k_head_elems(KW) + k_offset(off, m * DP + i, KW)] = from_f32<T>(v);
            }
        }
    }
    const float* vsrc = row + (int64_t)(H + G) * maps * d;
    for (int i = blockIdx.y * blockDim.x + threadIdx.x; i < G * dv; i += gridDim.y * blockDim.x) {
        const int g = i / dv, j = i - g * dv;
        vp[g * v_head_elems(dv) + v_offset(off, j, dv)] = from_f32<T>(vsrc[i]);
    }
}

extern "C" int li_qk_norm_store(const float* qkv, int stride, int col0, const float* qw, const float* kw, float eps,
                                const int* pos, const int* tok_slot, void* q_out, void* k_pages, void* v_pages,
                                int64_t page_stride, const int* page_table, int max_pages, int dt, int n, int H, int G,
                                int maps, int d, int dv, hipStream_t stream) {
    if (n <= 0) return LI_OK;
    if (H <= 0 || G <= 0 || maps <= 0 || d <= 0 || dv <= 0) return LI_BAD_ARG;
    MapPages pg{k_pages, v_pages, page_stride, page_table, max_pages};
    dim3 grid(n, n >= 512 ? 1 : ((H + G) * maps + 3) / 4);       // few tokens: a wave for every (head, map)
    DISPATCH_T(dt, (qk_norm_store_kernel<T><<<grid, 256, 0, stream>>>(qkv, stride, col0, qw, kw, eps, pos, tok_slot, (T*)q_out,
                                                                  pg, H, G, maps, d, dv)));
    LI_CHECK_LAUNCH();
    return LI_OK;
}

// ---------------------------------------------------------------------------
// Differential attention over blocks of positions, one workgroup per (token, query head): the kernel of the
// float32 path (the 16-bit path runs on the matrix cores, diff_attention.hip).
// A token at position p sees the keys lo .. p with lo = p - p % block (block 0: lo = 0; window w > 0: lo is at
// least p - w + 1).  Each of `maps` (1 or 2) maps is a softmax of its own over scores q_m . k_m * scale; with a_m
// the maps' weighted sums of the SAME values,  o = a_1 - lambda a_2  (one map: o = a_1).  out_eps >= 0: o is
// divided by its root mean square over dv and multiplied by out_scale.  `sink` not null: every map's sum of weights
// also counts exp(sink[head]), a score with no key and no value that is not scaled.  `slopes` not null: the score of
// the key at position j loses slopes[head] * (p - j) (the sink loses nothing).  `gate` not null: the head's output is
// multiplied by the sigmoid of gate[t][gate_col + head] (float32 rows of gate_stride numbers).  Scores, weights, sums: float32.
// The waves of the workgroup take the tiles of 64 keys in turn, a lane a key; each keeps a running maximum and
// sum per map (online softmax) and its share of the output, and the shares are merged through LDS in wave order.
// ---------------------------------------------------------------------------
#define DA_WAVES 4
#define DA_MAXV 8          // dv <= 64 * DA_MAXV

template <class T, int MAPS>
__global__ __launch_bounds__(64 * DA_WAVES) void diff_attn_kernel(
    const T* __restrict__ q, T* __restrict__ out, MapPages pg, const int* __restrict__ pos,
    const int* __restrict__ tok_slot, int H, int G, int d, int dv, float scale, int block, int window, float lambda,
    float out_eps, float out_scale, const float* __restrict__ sink, const float* __restrict__ slopes,
    const float* __restrict__ gate, int gate_stride, int gate_col) {
    extern __shared__ float lds[];
    const int DP = round_up(d, 16), KW = MAPS * DP;
    float* sq = lds;                                   // [KW]
    float* sm = sq + KW;                               // [DA_WAVES][MAPS] maxima
    float* sl = sm + DA_WAVES * MAPS;                  // [DA_WAVES][MAPS] sums
    float* so = sl + DA_WAVES * MAPS;                  // [DA_WAVES][MAPS][dv]
    __shared__ float scratch[16];
    const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int g = h / (H / G), p = pos[t];
    const float slope = slopes ? slopes[h] : 0.f;      // a score loses slope * (distance to its key)
    int lo = block > 0 ? p - p % block : 0;
    if (window > 0) lo = max(lo, p - window + 1);
    for (int i = threadIdx.x; i < KW; i += blockDim.x) sq[i] = to_f32(q[((int64_t)t * H + h) * KW + i]);
    __syncthreads();
    const int* table = pg.page_table + (int64_t)tok_slot[t] * pg.max_pages;
    float m[MAPS], l[MAPS], o[MAPS][DA_MAXV];
#pragma unroll
    for (int a = 0; a < MAPS; ++a) {
        m[a] = -INFINITY; l[a] = 0.f;
#pragma unroll
        for (int c = 0; c < DA_MAXV; ++c) o[a][c] = 0.f;
    }
    const int n_tiles = (p - lo) / 64 + 1;
    for (int tile = wave; tile < n_tiles; tile += DA_WAVES) {
        const int j = lo + tile * 64 + lane;           // this lane's key
        float s[MAPS];
        const T* kh = nullptr;
        if (j <= p) kh = (const T*)pg.k + (int64_t)table[j / PAGE] * pg.page_stride + g * k_head_elems(KW);
#pragma unroll
        for (int a = 0; a < MAPS; ++a) {
            float acc = 0.f;
            if (kh) for (int i = 0; i < d; ++i) acc += sq[a * DP + i] * to_f32(kh[k_offset(j % PAGE, a * DP + i, KW)]);
            s[a] = kh ? acc * scale - slope * (float)(p - j) : -INFINITY;
        }
        float pw[MAPS];
#pragma unroll
        for (int a = 0; a < MAPS; ++a) {
            const float mt = fmaxf(m[a], wave_max(s[a]));          // lane 0's key is always visible: finite
            const float f = expf(m[a] - mt);                       // 0 the first time (m = -inf)
            pw[a] = kh ? expf(s[a] - mt) : 0.f;
            l[a] = l[a] * f + wave_sum(pw[a]);
            m[a] = mt;
#pragma unroll
            for (int c = 0; c < DA_MAXV; ++c) o[a][c] *= f;
        }
        const int n_keys = min(64, p - (lo + tile * 64) + 1);
        for (int kk = 0; kk < n_keys; ++kk) {
            const int jj = lo + tile * 64 + kk;
            const T* vh = (const T*)pg.v + (int64_t)table[jj / PAGE] * pg.page_stride + g * v_head_elems(dv);
            float w[MAPS];
#pragma unroll
            for (int a = 0; a < MAPS; ++a) w[a] = __shfl(pw[a], kk, WAVE);
#pragma unroll
            for (int c = 0; c < DA_MAXV; ++c) {
                const int i = lane + 64 * c;
                if (i < dv) {
                    const float v = to_f32(vh[v_offset(jj % PAGE, i, dv)]);
#pragma unroll
                    for (int a = 0; a < MAPS; ++a) o[a][c] += w[a] * v;
                }
            }
        }
    }
    // merge the waves' shares in wave order
#pragma unroll
    for (int a = 0; a < MAPS; ++a) {
        if (lane == 0) { sm[wave * MAPS + a] = m[a]; sl[wave * MAPS + a] = l[a]; }
#pragma unroll
        for (int c = 0; c < DA_MAXV; ++c) {
            const int i = lane + 64 * c;
            if (i < dv) so[(wave * MAPS + a) * dv + i] = o[a][c];
        }
    }
    __syncthreads();
    float ss = 0.f;
    float res[DA_MAXV];
#pragma unroll
    for (int c = 0; c < DA_MAXV; ++c) res[c] = 0.f;
    if (wave == 0) {
#pragma unroll
        for (int c = 0; c < DA_MAXV; ++c) {
            const int i = lane + 64 * c;
            if (i < dv) {
                float am[MAPS];
#pragma unroll
                for (int a = 0; a < MAPS; ++a) {
                    float M = sm[a];
                    for (int w = 1; w < DA_WAVES; ++w) M = fmaxf(M, sm[w * MAPS + a]);
                    if (sink) M = fmaxf(M, sink[h]);
                    float L = sink ? expf(sink[h] - M) : 0.f, O = 0.f;
                    for (int w = 0; w < DA_WAVES; ++w) {
                        const float mw = sm[w * MAPS + a];
                        const float f = mw == -INFINITY ? 0.f : expf(mw - M);
                        L += sl[w * MAPS + a] * f;
                        O += so[(w * MAPS + a) * dv + i] * f;
                    }
                    am[a] = O / L;
                }
                res[c] = MAPS == 2 ? am[0] - lambda * am[MAPS - 1] : am[0];
                ss += res[c] * res[c];
            }
        }
    }
    float r = out_scale;
    if (out_eps >= 0.f) r = out_scale / sqrtf(block_sum(ss, scratch) / (float)dv + out_eps);   // waves 1.. add 0
    if (gate) r *= sigmoidf_(gate[(int64_t)t * gate_stride + gate_col + h]);                   // one number a head
    if (wave == 0) {
#pragma unroll
        for (int c = 0; c < DA_MAXV; ++c) {
            const int i = lane + 64 * c;
            if (i < dv) out[((int64_t)t * H + h) * dv + i] = from_f32<T>(res[c] * r);
        }
    }
}

extern "C" int li_diff_attn(const void* q, void* out, int dt, void* k_pages, void* v_pages, int64_t page_stride,
                            const int* page_table, int max_pages, const int* pos, const int* tok_slot, int n, int H, int G,
                            int maps, int d, int dv, float scale, int block, int window, float lambda, float out_eps,
                            float out_scale, const float* sink, const float* slopes, const float* gate, int gate_stride,
                            int gate_col, hipStream_t stream) {
    if (n <= 0) return LI_OK;
    if (H <= 0 || G <= 0 || H % G || d <= 0 || dv <= 0 || block < 0 || window < 0) return LI_BAD_ARG;
    if (gate && (gate_col < 0 || gate_col + H > gate_stride)) return LI_BAD_ARG;
    if (maps < 1 || maps > 2 || dv > 64 * DA_MAXV) return LI_UNSUPPORTED;
    MapPages pg{k_pages, v_pages, page_stride, page_table, max_pages};
    dim3 grid(n, H), blk(64 * DA_WAVES);
    const size_t lds = (size_t)(maps * round_up(d, 16) + 2 * DA_WAVES * maps + DA_WAVES * maps * dv) * sizeof(float);
    if (lds > 60000) return LI_UNSUPPORTED;
#define GO(M) diff_attn_kernel<T, M><<<grid, blk, lds, stream>>>((const T*)q, (T*)out, pg, pos, tok_slot, H, G, d, dv, scale, \
                                                                 block, window, lambda, out_eps, out_scale, sink, slopes, gate, \
                                                                 gate_stride, gate_col)
    DISPATCH_T(dt, { if (maps == 1) GO(1); else GO(2); });
#undef GO
    LI_CHECK_LAUNCH();
    return LI_OK;
}

// ---------------------------------------------------------------------------
// A short causal convolution per channel with its activation:
//   out[t][c] = silu(b[c] + sum over j < taps of w[c][j] u[t - (taps - 1 - j)][c])
// u are `channels` columns of the float32 rows `in` from column `col0` on.  Inputs before the first token that a
// sequence brings to this step come from its history `hist` [slots, taps - 1, channels] (the last taps - 1 inputs
// of the steps before, oldest first); before position 0 they are zero.  conv_history_kernel then leaves every
// sequence's last taps - 1 inputs there.
// ---------------------------------------------------------------------------
#define CONV_MAX_TAPS 16

template <class T, bool SILU, bool ADD>
__global__ void conv_silu_kernel(const float* __restrict__ in, int stride, int col0, const float* __restrict__ w,
                                 const float* __restrict__ b, const float* __restrict__ hist, const int* __restrict__ pos,
                                 const int* __restrict__ tok_slot, T* __restrict__ out, int channels, int taps) {
    const int t = blockIdx.x, p = pos[t], slot = tok_slot[t];
    // how many tokens before this one its sequence has in this step (at most taps - 1 matter)
    int inside = 0;
    while (inside < taps - 1 && t - inside - 1 >= 0 && tok_slot[t - inside - 1] == slot) ++inside;
    const float* h = hist + (int64_t)slot * (taps - 1) * channels;
    for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < channels; c += gridDim.y * blockDim.x) {
        float acc = b ? b[c] : 0.f;
        for (int back = 0; back < taps; ++back) {                  // back = taps - 1 - j
            float u = 0.f;
            if (back <= inside) u = in[(int64_t)(t - back) * stride + col0 + c];
            else if (p - back >= 0) u = h[(int64_t)(taps - 1 - (back - inside)) * channels + c];
            acc += w[(int64_t)c * taps + (taps - 1 - back)] * u;
        }
        if (ADD) acc += in[(int64_t)t * stride + col0 + c];        // the input itself beside its convolution
        out[(int64_t)t * channels + c] = from_f32<T>(SILU ? siluf_(acc) : acc);
    }
}

__global__ void conv_history_kernel(const float* __restrict__ in, int stride, int col0, float* __restrict__ hist,
                                    const int* __restrict__ seq_slot, const int* __restrict__ seq_qstart,
                                    const int* __restrict__ seq_qlen, int channels, int taps) {
    const int seq = blockIdx.x;
    const int q0 = seq_qstart ? seq_qstart[seq] : seq, n = seq_qlen ? seq_qlen[seq] : 1;
    float* h = hist + (int64_t)seq_slot[seq] * (taps - 1) * channels;
    for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < channels; c += gridDim.y * blockDim.x) {
        float keep[CONV_MAX_TAPS];
        for (int r = 0; r < taps - 1; ++r) {
            const int back = taps - 1 - r;                          // row r holds the input `back` tokens before the next
            keep[r] = back <= n ? in[(int64_t)(q0 + n - back) * stride + col0 + c] : h[(int64_t)(r + n) * channels + c];
        }
        for (int r = 0; r < taps - 1; ++r) h[(int64_t)r * channels + c] = keep[r];
    }
}

extern "C" int li_conv_silu(const float* in, int stride, int col0, const float* w, const float* b, float* hist,
                            const int* pos, const int* tok_slot, const int* seq_slot, const int* seq_qstart,
                            const int* seq_qlen, float* out, int n_tokens, int n_seqs, int channels, int taps,
                            hipStream_t stream) {
    if (n_tokens <= 0) return LI_OK;
    if (channels <= 0 || taps < 1 || taps > CONV_MAX_TAPS) return LI_BAD_ARG;
    dim3 cgrid(n_tokens, (channels + 255) / 256);
    conv_silu_kernel<float, true, false><<<cgrid, 256, 0, stream>>>(in, stride, col0, w, b, hist, pos, tok_slot, out, channels, taps);
    if (taps > 1) {
        dim3 grid(n_seqs, (channels + 255) / 256);
        conv_history_kernel<<<grid, 256, 0, stream>>>(in, stride, col0, hist, seq_slot, seq_qstart, seq_qlen, channels, taps);
    }
    LI_CHECK_LAUNCH();
    return LI_OK;
}

// The same convolution without an activation, the input added to it: out = u + conv(u), in type dt (what a mixer
// reads when its input first passes a short convolution over time).
extern "C" int li_conv_add(const float* in, int stride, int col0, const float* w, const float* b, float* hist,
                           const int* pos, const int* tok_slot, const int* seq_slot, const int* seq_qstart,
                           const int* seq_qlen, void* out, int dt, int n_tokens, int n_seqs, int channels, int taps,
                           hipStream_t stream) {
    if (n_tokens <= 0) return LI_OK;
    if (channels <= 0 || taps < 1 || taps > CONV_MAX_TAPS) return LI_BAD_ARG;
    dim3 cgrid(n_tokens, (channels + 255) / 256);
    DISPATCH_T(dt, (conv_silu_kernel<T, false, true><<<cgrid, 256, 0, stream>>>(in, stride, col0, w, b, hist, pos, tok_slot, (T*)out,
                                                                                channels, taps)));
    if (taps > 1) {
        dim3 grid(n_seqs, (channels + 255) / 256);
        conv_history_kernel<<<grid, 256, 0, stream>>>(in, stride, col0, hist, seq_slot, seq_qstart, seq_qlen, channels, taps);
    }
    LI_CHECK_LAUNCH();
    return LI_OK;
}

// A sequence's last taps - 1 inputs brought up to date alone (for a kernel that convolves while it does something else
// and only reads the history).
extern "C" int li_conv_history(const float* in, int stride, int col0, float* hist, const int* seq_slot, const int* seq_qstart,
                               const int* seq_qlen, int n_seqs, int channels, int taps, hipStream_t stream) {
    if (n_seqs <= 0 || taps <= 1) return LI_OK;
    if (channels <= 0 || taps > CONV_MAX_TAPS) return LI_BAD_ARG;
    dim3 grid(n_seqs, (channels + 255) / 256);
    conv_history_kernel<<<grid, 256, 0, stream>>>(in, stride, col0, hist, seq_slot, seq_qstart, seq_qlen, channels, taps);
    LI_CHECK_LAUNCH();
    return LI_OK;
}

// ---------------------------------------------------------------------------
// The selective state-space recurrence.  Per sequence and head h (group g = h / (P / G)), with x_t [dv],
// B_t, C_t [N] from the rows `xbc` (columns x | B | C) and the raw step size from `proj` column dt_col + h:
//   dt = softplus(raw + dt_bias[h]);   a = exp(-exp(A_log[h]) dt)
//   S <- a S + dt B_t x_t^T   (S is N x dv, float32, kept for every sequence in `state` [slots, P, N, dv])
//   y_t = S^T C_t + D[h] x_t
// One wave per (sequence, head, 64 columns of dv): a lane keeps its column of S in registers for all the tokens
// that the sequence brings; B_t and C_t lie across the lanes and reach every lane by lane reads.
// ---------------------------------------------------------------------------
// A prompt may also be walked in segments (ScanPlan): pass 1 runs every segment from a zero state and leaves its own
// contribution and the product of its decays; ssm_combine_kernel walks a sequence's segments in order, S <- a_seg S +
// D_seg, leaving the state before every segment where its contribution was; pass 3 runs every segment again from
// that state and writes y.  Twice the arithmetic, and as many waves as there are segments instead of sequences.
struct ScanPlan {
    int pass;                   // 0: a sequence's tokens in order; 1 and 3: see above
    const int* seg_seq;         // [segments] the sequence of a segment
    const int* seg_t0;          // [segments] its first token among the sequence's tokens of this step
    const int* seg_n;           // [segments] its tokens
    float* seg_state;           // [segments, P, N, dv]
    float* seg_decay;           // [segments, P]
};

template <int NMAX, int PASS>
__global__ __launch_bounds__(64) void ssm_scan_kernel(
    const float* __restrict__ xbc, int xbc_stride, const float* __restrict__ proj, int proj_stride, int dt_col,
    const float* __restrict__ dt_bias, const float* __restrict__ A_log, const float* __restrict__ D,
    float* __restrict__ state, const int* __restrict__ seq_slot, const int* __restrict__ seq_qstart,
    const int* __restrict__ seq_qlen, float* __restrict__ y, int P, int G, int N, int dv, ScanPlan plan) {
    const int h = blockIdx.y, lane = threadIdx.x, col = blockIdx.z * 64 + lane;
    const int g = h / (P / G), inner = P * dv;
    int q0, n;
    float* S;
    if (PASS == 0) {
        const int seq = blockIdx.x;
        q0 = seq_qstart ? seq_qstart[seq] : seq;
        n = seq_qlen ? seq_qlen[seq] : 1;
        S = state + (((int64_t)seq_slot[seq] * P + h) * N) * dv + col;
    } else {
        const int seg = blockIdx.x;
        q0 = seq_qstart[plan.seg_seq[seg]] + plan.seg_t0[seg];
        n = plan.seg_n[seg];
        S = plan.seg_state + (((int64_t)seg * P + h) * N) * dv + col;
    }
    const bool live = col < dv;
    float s[NMAX];
#pragma unroll
    for (int i = 0; i < NMAX; ++i) s[i] = (live && i < N && PASS != 1) ? S[(int64_t)i * dv] : 0.f;
    const float negA = -expf(A_log[h]), bias = dt_bias[h], dh = D ? D[h] : 0.f;
    const int b_off = inner + g * N, c_off = inner + G * N + g * N;
    float log_decay = 0.f;
    // B_t and C_t are the same for all lanes: lane j fetches elements j, j + 64, ... (a token ahead, so that the wait for
    // memory lies under the token at work), and element i reaches all lanes by a lane read, which costs no memory
    // or LDS bandwidth.  Elements from N on are zero and leave the state's zeros as they are.
    constexpr int NV = (NMAX + 63) / 64;
    float bv[NV], cv[NV], x = 0.f, dt = 0.f;
    auto fetch = [&](int t) {
        const float* __restrict__ row = xbc + (int64_t)(q0 + t) * xbc_stride;
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            const int i = v * 64 + lane;
            bv[v] = i < N ? row[b_off + i] : 0.f;
            cv[v] = i < N ? row[c_off + i] : 0.f;
        }
        x = live ? row[h * dv + col] : 0.f;
        dt = proj[(int64_t)(q0 + t) * proj_stride + dt_col + h];
    };
    if (n > 0) fetch(0);
    for (int t = 0; t < n; ++t) {
        float bt[NV], ct[NV];
#pragma unroll
        for (int v = 0; v < NV; ++v) { bt[v] = bv[v]; ct[v] = cv[v]; }
        const float xt = x, dtt = softplusf_(dt + bias);
        if (t + 1 < n) fetch(t + 1);
        const float lda = negA * dtt, a = expf(lda);
        log_decay += lda;
        const float dx = dtt * xt;
        float acc = 0.f;
#pragma unroll
        for (int i = 0; i < NMAX; ++i) {
            const float b = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(bt[i >> 6]), i & 63));
            s[i] = a * s[i] + b * dx;
            if (PASS != 1) {
                const float c = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(ct[i >> 6]), i & 63));
                acc += s[i] * c;
            }
        }
        if (live && PASS != 1) y[(int64_t)(q0 + t) * inner + h * dv + col] = acc + dh * xt;
    }
    if (live && PASS != 3) {
#pragma unroll
        for (int i = 0; i < NMAX; ++i) if (i < N) S[(int64_t)i * dv] = s[i];
    }
    if (PASS == 1 && lane == 0 && blockIdx.z == 0) plan.seg_decay[(int64_t)blockIdx.x * P + h] = expf(log_decay);
}

// One thread per element of a head's state: walks the sequence's segments in order.
__global__ void ssm_combine_kernel(float* __restrict__ state, const int* __restrict__ seq_slot,
                                   const int* __restrict__ seq_seg0, const int* __restrict__ seq_nseg,
                                   float* __restrict__ seg_state, const float* __restrict__ seg_decay, int P, int64_t per_head) {
    const int seq = blockIdx.x, h = blockIdx.y;
    const int c0 = seq_seg0[seq], nc = seq_nseg[seq];
    for (int64_t e = (int64_t)blockIdx.z * blockDim.x + threadIdx.x; e < per_head; e += (int64_t)gridDim.z * blockDim.x) {
        float* S = state + ((int64_t)seq_slot[seq] * P + h) * per_head + e;
        float s = *S;
        for (int c = c0; c < c0 + nc; ++c) {
            float* L = seg_state + ((int64_t)c * P + h) * per_head + e;
            const float own = *L;
            *L = s;
            s = seg_decay[(int64_t)c * P + h] * s + own;
        }
        *S = s;
    }
}

#define SSM_GO(NM, GRID, PLAN) ssm_scan_kernel<NM, SSM_PASS><<<GRID, 64, 0, stream>>>(xbc, xbc_stride, proj, proj_stride, dt_col, \
        dt_bias, A_log, D, state, seq_slot, seq_qstart, seq_qlen, y, P, G, N, dv, PLAN)
#define SSM_LAUNCH(GRID, PLAN)                                                                  \
    do {                                                                                        \
        if (N <= 16) SSM_GO(16, GRID, PLAN); else if (N <= 32) SSM_GO(32, GRID, PLAN);          \
        else if (N <= 64) SSM_GO(64, GRID, PLAN); else if (N <= 128) SSM_GO(128, GRID, PLAN);   \
        else SSM_GO(256, GRID, PLAN);                                                           \
    } while (0)

extern "C" int li_ssm_scan(const float* xbc, int xbc_stride, const float* proj, int proj_stride, int dt_col,
                           const float* dt_bias, const float* A_log, const float* D, float* state, const int* seq_slot,
                           const int* seq_qstart, const int* seq_qlen, float* y, int n_seqs, int P, int G, int N, int dv,
                           hipStream_t stream) {
    if (n_seqs <= 0) return LI_OK;
    if (P <= 0 || G <= 0 || P % G || N <= 0 || dv <= 0) return LI_BAD_ARG;
    if (N > 256) return LI_UNSUPPORTED;
    dim3 grid(n_seqs, P, (dv + 63) / 64);
    ScanPlan plan{0, nullptr, nullptr, nullptr, nullptr, nullptr};
#define SSM_PASS 0
    SSM_LAUNCH(grid, plan);
#undef SSM_PASS
    LI_CHECK_LAUNCH();
    return LI_OK;
}

// The same recurrence with every sequence's tokens cut into segments that run side by side (see ScanPlan).
// seg_state [segments, P, N, dv] and seg_decay [segments, P] are scratch memory of the caller.
extern "C" int li_ssm_scan_segments(const float* xbc, int xbc_stride, const float* proj, int proj_stride, int dt_col,
                                    const float* dt_bias, const float* A_log, const float* D, float* state,
                                    const int* seq_slot, const int* seq_qstart, const int* seq_qlen, float* y, int n_seqs,
                                    int P, int G, int N, int dv, const int* seg_seq, const int* seg_t0, const int* seg_n,
                                    const int* seq_seg0, const int* seq_nseg, int n_segs, float* seg_state, float* seg_decay,
                                    hipStream_t stream) {
    if (n_seqs <= 0 || n_segs <= 0) return LI_OK;
    if (P <= 0 || G <= 0 || P % G || N <= 0 || dv <= 0 || !seq_qstart || !seq_qlen) return LI_BAD_ARG;
    if (N > 256) return LI_UNSUPPORTED;
    dim3 grid(n_segs, P, (dv + 63) / 64);
    ScanPlan plan{1, seg_seq, seg_t0, seg_n, seg_state, seg_decay};
#define SSM_PASS 1
    SSM_LAUNCH(grid, plan);
#undef SSM_PASS
    const int64_t per_head = (int64_t)N * dv;
    dim3 cgrid(n_seqs, P, (unsigned)((per_head + 255) / 256));
    ssm_combine_kernel<<<cgrid, 256, 0, stream>>>(state, seq_slot, seq_seg0, seq_nseg, seg_state, seg_decay, P, per_head);
    plan.pass = 3;
#define SSM_PASS 3
    SSM_LAUNCH(grid, plan);
#undef SSM_PASS
    LI_CHECK_LAUNCH();
    return LI_OK;
}

// ---------------------------------------------------------------------------
// out = N_g(y * silu(z)) * w: the gate first, then each of `groups` equal parts of a row divided by its own
// root mean square.  y float32 [T, n]; z: n columns of the float32 rows `zrows` from column z_col on.
// ---------------------------------------------------------------------------
template <class T>
__global__ void gated_group_norm_kernel(const float* __restrict__ y, const float* __restrict__ zrows, int z_stride,
                                        int z_col, const float* __restrict__ w, T* __restrict__ out, int n, int groups,
                                        float eps) {
    __shared__ float scratch[16];
    const int t = blockIdx.x, grp = blockIdx.y, part = n / groups;
    const float* yr = y + (int64_t)t * n + grp * part;
    const float* zr = zrows + (int64_t)t * z_stride + z_col + grp * part;
    float ss = 0.f;
    for (int i = threadIdx.x; i < part; i += blockDim.x) { const float v = yr[i] * siluf_(zr[i]); ss += v * v; }
    const float r = 1.f / sqrtf(block_sum(ss, scratch) / (float)part + eps);
    for (int i = threadIdx.x; i < part; i += blockDim.x)
        out[(int64_t)t * n + grp * part + i] = from_f32<T>(yr[i] * siluf_(zr[i]) * r * w[grp * part + i]);
}

extern "C" int li_gated_group_norm(const float* y, const float* zrows, int z_stride, int z_col, const float* w, void* out,
                                   int dt, int n_rows, int n, int groups, float eps, hipStream_t stream) {
    if (n_rows <= 0) return LI_OK;
    if (n <= 0 || groups <= 0 || n % groups) return LI_BAD_ARG;
    dim3 grid(n_rows, groups);
    const int threads = n / groups >= 4096 ? 1024 : (n / groups >= 1024 ? 512 : 256);
    DISPATCH_T(dt, (gated_group_norm_kernel<T><<<grid, threads, 0, stream>>>(y, zrows, z_stride, z_col, w, (T*)out, n, groups, eps)));
    LI_CHECK_LAUNCH();
    return LI_OK;
}

// ---------------------------------------------------------------------------
// out[t][j] = w[j] . h[t] in float32 for a few rows of a float32 matrix w [n, width] (a router's): one
// workgroup per (token, output), its threads stride the width; every sum has one fixed order whatever the batch.
// ---------------------------------------------------------------------------
template <class T, int TOK>
__global__ __launch_bounds__(256) void small_logits_kernel(const T* __restrict__ h, const float* __restrict__ w,
                                                           float* __restrict__ out, int n_rows, int width, int n) {
    __shared__ float scratch[16];
    const int t0 = blockIdx.x * TOK, j = blockIdx.y, tid = threadIdx.x;
    const float* wj = w + (int64_t)j * width;
    float part[TOK][16];
#pragma unroll
    for (int k = 0; k < TOK; ++k)
#pragma unroll
        for (int u = 0; u < 16; ++u) part[k][u] = 0.f;
    for (int i0 = 0; i0 < width; i0 += 4096) {             // sixteen independent loads of each operand a thread at a time
#pragma unroll
        for (int u = 0; u < 16; ++u) {
            const int i = i0 + u * 256 + tid;
            if (i < width) {
                const float wv = wj[i];                    // a weight is fetched once for the workgroup's TOK tokens
#pragma unroll
                for (int k = 0; k < TOK; ++k)
                    if (t0 + k < n_rows) part[k][u] += wv * to_f32(h[(int64_t)(t0 + k) * width + i]);
            }
        }
    }
#pragma unroll
    for (int k = 0; k < TOK; ++k) {                        // the same order of sums for a token whatever TOK is
        float acc = 0.f;
#pragma unroll
        for (int u = 0; u < 16; ++u) acc += part[k][u];
        acc = block_sum(acc, scratch);                     // the waves' sums in wave order
        if (tid == 0 && t0 + k < n_rows) out[(int64_t)(t0 + k) * n + j] = acc;
    }
}

extern "C" int li_small_logits(const void* h, int dt, const float* w, float* out, int n_rows, int width, int n,
                               hipStream_t stream) {
    if (n_rows <= 0 || n <= 0) return LI_OK;
    if (width <= 0 || n > 65535) return LI_BAD_ARG;
    if (n_rows >= 256) {                                   // many tokens: four a workgroup share every weight fetched
        dim3 grid((n_rows + 3) / 4, n);
        DISPATCH_T(dt, (small_logits_kernel<T, 4><<<grid, 256, 0, stream>>>((const T*)h, w, out, n_rows, width, n)));
    } else {
        dim3 grid(n_rows, n);
        DISPATCH_T(dt, (small_logits_kernel<T, 1><<<grid, 256, 0, stream>>>((const T*)h, w, out, n_rows, width, n)));
    }
    LI_CHECK_LAUNCH();
    return LI_OK;
}

// ---------------------------------------------------------------------------
// The router of a mixture of experts, one wave per token.  `logits` float32 [T, n_cols]: n_route router outputs,
// then (has_gate 1) one column whose sigmoid weighs an expert that every token uses (has_gate 2: its weight is 1).  s = softmax over the n_route
// outputs; the `top` outputs with the largest s + correction are chosen (the first of equals); their weights are
// s / (sum of the chosen s + 1e-20) * route_scale.  The first n_real outputs are experts with matrices: their
// weights (0 where not chosen) go to `weights` [T, n_real (+ 1)], the gate's sigmoid into the last column.  The
// outputs behind them pass the token's input on: residual[t] += (sum of their weights) * h[t].
// `sigmoid_scores`: s = sigmoid of every output's logit instead of the softmax.  `renorm` 0: a chosen output's weight
// is its own s * route_scale, not divided by the sum of the chosen.
// ---------------------------------------------------------------------------
template <class T>
__global__ __launch_bounds__(64) void moe_route_kernel(const float* __restrict__ logits, int n_cols,
                                                       const float* __restrict__ correction, const T* __restrict__ h,
                                                       float* __restrict__ residual, float* __restrict__ weights,
                                                       int width, int n_route, int n_real, int top, int has_gate,
                                                       float route_scale, int sigmoid_scores, int renorm) {
    extern __shared__ float lds[];
    float* s = lds;                      // [n_route] softmax scores
    float* c = s + n_route;              // [n_route] choice scores, -inf once chosen
    const int t = blockIdx.x, lane = threadIdx.x;
    const float* z = logits + (int64_t)t * n_cols;
    float mx = -INFINITY;
    for (int i = lane; i < n_route; i += 64) mx = fmaxf(mx, z[i]);
    mx = wave_max(mx);
    float sum = 0.f;
    for (int i = lane; i < n_route; i += 64) { const float e = expf(z[i] - mx); s[i] = e; sum += e; }
    sum = wave_sum(sum);
    if (sigmoid_scores) {
        sum = 1.f;
        for (int i = lane; i < n_route; i += 64) s[i] = sigmoidf_(z[i]);
    }
    const int wcols = n_real + (has_gate ? 1 : 0);
    for (int i = lane; i < n_route; i += 64) {
        s[i] /= sum;
        c[i] = s[i] + (correction ? correction[i] : 0.f);
    }
    for (int i = lane; i < wcols; i += 64) weights[(int64_t)t * wcols + i] = 0.f;
    __syncthreads();
    float chosen_sum = 0.f;
    for (int k = 0; k < top; ++k) {
        float best = -INFINITY; int bi = 0x7fffffff;
        for (int i = lane; i < n_route; i += 64) if (c[i] > best) { best = c[i]; bi = i; }
        for (int o = 32; o > 0; o >>= 1) {
            const float ob = __shfl_xor(best, o, WAVE); const int oi = __shfl_xor(bi, o, WAVE);
            if (ob > best || (ob == best && oi < bi)) { best = ob; bi = oi; }
        }
        chosen_sum += s[bi];
        __syncthreads();
        if (lane == 0) c[bi] = -INFINITY;
        __syncthreads();
    }
    const float f = renorm ? route_scale / (chosen_sum + 1e-20f) : route_scale;
    float pass = 0.f;                    // the weight of the outputs that pass the input on
    // every lane knows the chosen set through c == -inf
    for (int i = lane; i < n_route; i += 64) {
        if (c[i] == -INFINITY) {
            const float w = s[i] * f;
            if (i < n_real) weights[(int64_t)t * wcols + i] = w; else pass += w;
        }
    }
    pass = wave_sum(pass);
    if (has_gate && lane == 0) weights[(int64_t)t * wcols + n_real] = has_gate == 2 ? 1.f : sigmoidf_(z[n_route]);
    if (pass != 0.f)
        for (int i = lane; i < width; i += 64) residual[(int64_t)t * width + i] += pass * to_f32(h[(int64_t)t * width + i]);
}

extern "C" int li_moe_route(const float* logits, int n_cols, const float* correction, const void* h, int dt,
                            float* residual, float* weights, int n, int width, int n_route, int n_real, int top,
                            int has_gate, float route_scale, int sigmoid_scores, int renorm, hipStream_t stream) {
    if (n <= 0) return LI_OK;
    if (n_route <= 0 || n_real < 0 || n_real > n_route || top < 1 || top > n_route || n_cols < n_route + (has_gate == 1 ? 1 : 0) ||
        has_gate < 0 || has_gate > 2)
        return LI_BAD_ARG;
    if (n_route > 4096) return LI_UNSUPPORTED;
    const size_t lds = (size_t)2 * n_route * sizeof(float);
    DISPATCH_T(dt, (moe_route_kernel<T><<<n, 64, lds, stream>>>(logits, n_cols, correction, (const T*)h, residual, weights,
                                                                 width, n_route, n_real, top, has_gate, route_scale,
                                                                 sigmoid_scores, renorm)));
    LI_CHECK_LAUNCH();
    return LI_OK;
}

// ---------------------------------------------------------------------------
// The experts' hidden rows side by side, t [T, n_blocks * ff + tail]: block e of a row is multiplied by
// weights[t][e], the tail (an expert of another width that every token uses) by weights[t][n_blocks].
// ---------------------------------------------------------------------------
template <class T>
__global__ void scale_blocks_kernel(T* __restrict__ t, const float* __restrict__ weights, int n_blocks, int ff, int tail) {
    const int64_t row = blockIdx.x;
    const int cols = n_blocks * ff + tail, wcols = n_blocks + (tail ? 1 : 0);
    for (int i = blockIdx.y * blockDim.x + threadIdx.x; i < cols; i += gridDim.y * blockDim.x) {
        const int e = i < n_blocks * ff ? i / ff : n_blocks;
        const float w = weights[row * wcols + e];
        t[row * cols + i] = from_f32<T>(w == 0.f ? 0.f : to_f32(t[row * cols + i]) * w);
    }
}

extern "C" int li_scale_blocks(void* t, int dt, const float* weights, int n, int n_blocks, int ff, int tail,
                               hipStream_t stream) {
    if (n <= 0) return LI_OK;
    if (n_blocks < 0 || ff < 0 || tail < 0) return LI_BAD_ARG;
    const int cols = n_blocks * ff + tail;
    dim3 grid(n, n >= 1024 ? 1 : (cols + 1023) / 1024);        // few rows: the columns over the grid as well
    DISPATCH_T(dt, (scale_blocks_kernel<T><<<grid, 256, 0, stream>>>((T*)t, weights, n_blocks, ff, tail)));
    LI_CHECK_LAUNCH();
    return LI_OK;
}

// ---------------------------------------------------------------------------
// Tokens sorted by expert, for prompts long enough that every expert gets a product of its own.
// moe_bucket_kernel: workgroup e lists, in ascending order, the tokens whose weight for expert e is not zero
// (idx [E, T]) and counts them (counts [E]).  gather_rows: out[r] = h[idx[r]].  scatter_add_rows:
// residual[idx[r]] += weights[idx[r]][col] * y[r]  (idx null: row r itself).
// ---------------------------------------------------------------------------
__global__ void moe_bucket_kernel(const float* __restrict__ weights, int wcols, int n_tokens, int* __restrict__ idx,
                                  int* __restrict__ counts) {
    __shared__ int part[256];
    const int e = blockIdx.x, tid = threadIdx.x;
    const int per = (n_tokens + 255) / 256, lo = min(n_tokens, tid * per), hi = min(n_tokens, lo + per);
    int mine = 0;
    for (int t = lo; t < hi; ++t) mine += weights[(int64_t)t * wcols + e] != 0.f;
    part[tid] = mine;
    __syncthreads();
    if (tid == 0) {
        int run = 0;
        for (int i = 0; i < 256; ++i) { const int c = part[i]; part[i] = run; run += c; }
        counts[e] = run;
    }
    __syncthreads();
    int at = part[tid];
    for (int t = lo; t < hi; ++t)
        if (weights[(int64_t)t * wcols + e] != 0.f) idx[(int64_t)e * n_tokens + at++] = t;
}

extern "C" int li_moe_buckets(const float* weights, int wcols, int n_tokens, int n_experts, int* idx, int* counts,
                              hipStream_t stream) {
    if (n_tokens <= 0 || n_experts <= 0) return LI_OK;
    if (wcols < n_experts) return LI_BAD_ARG;
    moe_bucket_kernel<<<n_experts, 256, 0, stream>>>(weights, wcols, n_tokens, idx, counts);
    LI_CHECK_LAUNCH();
    return LI_OK;
}

template <class T>
__global__ void gather_rows_kernel(const T* __restrict__ h, const int* __restrict__ idx, T* __restrict__ out, int width) {
    const int64_t r = blockIdx.x, src = idx[r];
    for (int i = blockIdx.y * blockDim.x + threadIdx.x; i < width; i += gridDim.y * blockDim.x)
        out[r * width + i] = h[src * width + i];
}

extern "C" int li_gather_rows(const void* h, int dt, const int* idx, void* out, int n, int width, hipStream_t stream) {
    if (n <= 0) return LI_OK;
    if (width <= 0) return LI_BAD_ARG;
    dim3 grid(n, n >= 1024 ? 1 : (width + 1023) / 1024);
    DISPATCH_T(dt, (gather_rows_kernel<T><<<grid, 256, 0, stream>>>((const T*)h, idx, (T*)out, width)));
    LI_CHECK_LAUNCH();
    return LI_OK;
}

__global__ void scatter_add_rows_kernel(float* __restrict__ residual, const float* __restrict__ y,
                                        const int* __restrict__ idx, const float* __restrict__ weights, int wcols, int col,
                                        int width) {
    const int64_t r = blockIdx.x, dst = idx ? idx[r] : r;
    const float w = col >= 0 ? weights[dst * wcols + col] : 1.f;        // col < 0: the rows are added as they are
    for (int i = blockIdx.y * blockDim.x + threadIdx.x; i < width; i += gridDim.y * blockDim.x)
        residual[dst * width + i] += w * y[r * width + i];
}

extern "C" int li_scatter_add_rows(float* residual, const float* y, const int* idx, const float* weights, int wcols,
                                   int col, int n, int width, hipStream_t stream) {
    if (n <= 0) return LI_OK;
    if (width <= 0 || col >= wcols) return LI_BAD_ARG;
    dim3 grid(n, n >= 1024 ? 1 : (width + 1023) / 1024);
    scatter_add_rows_kernel<<<grid, 256, 0, stream>>>(residual, y, idx, weights, wcols, col, width);
    LI_CHECK_LAUNCH();
    return LI_OK;
}
