// Kernels of decoders whose sub-layers stand between two norms and whose softmax attention carries a sink, a gate
// per head and either a rotation of half-paired dimensions or a bias by distance: a bias added to the columns of a
// product's float32 rows, the rotation of q and k with the write of keys and values into the paged cache, the norm
// of a sub-layer's output added into the residual stream, and the routing weights of experts that a table assigns
// to token ids.  The attention itself is hybrid.hip's (float32) and diff_attention.hip's (matrix cores); the clamped
// gated activation of the feed-forwards and the biases of products are epilogues of the matrix products (gemm_common.h).  Every size is a run-time
// value; norms, angles and the residual sum are float32 whatever the type of the matrices.
#include "common.h"

#define DISPATCH_T(dt, CALL)                                     \
    do {                                                         \
        if ((dt) == DT_F32) { typedef float T; CALL; }           \
        else if ((dt) == DT_F16) { typedef f16 T; CALL; }        \
        else if ((dt) == DT_BF16) { typedef bf16 T; CALL; }      \
        else return LI_BAD_ARG;                                  \
    } while (0)

// ---------------------------------------------------------------------------
// rows[t][col0 + i] += b[i] for i < n: the bias of a product whose kernel has none.
// ---------------------------------------------------------------------------
__global__ void add_bias_kernel(float* __restrict__ rows, int stride, int col0, const float* __restrict__ b, int n) {
    float* row = rows + (int64_t)blockIdx.x * stride + col0;
    for (int i = blockIdx.y * blockDim.x + threadIdx.x; i < n; i += gridDim.y * blockDim.x) row[i] += b[i];
}

extern "C" int li_add_bias(float* rows, int stride, int col0, const float* b, int n_rows, int n, hipStream_t stream) {
    if (n_rows <= 0 || n <= 0) return LI_OK;
    if (col0 < 0 || col0 + n > stride) return LI_BAD_ARG;
    dim3 grid(n_rows, n_rows >= 1024 ? 1 : (n + 1023) / 1024);
    add_bias_kernel<<<grid, 256, 0, stream>>>(rows, stride, col0, b, n);
    LI_CHECK_LAUNCH();
    return LI_OK;
}

// x[i] *= s for n float32 numbers (a model's logits times a constant).
__global__ void scale_values_kernel(float* __restrict__ x, int64_t n, float s) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) x[i] *= s;
}

extern "C" int li_scale_values(float* x, int64_t n, float s, hipStream_t stream) {
    if (n <= 0) return LI_OK;
    const int blocks = (int)((n + 255) / 256 < 4096 ? (n + 255) / 256 : 4096);
    scale_values_kernel<<<blocks, 256, 0, stream>>>(x, n, s);
    LI_CHECK_LAUNCH();
    return LI_OK;
}

// ---------------------------------------------------------------------------
// From float32 rows that hold a token's q heads [H, d] from column q_col, its k heads [G, d] from k_col and its
// values [G, dv] from v_col (v_col may be k_col: the values are the keys as projected): q and k are turned by the
// token's position p in their first `rot` dimensions, dimension i paired with i + rot / 2,
//   (u, v) -> (u cos a - v sin a, v cos a + u sin a),  a = p * inv_freq[i]   (float32 angles, accurate sin and cos),
// the values are not.  q goes to q_out [T, H, DP] in the cache's type (DP = d rounded up to 16, zeros behind d),
// k (padded likewise) and v into the page of position p in matrix-operand order (common.h; one map of keys).
// G_store 0: only q (a layer that reads another layer's keys and values).
// `conv_w` not null (float32 [channels, taps]): what is read of the rows is first convolved over time, channel by
// channel (column c of the rows is channel c; the last tap is the token's own), y_t = sum_j w[c][j] u_(t - taps + 1 + j):
// inputs before the first token that a sequence brings to this step come from `hist` [slots, taps - 1, channels] (the
// last inputs of the steps before, oldest first; before position 0 they are zero), which this kernel only reads.
// ---------------------------------------------------------------------------
struct StorePages {
    void* k;
    void* v;
    int64_t page_stride;
    const int* page_table;
    int max_pages;
};

#define ROT_MAX_PAIRS 256

template <class T>
__global__ void rot_store_kernel(const float* __restrict__ rows, int stride, int q_col, int k_col, int v_col,
                                 const float* __restrict__ inv_freq, int rot, const int* __restrict__ pos,
                                 const int* __restrict__ tok_slot, T* __restrict__ q_out, StorePages pg, int H, int G,
                                 int d, int dv, const float* __restrict__ conv_w, int taps, const float* __restrict__ hist,
                                 int channels) {
    __shared__ float cs[2 * ROT_MAX_PAIRS];               // cos and sin of the token's angles, one pair of them a pair of dimensions
    const int t = blockIdx.x, p = pos[t], DP = round_up(d, 16), half = rot >> 1;
    for (int j = threadIdx.x; j < half; j += blockDim.x) sincosf((float)p * inv_freq[j], &cs[2 * j + 1], &cs[2 * j]);
    if (half) __syncthreads();
    const float* row = rows + (int64_t)t * stride;
    const int slot = tok_slot[t];
    // how many tokens before this one its sequence has in this step (at most taps - 1 matter)
    int inside = 0;
    if (conv_w) while (inside < taps - 1 && t - inside - 1 >= 0 && tok_slot[t - inside - 1] == slot) ++inside;
    const float* h = conv_w ? hist + (int64_t)slot * (taps - 1) * channels : nullptr;
    auto value = [&](int c) {                             // column c of this token's row, convolved where asked
        if (!conv_w) return row[c];
        float acc = 0.f;
        for (int back = 0; back < taps; ++back) {
            float u = 0.f;
            if (back <= inside) u = row[c - (int64_t)back * stride];
            else if (p - back >= 0) u = h[(int64_t)(taps - 1 - (back - inside)) * channels + c];
            acc += conv_w[(int64_t)c * taps + (taps - 1 - back)] * u;
        }
        return acc;
    };
    T* kp = nullptr;
    T* vp = nullptr;
    const int off = p % PAGE;
    if (G > 0) {
        const int page = pg.page_table[(int64_t)slot * pg.max_pages + p / PAGE];
        kp = (T*)pg.k + (int64_t)page * pg.page_stride;
        vp = (T*)pg.v + (int64_t)page * pg.page_stride;
    }
    const int n_qk = (H + G) * DP, total = n_qk + G * dv;
    for (int e = blockIdx.y * blockDim.x + threadIdx.x; e < total; e += gridDim.y * blockDim.x) {
        if (e < n_qk) {
            const int u = e / DP, i = e - u * DP;
            const bool is_q = u < H;
            const int src = is_q ? q_col + u * d : k_col + (u - H) * d;
            float val = 0.f;
            if (i < d) {
                val = value(src + i);
                if (i < rot) {
                    const int j = i < half ? i : i - half;
                    const float c_ = cs[2 * j], s_ = cs[2 * j + 1];
                    val = i < half ? val * c_ - value(src + i + half) * s_ : val * c_ + value(src + i - half) * s_;
                }
            }
            if (is_q) q_out[((int64_t)t * H + u) * DP + i] = from_f32<T>(val);
            else kp[(int64_t)(u - H) * k_head_elems(DP) + k_offset(off, i, DP)] = from_f32<T>(val);
        } else {
            const int r = e - n_qk, g = r / dv, j = r - g * dv;
            vp[(int64_t)g * v_head_elems(dv) + v_offset(off, j, dv)] = from_f32<T>(value(v_col + r));
        }
    }
}

extern "C" int li_rot_store(const float* rows, int stride, int q_col, int k_col, int v_col, const float* inv_freq, int rot,
                            const int* pos, const int* tok_slot, void* q_out, void* k_pages, void* v_pages,
                            int64_t page_stride, const int* page_table, int max_pages, int dt, int n, int H, int G_store,
                            int d, int dv, const float* conv_w, int taps, const float* hist, int channels,
                            hipStream_t stream) {
    if (n <= 0) return LI_OK;
    if (H <= 0 || G_store < 0 || d <= 0 || dv <= 0 || rot < 0 || rot > d || (rot & 1) || (rot && !inv_freq)) return LI_BAD_ARG;
    if (rot > 2 * ROT_MAX_PAIRS) return LI_UNSUPPORTED;
    if (q_col < 0 || q_col + H * d > stride) return LI_BAD_ARG;
    if (G_store && (k_col < 0 || v_col < 0 || k_col + G_store * d > stride || v_col + G_store * dv > stride)) return LI_BAD_ARG;
    if (conv_w) {
        // every column that is read is a channel of the convolution
        const int last = G_store ? (k_col + G_store * d > v_col + G_store * dv ? k_col + G_store * d : v_col + G_store * dv) : 0;
        if (taps < 1 || taps > 16 || (taps > 1 && !hist) || channels > stride || q_col + H * d > channels || last > channels)
            return LI_BAD_ARG;
    }
    StorePages pg{k_pages, v_pages, page_stride, page_table, max_pages};
    const int total = (H + G_store) * round_up(d, 16) + G_store * dv;
    dim3 grid(n, n >= 512 ? 1 : (total + 255) / 256);
    DISPATCH_T(dt, (rot_store_kernel<T><<<grid, 256, 0, stream>>>(rows, stride, q_col, k_col, v_col, inv_freq, rot, pos, tok_slot,
                                                              (T*)q_out, pg, H, G_store, d, dv, conv_w, taps, hist, channels)));
    LI_CHECK_LAUNCH();
    return LI_OK;
}

// ---------------------------------------------------------------------------
// x[t] += (y[t] + b) / sqrt(mean((y[t] + b)^2) + eps) * w: the norm on a sub-layer's output and the residual sum in
// one pass over the row (b may be null).  `next_w` not null: the norm that reads the finished row next is taken too,
// next[t] = x[t] / sqrt(mean(x[t]^2) + next_eps) * next_w in type TN, while the row is still in registers.
// One workgroup a row; the row stays in registers up to 8,192 elements (a multiple of 4), else it is read again.
// ---------------------------------------------------------------------------
#define RA_THREADS 256
#define RA_KEEP 8          // 4 elements x RA_KEEP x RA_THREADS = 8,192 elements kept

// EARLY (the few rows of a decode step): everything the row needs is asked for at once (y, the bias, x and the weight), so
// that a row waits for memory once and not once a phase; many rows fill the chip anyway and do better with fewer registers.
template <class TN, bool EARLY>
__global__ __launch_bounds__(RA_THREADS) void rmsnorm_add_kernel(float* __restrict__ x, const float* __restrict__ y,
                                                                 const float* __restrict__ b, const float* __restrict__ w,
                                                                 float eps, int width, const float* __restrict__ next_w,
                                                                 float next_eps, TN* __restrict__ next) {
    __shared__ float scratch[16];
    const int64_t row = blockIdx.x;
    const float* yr = y + row * width;
    float* xr = x + row * width;
    TN* nr = next + row * width;
    float ss = 0.f, s2 = 0.f;
    if ((width & 3) == 0 && width <= 4 * RA_KEEP * RA_THREADS) {
        f32x4 keep[RA_KEEP], xs[RA_KEEP], ws[RA_KEEP];
        const int quads = width >> 2;
#pragma unroll
        for (int c = 0; c < RA_KEEP; ++c) {
            const int i = threadIdx.x + c * RA_THREADS;
            if (i < quads) {
                f32x4 v = *(const f32x4*)(yr + 4 * i);
                if (EARLY) {
                    xs[c] = *(const f32x4*)(xr + 4 * i);
                    ws[c] = *(const f32x4*)(w + 4 * i);
                }
                if (b) { const f32x4 bb = *(const f32x4*)(b + 4 * i); v[0] += bb[0]; v[1] += bb[1]; v[2] += bb[2]; v[3] += bb[3]; }
                keep[c] = v;
                ss += v[0] * v[0] + v[1] * v[1] + v[2] * v[2] + v[3] * v[3];
            }
        }
        const float r = 1.f / sqrtf(block_sum(ss, scratch) / (float)width + eps);
#pragma unroll
        for (int c = 0; c < RA_KEEP; ++c) {
            const int i = threadIdx.x + c * RA_THREADS;
            if (i < quads) {
                if (!EARLY) {
                    xs[c] = *(const f32x4*)(xr + 4 * i);
                    ws[c] = *(const f32x4*)(w + 4 * i);
                }
                f32x4 o = xs[c];
                o[0] += keep[c][0] * r * ws[c][0]; o[1] += keep[c][1] * r * ws[c][1];
                o[2] += keep[c][2] * r * ws[c][2]; o[3] += keep[c][3] * r * ws[c][3];
                *(f32x4*)(xr + 4 * i) = o;
                keep[c] = o;
                s2 += o[0] * o[0] + o[1] * o[1] + o[2] * o[2] + o[3] * o[3];
                if (next_w) ws[c] = *(const f32x4*)(next_w + 4 * i);
            }
        }
        if (!next_w) return;
        const float r2 = 1.f / sqrtf(block_sum(s2, scratch) / (float)width + next_eps);
#pragma unroll
        for (int c = 0; c < RA_KEEP; ++c) {
            const int i = threadIdx.x + c * RA_THREADS;
            if (i < quads) {
#pragma unroll
                for (int k = 0; k < 4; ++k) nr[4 * i + k] = from_f32<TN>(keep[c][k] * r2 * ws[c][k]);
            }
        }
        return;
    }
    for (int i = threadIdx.x; i < width; i += RA_THREADS) { const float v = yr[i] + (b ? b[i] : 0.f); ss += v * v; }
    const float r = 1.f / sqrtf(block_sum(ss, scratch) / (float)width + eps);
    for (int i = threadIdx.x; i < width; i += RA_THREADS) {
        const float o = xr[i] + (yr[i] + (b ? b[i] : 0.f)) * r * w[i];
        xr[i] = o;
        s2 += o * o;
    }
    if (!next_w) return;
    const float r2 = 1.f / sqrtf(block_sum(s2, scratch) / (float)width + next_eps);
    for (int i = threadIdx.x; i < width; i += RA_THREADS) nr[i] = from_f32<TN>(xr[i] * r2 * next_w[i]);   // (this thread's own writes)
}

extern "C" int li_rmsnorm_add(float* x, const float* y, const float* b, const float* w, float eps, int n_rows, int width,
                              const float* next_w, float next_eps, void* next, int next_dt, hipStream_t stream) {
    if (n_rows <= 0) return LI_OK;
    if (width <= 0 || !x || !y || !w || (next_w && !next)) return LI_BAD_ARG;
    if (!next_w) next_dt = DT_F32;
    if (n_rows <= 64)
        DISPATCH_T(next_dt, (rmsnorm_add_kernel<T, true><<<n_rows, RA_THREADS, 0, stream>>>(x, y, b, w, eps, width, next_w, next_eps, (T*)next)));
    else
        DISPATCH_T(next_dt, (rmsnorm_add_kernel<T, false><<<n_rows, RA_THREADS, 0, stream>>>(x, y, b, w, eps, width, next_w, next_eps, (T*)next)));
    LI_CHECK_LAUNCH();
    return LI_OK;
}

// ---------------------------------------------------------------------------
// Experts by table: row table[token] [top] names the experts of a token (they differ), each with weight 1 / top.
// weights [T, wcols] gets the dense row (0 where not named); with has_gate 1 its last column is the sigmoid of the
// token's gate logit (float32 [T]) for an expert that every token uses, with has_gate 2 it is 1.
// ---------------------------------------------------------------------------
__global__ void table_route_kernel(const int* __restrict__ tokens, const int* __restrict__ table, int top, int n_experts,
                                   const float* __restrict__ gate_logits, int has_gate, float* __restrict__ weights) {
    const int64_t t = blockIdx.x;
    const int wcols = n_experts + (has_gate ? 1 : 0);
    float* w = weights + t * wcols;
    const int* mine = table + (int64_t)tokens[t] * top;
    for (int e = threadIdx.x; e < n_experts; e += blockDim.x) {
        float v = 0.f;
        for (int k = 0; k < top; ++k) if (mine[k] == e) v = 1.f / (float)top;
        w[e] = v;
    }
    if (has_gate && threadIdx.x == 0) w[n_experts] = has_gate == 2 ? 1.f : 1.f / (1.f + expf(-gate_logits[t]));
}

extern "C" int li_table_route(const int* tokens, const int* table, int top, int n_experts, const float* gate_logits,
                              int has_gate, float* weights, int n, hipStream_t stream) {
    if (n <= 0) return LI_OK;
    if (top < 1 || n_experts < 1 || top > n_experts || has_gate < 0 || has_gate > 2 || (has_gate == 1 && !gate_logits)) return LI_BAD_ARG;
    table_route_kernel<<<n, 64, 0, stream>>>(tokens, table, top, n_experts, gate_logits, has_gate, weights);
    LI_CHECK_LAUNCH();
    return LI_OK;
}
