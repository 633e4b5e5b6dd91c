// Differential attention over blocks of positions on the matrix cores, for one pair of sizes: MAP_DIM (a map's
// key size rounded up to 16) and VALUE_DIM (the value size rounded up to 32), both compile-time.  16-bit keys,
// values and queries; scores, weights, sums and the norm of the output float32.
//
// One wave per (tile of up to 32 consecutive tokens of a sequence, query head); a decode step's tiles hold one
// token, and four waves then take every fourth 32 keys each and merge their running maxima, sums and outputs
// through LDS in wave order.  A token at position p sees the keys lo .. p, lo = p - p % block (block 0: 0; window w: at least p - w + 1).
// Keys are walked 32 at a time.  Per map m:  S^T = K_m Q_m^T  (rows keys, columns queries; operand A straight from
// the page, which holds keys in operand order), online softmax down the rows (a query's 32 scores lie in the 16
// accumulator elements of two lanes), then O_m^T += V^T P_m^T with the accumulators' own order of the keys, in which the
// page holds the values.  A weight enters the second product as the sum of two 16-bit numbers (its rounding and the
// rounding of the remainder), so that the product sees 16 bits of it.  At the end o = O_1 / l_1 - lambda O_2 / l_2,
// divided by its root mean square over the value size and multiplied by out_scale.  `sink` not null: every map's sum
// of weights also counts exp(sink[head]), a score with no key and no value that is not scaled.  `slopes` not null:
// the score of the key at position j loses slopes[head] * (p - j), the sink nothing.  `gate` not null: a head's output
// is multiplied by the sigmoid of gate[token][gate_col + head] (float32 rows of gate_stride numbers).
#include "common.h"

#ifndef MAP_DIM
#error "compile with -DMAP_DIM=<multiple of 16> -DVALUE_DIM=<multiple of 32>"
#endif
static_assert(MAP_DIM % 16 == 0 && MAP_DIM >= 16 && MAP_DIM <= 256, "a map's key size: a multiple of 16 up to 256");
static_assert(VALUE_DIM % 32 == 0 && VALUE_DIM >= 32 && VALUE_DIM <= 256, "value size: a multiple of 32 up to 256");

struct MapPages {
    const void* k;
    const void* v;
    int64_t page_stride;
    const int* page_table;
    int max_pages;
};

// HC (decode steps, several query heads on a key/value head): the 32 columns of a tile are 32 query heads of one
// key/value head for one token instead of 32 tokens of one head, so the keys and values of a token are fetched once for
// all of them; the four waves of the workgroup share the token's keys and merge all 32 columns' states.
// One map needs no second half of a weight (nothing is subtracted afterwards): a weight enters the second product
// rounded once, as in the softmax attention of the other decoders.
template <class T, int MAPS, bool PROMPT, bool HC>
__global__ __launch_bounds__(256) void diff_attn_mfma_kernel(
    const T* __restrict__ q, T* __restrict__ out, MapPages pg, const int* __restrict__ pos,
    const int* __restrict__ tok_slot, const int* __restrict__ tile_t0, const int* __restrict__ tile_n, int H, int G,
    int dv, float scale, int block, int window, float lambda, float out_eps, float out_scale, int split,
    const float* __restrict__ sink, float* __restrict__ shares_out, const float* __restrict__ slopes,
    const float* __restrict__ gate, int gate_stride, int gate_col) {
    typedef typename Vec<T>::v8 v8;
    constexpr int D16 = MAP_DIM / 16, KW = MAPS * MAP_DIM, DVB = VALUE_DIM / 32;
    extern __shared__ float lds[];
    // Workgroups go to the 8 XCDs in turn (workgroup L to XCD L % 8) and every XCD has an L2 of its own: the grid is
    // renumbered so that an XCD works on one stretch of it, (head group, tile) with the tile running fastest, and so
    // on the keys and values of as few KV heads as can be (one, where there are eight) instead of all of them
    const int L = blockIdx.x + gridDim.x * blockIdx.y, total = gridDim.x * gridDim.y;
    const int xcd = L & 7, per = total >> 3, rem = total & 7;
    const int id = PROMPT ? xcd * per + min(xcd, rem) + (L >> 3) : L;       // (a decode step's few workgroups stay as they are)
    const int item = id % gridDim.x, group = id / gridDim.x;
    const int lane = threadIdx.x & 63, col = lane & 31, half = lane >> 5;
    const int wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
    // the waves of a workgroup: the query heads of one KV head on the same tile (they fetch the same keys and
    // values, which then come from the CU's cache), or, `split`, shares of the keys of a tile of one token
    const int per_kv = H / G, hc_tiles = (per_kv + 31) / 32;
    // HC: this lane's head, the column's; h itself may lie beyond the key/value head's last (such a column has no query)
    const int h = HC ? (group / hc_tiles) * per_kv + (group % hc_tiles) * 32 + col : (split ? group : group * nw + wave);
    const bool head_ok = !HC || (group % hc_tiles) * 32 + col < per_kv;
    const int hq = head_ok ? h : (group / hc_tiles) * per_kv;          // a head that exists, for addresses
    // HC: the workgroups along the grid's third dimension share a token's keys as the waves of one do
    const int kwave = split ? (HC ? blockIdx.z * nw + wave : wave) : 0, kstep = split ? (HC ? nw * gridDim.z : nw) : 1;
    const int g = HC ? group / hc_tiles : h / per_kv;
    constexpr bool SPLIT_W = MAPS == 2;
    // an item of a prompt is two tiles, one that sees many keys and one that sees few (the host pairs them), so that
    // every wave has about the same work; a decode step's item is its one token
    constexpr int parts = PROMPT ? 2 : 1;
    for (int part = 0; part < parts; ++part) {
    const int t0 = PROMPT ? tile_t0[parts * item + part] : item, n = PROMPT ? tile_n[parts * item + part] : 1;
    if (n <= 0) continue;
    const int p0 = pos[t0];                            // the tile's tokens stand at p0, p0 + 1, ...
    const bool has_query = HC ? head_ok : col < n;
    const int pq = p0 + min(col, n - 1);
    int lo_q = block > 0 ? pq - pq % block : 0;
    if (window > 0) lo_q = max(lo_q, pq - window + 1);
    int lo_tile = block > 0 ? p0 - p0 % block : 0;     // the first token's: the smallest
    if (window > 0) lo_tile = max(lo_tile, p0 - window + 1);
    const int p_last = p0 + n - 1;
    int lo_last = block > 0 ? p_last - p_last % block : 0;       // the last token's: the largest
    if (window > 0) lo_last = max(lo_last, p_last - window + 1);
    const bool whole_tile = n == 32;
    const float scale2 = scale * 1.4426950408889634f;
    const float slope2 = slopes ? slopes[hq] * 1.4426950408889634f : 0.f;      // what a score loses for every position of distance
    const int* table = pg.page_table + (int64_t)tok_slot[t0] * pg.max_pages;

    v8 qf[MAPS][D16];
    {
        const T* qrow = q + ((int64_t)(t0 + (HC ? 0 : min(col, n - 1))) * H + hq) * KW;
#pragma unroll
        for (int a = 0; a < MAPS; ++a)
#pragma unroll
            for (int s = 0; s < D16; ++s) qf[a][s] = *(const v8*)(qrow + a * MAP_DIM + s * 16 + half * 8);
    }
    f32x16 o[MAPS][DVB];
    float m[MAPS], l[MAPS];
#pragma unroll
    for (int a = 0; a < MAPS; ++a) {
        m[a] = -INFINITY; l[a] = 0.f;
#pragma unroll
        for (int b = 0; b < DVB; ++b)
#pragma unroll
            for (int r = 0; r < 16; ++r) o[a][b][r] = 0.f;
    }

    // the fragments of the 32 keys after the ones at work are fetched before the work begins
    v8 kn[MAPS][D16], vn[DVB][2];
    auto fetch = [&](int kt) {
        const int page = table[kt >> 1], tb = kt & 1;                      // two blocks of 32 keys a page
        const T* kh = (const T*)pg.k + (int64_t)page * pg.page_stride + g * k_head_elems(KW);
        const T* vh = (const T*)pg.v + (int64_t)page * pg.page_stride + g * v_head_elems(VALUE_DIM);
#pragma unroll
        for (int a = 0; a < MAPS; ++a)
#pragma unroll
            for (int s = 0; s < D16; ++s) kn[a][s] = *(const v8*)(kh + ((int64_t)(tb * (KW / 16) + a * D16 + s) * 64 + lane) * 8);
#pragma unroll
        for (int b = 0; b < DVB; ++b)
#pragma unroll
            for (int u = 0; u < 2; ++u) vn[b][u] = *(const v8*)(vh + ((int64_t)(b * (PAGE / 16) + tb * 2 + u) * 64 + lane) * 8);
    };
    const int kt_last = p_last / 32, kt_first = lo_tile / 32 + kwave;
    if (kt_first <= kt_last) fetch(kt_first);
    for (int kt = kt_first; kt <= kt_last; kt += kstep) {
        v8 kf[MAPS][D16], vf[DVB][2];
#pragma unroll
        for (int a = 0; a < MAPS; ++a)
#pragma unroll
            for (int s = 0; s < D16; ++s) kf[a][s] = kn[a][s];
#pragma unroll
        for (int b = 0; b < DVB; ++b)
#pragma unroll
            for (int u = 0; u < 2; ++u) vf[b][u] = vn[b][u];
        if (kt + kstep <= kt_last) fetch(kt + kstep);
        v8 phi[MAPS][2], plo[MAPS][2];
#pragma unroll
        for (int a = 0; a < MAPS; ++a) {
            f32x16 acc;
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[r] = 0.f;
#pragma unroll
            for (int s = 0; s < D16; ++s) {
                acc = mfma32(kf[a][s], qf[a][s], acc);
            }
            // scores in units of log 2, so that a weight is one hardware 2^x; 32 keys that every query of a whole tile
            // sees need no mask
            float tmax = -INFINITY;
            if (whole_tile && kt * 32 >= lo_last && kt * 32 + 31 <= p0) {
                if (slopes) {
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const int key = kt * 32 + 8 * (r >> 2) + 4 * half + (r & 3);
                        acc[r] = acc[r] * scale2 - slope2 * (float)(pq - key);
                        tmax = fmaxf(tmax, acc[r]);
                    }
                } else {
#pragma unroll
                    for (int r = 0; r < 16; ++r) { acc[r] *= scale2; tmax = fmaxf(tmax, acc[r]); }
                }
            } else {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int key = kt * 32 + 8 * (r >> 2) + 4 * half + (r & 3);
                    const bool seen = has_query && key >= lo_q && key <= pq;
                    acc[r] = seen ? acc[r] * scale2 - slope2 * (float)(pq - key) : -INFINITY;
                    tmax = fmaxf(tmax, acc[r]);
                }
            }
            tmax = fmaxf(tmax, __shfl_xor(tmax, 32, WAVE));
            const float mn = fmaxf(m[a], tmax);
            float f = 1.f, sum = 0.f;
            float pr[16];
            if (mn == -INFINITY) {                                         // nothing seen yet by this query
#pragma unroll
                for (int r = 0; r < 16; ++r) pr[r] = 0.f;
            } else {
                f = __builtin_amdgcn_exp2f(m[a] - mn);                     // 0 while m is still -inf
#pragma unroll
                for (int r = 0; r < 16; ++r) { pr[r] = __builtin_amdgcn_exp2f(acc[r] - mn); sum += pr[r]; }
            }
            sum += __shfl_xor(sum, 32, WAVE);
            l[a] = l[a] * f + sum;
            m[a] = mn;
            if (f != 1.f) {
#pragma unroll
                for (int b = 0; b < DVB; ++b)
#pragma unroll
                    for (int r = 0; r < 16; ++r) o[a][b][r] *= f;
            }
#pragma unroll
            for (int u = 0; u < 2; ++u)
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const T hi = from_f32<T>(pr[8 * u + i]);
                    phi[a][u][i] = hi;
                    if (SPLIT_W) plo[a][u][i] = from_f32<T>(pr[8 * u + i] - to_f32(hi));
                }
        }
#pragma unroll
        for (int b = 0; b < DVB; ++b)
#pragma unroll
            for (int u = 0; u < 2; ++u) {
#pragma unroll
                for (int a = 0; a < MAPS; ++a) {
                    o[a][b] = mfma32(vf[b][u], phi[a][u], o[a][b]);
                    if (SPLIT_W) o[a][b] = mfma32(vf[b][u], plo[a][u], o[a][b]);
                }
            }
    }
    if (split && nw > 1) {
        // a tile of one token whose keys the waves have shared: wave 0 adds up their states in wave order
        constexpr int W = 2 + VALUE_DIM;
        if (HC || col == 0) {
#pragma unroll
            for (int a = 0; a < MAPS; ++a) {
                float* mine = lds + ((wave * MAPS + a) * (HC ? 32 : 1) + (HC ? col : 0)) * W;
                if (half == 0) { mine[0] = m[a]; mine[1] = l[a]; }
#pragma unroll
                for (int b = 0; b < DVB; ++b)
#pragma unroll
                    for (int r = 0; r < 16; ++r) mine[2 + b * 32 + 8 * (r >> 2) + 4 * half + (r & 3)] = o[a][b][r];
            }
        }
        __syncthreads();
        if (wave != 0) return;
        if (HC || col == 0) {
            const int cs = HC ? 32 : 1, c0 = HC ? col : 0;
#pragma unroll
            for (int a = 0; a < MAPS; ++a) {
                float M = -INFINITY;
                for (int w = 0; w < nw; ++w) M = fmaxf(M, lds[((w * MAPS + a) * cs + c0) * W]);
                float L = 0.f;
#pragma unroll
                for (int b = 0; b < DVB; ++b)
#pragma unroll
                    for (int r = 0; r < 16; ++r) o[a][b][r] = 0.f;
                for (int w = 0; w < nw; ++w) {
                    const float* theirs = lds + ((w * MAPS + a) * cs + c0) * W;
                    if (theirs[0] == -INFINITY) continue;
                    const float f = __builtin_amdgcn_exp2f(theirs[0] - M);
                    L += theirs[1] * f;
#pragma unroll
                    for (int b = 0; b < DVB; ++b)
#pragma unroll
                        for (int r = 0; r < 16; ++r) o[a][b][r] += theirs[2 + b * 32 + 8 * (r >> 2) + 4 * half + (r & 3)] * f;
                }
                m[a] = M; l[a] = L;
            }
        }
    }
    if (HC && gridDim.z > 1) {
        // the keys were shared among workgroups: this one's state goes to `shares_out` [token, head, share, map, 2 + VALUE_DIM]
        // and diff_attn_merge_kernel finishes
        constexpr int W = 2 + VALUE_DIM;
        if (has_query) {
#pragma unroll
            for (int a = 0; a < MAPS; ++a) {
                float* mine = shares_out + ((((int64_t)t0 * H + hq) * gridDim.z + blockIdx.z) * MAPS + a) * W;
                if (half == 0) { mine[0] = m[a]; mine[1] = l[a]; }
#pragma unroll
                for (int b = 0; b < DVB; ++b)
#pragma unroll
                    for (int r = 0; r < 16; ++r) mine[2 + b * 32 + 8 * (r >> 2) + 4 * half + (r & 3)] = o[a][b][r];
            }
        }
        return;
    }
    if (sink) {
        // the sink joins every map's sum as one more weight, exp(sink - maximum), with nothing to add to the output
        const float s2 = sink[hq] * 1.4426950408889634f;
#pragma unroll
        for (int a = 0; a < MAPS; ++a) {
            const float M = fmaxf(m[a], s2), f = __builtin_amdgcn_exp2f(m[a] - M);
            l[a] = l[a] * f + __builtin_amdgcn_exp2f(s2 - M);
#pragma unroll
            for (int b = 0; b < DVB; ++b)
#pragma unroll
                for (int r = 0; r < 16; ++r) o[a][b][r] *= f;
        }
    }
    // o = O_1 / l_1 - lambda O_2 / l_2 for this lane's query; its values lie in this lane and in lane ^ 32
    float ss = 0.f;
#pragma unroll
    for (int b = 0; b < DVB; ++b)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int dim = b * 32 + 8 * (r >> 2) + 4 * half + (r & 3);
            float v = o[0][b][r] / l[0];
            if (MAPS == 2) v -= lambda * (o[MAPS - 1][b][r] / l[MAPS - 1]);
            v = dim < dv ? v : 0.f;
            o[0][b][r] = v;
            ss += v * v;
        }
    ss += __shfl_xor(ss, 32, WAVE);
    float rr = out_eps >= 0.f ? out_scale / sqrtf(ss / (float)dv + out_eps) : out_scale;
    if (gate && has_query)             // one number a (token, head)
        rr *= 1.f / (1.f + expf(-gate[(int64_t)(t0 + (HC ? 0 : col)) * gate_stride + gate_col + hq]));
    if (has_query) {
        T* orow = out + ((int64_t)(t0 + (HC ? 0 : col)) * H + hq) * dv;
#pragma unroll
        for (int b = 0; b < DVB; ++b)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int dim = b * 32 + 8 * (r >> 2) + 4 * half + (r & 3);
                if (dim < dv) orow[dim] = from_f32<T>(o[0][b][r] * rr);
            }
    }
    }      // the item's tiles
}

// The states of the workgroups that shared a token's keys (`part` [token, head, shares, map, 2 + VALUE_DIM]: maximum in
// units of log 2, sum, output) added up in the order of the shares, then the sink, the difference of the maps and the
// norm as above: one wave per (token, head).
template <class T, int MAPS>
__global__ __launch_bounds__(64) void diff_attn_merge_kernel(const float* __restrict__ part, T* __restrict__ out, int H,
                                                             int S, int dv, float lambda, float out_eps, float out_scale,
                                                             const float* __restrict__ sink, const float* __restrict__ gate,
                                                             int gate_stride, int gate_col) {
    constexpr int W = 2 + VALUE_DIM, NV = (VALUE_DIM + 63) / 64;
    const int64_t unit = blockIdx.x;
    const int h = (int)(unit % H), lane = threadIdx.x;
    float val[MAPS][NV];
#pragma unroll
    for (int a = 0; a < MAPS; ++a) {
        const float* p = part + (unit * S * MAPS + a) * W;
        // lane s fetches share s's maximum and sum (S is at most 64), so no load waits for another
        const float ms = lane < S ? p[(int64_t)lane * MAPS * W] : -INFINITY, ls = lane < S ? p[(int64_t)lane * MAPS * W + 1] : 0.f;
        const float s2 = sink ? sink[h] * 1.4426950408889634f : -INFINITY;
        const float M = fmaxf(wave_max(ms), s2);
        const float fs = ms == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(ms - M);
        const float L = wave_sum(ls * fs) + (sink ? __builtin_amdgcn_exp2f(s2 - M) : 0.f);
        float O[NV];
#pragma unroll
        for (int v = 0; v < NV; ++v) O[v] = 0.f;
#pragma unroll 4
        for (int s = 0; s < S; ++s) {
            const float f = __shfl(fs, s, WAVE);
            const float* q = p + (int64_t)s * MAPS * W + 2;
#pragma unroll
            for (int v = 0; v < NV; ++v) if (v * 64 + lane < VALUE_DIM) O[v] += q[v * 64 + lane] * f;
        }
#pragma unroll
        for (int v = 0; v < NV; ++v) val[a][v] = O[v] / L;
    }
    float ss = 0.f, res[NV];
#pragma unroll
    for (int v = 0; v < NV; ++v) {
        float x = val[0][v];
        if (MAPS == 2) x -= lambda * val[MAPS - 1][v];
        res[v] = v * 64 + lane < dv ? x : 0.f;
        ss += res[v] * res[v];
    }
    ss = wave_sum(ss);
    float rr = out_eps >= 0.f ? out_scale / sqrtf(ss / (float)dv + out_eps) : out_scale;
    if (gate) rr *= 1.f / (1.f + expf(-gate[(unit / H) * gate_stride + gate_col + h]));
#pragma unroll
    for (int v = 0; v < NV; ++v) if (v * 64 + lane < dv) out[unit * dv + v * 64 + lane] = from_f32<T>(res[v] * rr);
}

extern "C" int li_diffattn_map_dim() { return MAP_DIM; }
extern "C" int li_diffattn_value_dim() { return VALUE_DIM; }

// q [T, H, maps * MAP_DIM] and out [T, H * dv] of type dt (float16 or bfloat16), as are the pages.  tile_t0 / tile_n
// (device, may be null: every token an item of its own): first row and number of rows (0 .. 32) of the two tiles of
// every one of the n_tiles items (2 n_tiles entries each; a tile of no rows is skipped).
extern "C" int li_diffattn(const void* q, void* out, int dt, const void* k_pages, const void* v_pages, int64_t page_stride,
                           const int* page_table, int max_pages, const int* pos, const int* tok_slot, const int* tile_t0,
                           const int* tile_n, int n_tiles, int H, int G, int maps, int dv, float scale, int block, int window,
                           float lambda, float out_eps, float out_scale, const float* sink, int key_shares, float* part,
                           const float* slopes, const float* gate, int gate_stride, int gate_col, hipStream_t stream) {
    if (n_tiles <= 0) return LI_OK;
    if (gate && (gate_col < 0 || gate_col + H > gate_stride)) return LI_BAD_ARG;
    if (H <= 0 || G <= 0 || H % G || dv <= 0 || dv > VALUE_DIM || block < 0 || window < 0) return LI_BAD_ARG;
    if (maps < 1 || maps > 2 || (dt != DT_F16 && dt != DT_BF16)) return LI_UNSUPPORTED;
    if ((tile_t0 == nullptr) != (tile_n == nullptr)) return LI_BAD_ARG;
    MapPages pg{k_pages, v_pages, page_stride, page_table, max_pages};
    // tiles of one token (a decode step): four waves share a token's keys and merge through LDS; else the waves of
    // a workgroup are query heads of one KV head (4, 2 or 1 of them)
    const int split = tile_t0 ? 0 : 1, per_kv = H / G;
    const int heads = split ? 1 : (per_kv % 4 == 0 ? 4 : (per_kv % 2 == 0 ? 2 : 1));
    // a decode step with four or more query heads on a key/value head: the heads are a tile's columns
    // (where the 32 columns' states of four waves fit into the 160 KiB of LDS: two maps of wide values do not)
    const bool hc = split && per_kv >= 4 && (size_t)4 * maps * 32 * (2 + VALUE_DIM) * sizeof(float) <= 150 * 1024;
    // (then `key_shares` workgroups share a token's keys and leave their states in `part`, float32 [tokens, H, shares,
    // maps, 2 + VALUE_DIM], for a second kernel)
    const int shares = hc && key_shares > 1 && part ? key_shares : 1;
    dim3 grid(n_tiles, hc ? G * ((per_kv + 31) / 32) : H / heads, shares);
    const int threads = split ? 256 : 64 * heads;
    const size_t lds = split ? (size_t)4 * maps * (hc ? 32 : 1) * (2 + VALUE_DIM) * sizeof(float) : 0;
#define GO1(T, M, P, C)                                                                                                              \
    do {                                                                                                                             \
        auto kfn = diff_attn_mfma_kernel<T, M, P, C>;                                                                                \
        if (lds > 48 * 1024 &&                                                                                                       \
            hipFuncSetAttribute((const void*)kfn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)              \
            return LI_HIP_ERROR;                                                                                                     \
        kfn<<<grid, threads, lds, stream>>>((const T*)q, (T*)out, pg, pos, tok_slot, tile_t0, tile_n, H, G, dv, scale, block, window, \
                                            lambda, out_eps, out_scale, split, sink, part, slopes, gate, gate_stride, gate_col);     \
        if (shares > 1)                                                                                                              \
            diff_attn_merge_kernel<T, M><<<n_tiles * H, 64, 0, stream>>>(part, (T*)out, H, shares, dv, lambda, out_eps, out_scale, sink, \
                                                                      gate, gate_stride, gate_col);                                  \
    } while (0)
#define GO(T, M) do { if (hc) GO1(T, M, false, true); else if (split) GO1(T, M, false, false); else GO1(T, M, true, false); } while (0)
    if (dt == DT_F16) { if (maps == 1) GO(f16, 1); else GO(f16, 2); }
    else { if (maps == 1) GO(bf16, 1); else GO(bf16, 2); }
#undef GO
#undef GO1
    LI_CHECK_LAUNCH();
    return LI_OK;
}
