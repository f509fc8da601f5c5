// Gated linear attention: a matrix-valued state per request and head that decays per key channel.
//
//   S_t = diag(a_t) S_(t-1) + k_t v_t^T          S: [key_dim, value_dim], float, one per (slot, head)
//   o_t = scale * S_t^T q_t
//
// One kernel serves whole prompts, portions and single decoded tokens: it loads the state of the
// item's slot, walks over the item's rows in order and stores the state back, so the sum that
// reaches a position is formed in the same order however the tokens were cut into steps.
//
// Work split: the columns of S (value channels) never mix, so a wave takes 16 of them; its four
// 16-lane rows each take a quarter of the key channels, keep their part of S in registers and
// sum their partial dot products with q by row swaps.  Per token a lane does 2 * key_dim / 4
// multiply-adds; the next token's operands are loaded while the current one is computed.
// The state, the decay and every sum are float whatever the storage type of q, k and v.
#include "api.h"
#include "common.h"

namespace st {

__global__ __launch_bounds__(256) void decay_gate_kernel(float* __restrict__ z, int64_t n, float inv_tau) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    const float v = z[i];
    // log sigmoid(v) = min(v, 0) - log(1 + exp(-|v|))
    const float ls = fminf(v, 0.f) - log1pf(expf(-fabsf(v)));
    z[i] = expf(ls * inv_tau);
}

// DQ: key channels a lane holds (a multiple of 4; 4 * DQ >= key_dim).  VEC: rows, heads and
// quarters start at multiples of four elements, so operands are loaded four at a time.
template <typename T, int DQ, bool VEC>
struct GlaOperands {
    float q[DQ], k[DQ], a[DQ], v;

    __device__ inline void load(const T* qp, const T* kp, const float* ap, const T* vp, int d0, int key_dim,
                                bool col_ok) {
        if (VEC) {
#pragma unroll
            for (int i = 0; i < DQ; i += 4) {
                if (d0 + i < key_dim) {                         // key_dim % 4 == 0: all four or none
                    load4(qp + i, q + i);
                    load4(kp + i, k + i);
                    const float4 av = *reinterpret_cast<const float4*>(ap + i);
                    a[i] = av.x; a[i + 1] = av.y; a[i + 2] = av.z; a[i + 3] = av.w;
                } else {
#pragma unroll
                    for (int u = 0; u < 4; ++u) { q[i + u] = 0.f; k[i + u] = 0.f; a[i + u] = 0.f; }
                }
            }
        } else {
#pragma unroll
            for (int i = 0; i < DQ; ++i) {
                const bool ok = d0 + i < key_dim;
                q[i] = ok ? Elem<T>::load(qp + i) : 0.f;
                k[i] = ok ? Elem<T>::load(kp + i) : 0.f;
                a[i] = ok ? ap[i] : 0.f;
            }
        }
        v = col_ok ? Elem<T>::load(vp) : 0.f;
    }

    __device__ static inline void load4(const float* p, float* out) {
        const float4 x = *reinterpret_cast<const float4*>(p);
        out[0] = x.x; out[1] = x.y; out[2] = x.z; out[3] = x.w;
    }
    __device__ static inline void load4(const bf16_t* p, float* out) {
        const uint2 x = *reinterpret_cast<const uint2*>(p);
        out[0] = __uint_as_float(x.x << 16); out[1] = __uint_as_float(x.x & 0xffff0000u);
        out[2] = __uint_as_float(x.y << 16); out[3] = __uint_as_float(x.y & 0xffff0000u);
    }
};

template <typename T, int DQ, bool VEC>
__global__ __launch_bounds__(64) void gla_scan_kernel(
    float* __restrict__ o, const T* __restrict__ q, int64_t q_stride, const T* __restrict__ k, int64_t k_stride,
    const T* __restrict__ v, int64_t v_stride, const float* __restrict__ a, float* __restrict__ state,
    const int* __restrict__ item_len, const int* __restrict__ item_tok_off, const int* __restrict__ item_slot,
    int heads, int key_dim, int value_dim, float scale) {
    const int h = blockIdx.x, item = blockIdx.z;
    const int slot = item_slot[item], n = item_len[item];
    if (slot < 0 || n <= 0) return;                    // a padding item of a batch of fixed size
    const int lane = threadIdx.x, c16 = lane & 15, g = lane >> 4;
    const int col = blockIdx.y * 16 + c16;
    const bool col_ok = col < value_dim;
    const int d0 = g * DQ;
    const int row0 = item_tok_off[item];

    float* s_ptr = state + (((int64_t)slot * heads + h) * key_dim + d0) * value_dim + col;
    float S[DQ];
#pragma unroll
    for (int i = 0; i < DQ; ++i) S[i] = (col_ok && d0 + i < key_dim) ? s_ptr[(int64_t)i * value_dim] : 0.f;

    const T* qp = q + (int64_t)row0 * q_stride + (int64_t)h * key_dim + d0;
    const T* kp = k + (int64_t)row0 * k_stride + (int64_t)h * key_dim + d0;
    const T* vp = v + (int64_t)row0 * v_stride + (int64_t)h * value_dim + (col_ok ? col : 0);
    const float* ap = a + ((int64_t)row0 * heads + h) * key_dim + d0;
    float* op = o + ((int64_t)row0 * heads + h) * value_dim + col;
    const int64_t a_stride = (int64_t)heads * key_dim, o_stride = (int64_t)heads * value_dim;

    GlaOperands<T, DQ, VEC> cur, nxt;
    cur.load(qp, kp, ap, vp, d0, key_dim, col_ok);
    for (int r = 0; r < n; ++r) {
        if (r + 1 < n)
            nxt.load(qp + (r + 1) * q_stride, kp + (r + 1) * k_stride, ap + (r + 1) * a_stride,
                     vp + (r + 1) * v_stride, d0, key_dim, col_ok);
        float acc = 0.f;
#pragma unroll
        for (int i = 0; i < DQ; ++i) {
            S[i] = fmaf(cur.a[i], S[i], cur.k[i] * cur.v);
            acc = fmaf(S[i], cur.q[i], acc);
        }
        acc = rows4_sum(acc);
        if (g == 0 && col_ok) op[(int64_t)r * o_stride] = acc * scale;
        if (r + 1 < n) cur = nxt;
    }
#pragma unroll
    for (int i = 0; i < DQ; ++i)
        if (col_ok && d0 + i < key_dim) s_ptr[(int64_t)i * value_dim] = S[i];
}

// One wave per (token, head): root-mean-square norm over the head's value channels, the gain, and
// the gate silu(g).
template <typename T>
__global__ __launch_bounds__(256) void gated_head_norm_kernel(
    T* __restrict__ out, const float* __restrict__ o, const T* __restrict__ g, int64_t g_stride,
    const float* __restrict__ gain, int num_tokens, int heads, int value_dim, float eps) {
    const int lane = threadIdx.x & 63;
    const int64_t unit = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);      // (token, head)
    if (unit >= (int64_t)num_tokens * heads) return;
    const int64_t t = unit / heads;
    const int h = (int)(unit - t * heads);
    const float* op = o + unit * value_dim;
    const T* gp = g + t * g_stride + (int64_t)h * value_dim;
    T* dst = out + unit * value_dim;
    float ss = 0.f;
    for (int j = lane; j < value_dim; j += 64) { const float x = op[j]; ss = fmaf(x, x, ss); }
    ss = wave_sum(ss);
    const float r = 1.f / sqrtf(ss / (float)value_dim + eps);
    for (int j = lane; j < value_dim; j += 64) {
        const float gv = Elem<T>::load(gp + j);
        const float y = op[j] * r * gain[j] * (gv / (1.f + expf(-gv)));
        Elem<T>::store(dst + j, y);
    }
}

template <typename T, bool VEC>
static int launch_gla(float* o, const void* q, int64_t qs, const void* k, int64_t ks, const void* v, int64_t vs,
                      const float* a, float* state, const int* item_len, const int* item_tok_off,
                      const int* item_slot, int num_items, int heads, int key_dim, int value_dim, float scale,
                      hipStream_t stream) {
    const dim3 grid(heads, (value_dim + 15) / 16, num_items);
    const int dq = (key_dim + 3) / 4;
#define ST_GLA(DQ)                                                                                              \
    gla_scan_kernel<T, DQ, VEC><<<grid, 64, 0, stream>>>(o, (const T*)q, qs, (const T*)k, ks, (const T*)v, vs,  \
        a, state, item_len, item_tok_off, item_slot, heads, key_dim, value_dim, scale)
    if (dq <= 4) ST_GLA(4);
    else if (dq <= 8) ST_GLA(8);
    else if (dq <= 12) ST_GLA(12);
    else if (dq <= 16) ST_GLA(16);
    else if (dq <= 24) ST_GLA(24);
    else if (dq <= 32) ST_GLA(32);
    else if (dq <= 48) ST_GLA(48);
    else ST_GLA(64);
#undef ST_GLA
    ST_LAUNCH_CHECK("gla_scan");
    return 0;
}

}  // namespace st

using namespace st;

extern "C" int st_decay_gate(float* z, int64_t n, float inv_tau, hipStream_t stream) {
    ST_CHECK(n >= 0 && (z || n == 0), "decay_gate: bad operands");
    ST_CHECK(inv_tau > 0.f, "decay_gate: the exponent must be positive");
    if (n == 0) return 0;
    decay_gate_kernel<<<(unsigned)((n + 255) / 256), 256, 0, stream>>>(z, n, inv_tau);
    ST_LAUNCH_CHECK("decay_gate");
    return 0;
}

extern "C" int st_gla_scan(float* o, const void* q, int64_t q_stride, const void* k, int64_t k_stride,
                           const void* v, int64_t v_stride, const float* a, float* state,
                           const int* item_len, const int* item_tok_off, const int* item_slot, int num_items,
                           int heads, int key_dim, int value_dim, float scale, int dtype, hipStream_t stream) {
    ST_CHECK(num_items >= 0 && heads > 0 && key_dim > 0 && value_dim > 0, "gla_scan: bad sizes");
    ST_CHECK(key_dim <= 256, "gla_scan: up to 256 key channels a head, not %d", key_dim);
    ST_CHECK(num_items <= 65535 && (value_dim + 15) / 16 <= 65535, "gla_scan: too many items or value channels");
    ST_CHECK(o && q && k && v && a && state && item_len && item_tok_off && item_slot, "gla_scan: null operand");
    ST_CHECK(dtype == kF32 || dtype == kBF16, "gla_scan: unknown dtype %d", dtype);
    if (num_items == 0) return 0;
    const int es = dtype == kF32 ? 4 : 2;
    const bool vec = key_dim % 4 == 0 && q_stride % 4 == 0 && k_stride % 4 == 0 &&
                     (reinterpret_cast<uintptr_t>(q) % (4 * es)) == 0 && (reinterpret_cast<uintptr_t>(k) % (4 * es)) == 0 &&
                     (reinterpret_cast<uintptr_t>(a) % 16) == 0;
#define ST_ARGS o, q, q_stride, k, k_stride, v, v_stride, a, state, item_len, item_tok_off, item_slot, num_items, \
                heads, key_dim, value_dim, scale, stream
    if (dtype == kF32) return vec ? launch_gla<float, true>(ST_ARGS) : launch_gla<float, false>(ST_ARGS);
    return vec ? launch_gla<bf16_t, true>(ST_ARGS) : launch_gla<bf16_t, false>(ST_ARGS);
#undef ST_ARGS
}

extern "C" int st_gated_head_norm(void* out, const float* o, const void* g, int64_t g_stride, const float* gain,
                                  int num_tokens, int heads, int value_dim, float eps, int dtype, hipStream_t stream) {
    ST_CHECK(num_tokens >= 0 && heads > 0 && value_dim > 0, "gated_head_norm: bad sizes");
    ST_CHECK(out && o && g && gain, "gated_head_norm: null operand");
    ST_CHECK(eps > 0.f, "gated_head_norm: eps must be positive");
    if (num_tokens == 0) return 0;
    const int64_t units = (int64_t)num_tokens * heads;
    const unsigned grid = (unsigned)((units + 3) / 4);
    if (dtype == kF32)
        gated_head_norm_kernel<float><<<grid, 256, 0, stream>>>((float*)out, o, (const float*)g, g_stride, gain,
                                                                num_tokens, heads, value_dim, eps);
    else if (dtype == kBF16)
        gated_head_norm_kernel<bf16_t><<<grid, 256, 0, stream>>>((bf16_t*)out, o, (const bf16_t*)g, g_stride, gain,
                                                                 num_tokens, heads, value_dim, eps);
    else ST_CHECK(false, "gated_head_norm: unknown dtype %d", dtype);
    ST_LAUNCH_CHECK("gated_head_norm");
    return 0;
}
