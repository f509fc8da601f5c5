// Gated linear attention: a matrix-valued state per request and head that decays per key channel.
//
//   S_t = diag(a_t) S_(t-1) + k_t v_t^T          S: [key_dim, value_dim], float, one per (slot, head)
//   o_t = scale * S_t^T q_t
//
// One kernel serves whole prompts, portions and single decoded tokens: it loads the state of the
// item's slot, walks over the item's rows in order and stores the state back, so the sum that
// reaches a position is formed in the same order however the tokens were cut into steps.
//
// The columns of S (value channels) never mix and the rows (key channels) only meet in the dot
// product with q.  The state, the decay and every sum are float whatever the storage type of q,
// k and v.
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

// One workgroup per (item, head): wave w takes the value channels 16 w .. 16 w + 15, its four
// 16-lane rows a quarter of the key channels each (DQ a lane, state in registers).  The item's
// rows are walked in chunks: all threads together bring a chunk's q, k, decay logits and v from
// memory into registers (every load in flight at once, while the chunk before is being
// computed), then into LDS as floats, the decay a = exp(log sigmoid(z) / tau) computed on the way
// once an element; then every lane reads what it needs from LDS, a token at a time.
// LDS row of a token: q [KP] | k [KP] | a [KP] | v [VP], KP = 4 DQ >= key_dim and VP = 16 waves,
// the padding zero (a padded key channel then adds nothing).  J: columns of that row a thread
// stages; C = 32 / J tokens a chunk.
template <typename T, int DQ, int J>
__global__ __launch_bounds__(1024) void gla_scan_kernel(
    float* __restrict__ o, const T* __restrict__ q, int64_t q_stride, const T* __restrict__ k, int64_t k_stride,
    const T* __restrict__ v, int64_t v_stride, const float* __restrict__ z, float* __restrict__ state,
    const int* __restrict__ item_len, const int* __restrict__ item_tok_off, const int* __restrict__ item_slot,
    int heads, int key_dim, int value_dim, float scale, float inv_tau) {
    constexpr int C = 32 / J, KP = 4 * DQ;
    extern __shared__ float lds[];
    const int h = blockIdx.x, item = blockIdx.y;
    const int slot = item_slot[item], n = item_len[item];
    if (slot < 0 || n <= 0) return;                    // a padding item of a batch of fixed size
    const int tid = threadIdx.x, threads = blockDim.x;
    const int lane = tid & 63, wave = tid >> 6, c16 = lane & 15, g = lane >> 4;
    const int VP = threads >> 2, per = 3 * KP + VP;
    const int col = wave * 16 + c16;
    const bool col_ok = col < value_dim;
    const int d0 = g * DQ;
    const int row0 = item_tok_off[item];

    float* s_ptr = state + (((int64_t)slot * heads + h) * key_dim + d0) * value_dim + col;
    float S[DQ];
#pragma unroll
    for (int i = 0; i < DQ; ++i) S[i] = (col_ok && d0 + i < key_dim) ? s_ptr[(int64_t)i * value_dim] : 0.f;

    // the columns of the LDS row this thread stages: where each comes from (kind 0 q, 1 k, 2 z, 3 v, -1 padding)
    int kind[J];
    int64_t src[J], stride[J];
#pragma unroll
    for (int j = 0; j < J; ++j) {
        const int e = tid + j * threads;
        kind[j] = -1; src[j] = 0; stride[j] = 0;
        if (e < 3 * KP) {
            const int seg = e / KP, d = e - seg * KP;
            if (d < key_dim) {
                kind[j] = seg;
                stride[j] = seg == 0 ? q_stride : seg == 1 ? k_stride : (int64_t)heads * key_dim;
                src[j] = (int64_t)row0 * stride[j] + (int64_t)h * key_dim + d;
            }
        } else if (e < per && e - 3 * KP < value_dim) {
            kind[j] = 3; stride[j] = v_stride;
            src[j] = (int64_t)row0 * v_stride + (int64_t)h * value_dim + (e - 3 * KP);
        }
    }
    float stage[J][C];
    auto fetch = [&](int r0) {
#pragma unroll
        for (int j = 0; j < J; ++j)
#pragma unroll
            for (int r = 0; r < C; ++r) {
                float x = 0.f;
                if (r0 + r < n) {
                    const int64_t at = src[j] + (int64_t)(r0 + r) * stride[j];
                    if (kind[j] == 0) x = Elem<T>::load(q + at);
                    else if (kind[j] == 1) x = Elem<T>::load(k + at);
                    else if (kind[j] == 2) x = z[at];
                    else if (kind[j] == 3) x = Elem<T>::load(v + at);
                }
                stage[j][r] = x;
            }
    };
    float* op = o + ((int64_t)row0 * heads + h) * value_dim + col;
    const int64_t o_stride = (int64_t)heads * value_dim;
    const float* lq = lds + d0;
    const float* lv = lds + 3 * KP + col;

    fetch(0);
    for (int r0 = 0; r0 < n; r0 += C) {
        __syncthreads();                               // the chunk before has been read
#pragma unroll
        for (int j = 0; j < J; ++j) {
            const int e = tid + j * threads;
            if (e >= per) continue;
#pragma unroll
            for (int r = 0; r < C; ++r) {
                float x = stage[j][r];
                if (kind[j] == 2) {
                    // a = sigmoid(z)^(1/tau);  log sigmoid(z) = min(z, 0) - log(1 + exp(-|z|))
                    x = expf((fminf(x, 0.f) - log1pf(expf(-fabsf(x)))) * inv_tau);
                }
                lds[r * per + e] = x;
            }
        }
        __syncthreads();
        if (r0 + C < n) fetch(r0 + C);
        const int rows = min(C, n - r0);
        for (int r = 0; r < rows; ++r) {
            const float* row = lq + r * per;
            const float vv = lv[r * per];
            float acc = 0.f;
#pragma unroll
            for (int i = 0; i < DQ; i += 4) {
                const float4 q4 = *reinterpret_cast<const float4*>(row + i);
                const float4 k4 = *reinterpret_cast<const float4*>(row + KP + i);
                const float4 a4 = *reinterpret_cast<const float4*>(row + 2 * KP + i);
                S[i] = fmaf(a4.x, S[i], k4.x * vv);         acc = fmaf(S[i], q4.x, acc);
                S[i + 1] = fmaf(a4.y, S[i + 1], k4.y * vv); acc = fmaf(S[i + 1], q4.y, acc);
                S[i + 2] = fmaf(a4.z, S[i + 2], k4.z * vv); acc = fmaf(S[i + 2], q4.z, acc);
                S[i + 3] = fmaf(a4.w, S[i + 3], k4.w * vv); acc = fmaf(S[i + 3], q4.w, acc);
            }
            acc = rows4_sum(acc);
            if (g == 0 && col_ok) op[(int64_t)(r0 + r) * o_stride] = acc * scale;
        }
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

template <typename T, int DQ>
static int launch_gla_dq(float* o, const void* q, int64_t qs, const void* k, int64_t ks, const void* v, int64_t vs,
                         const float* z, float* state, const int* item_len, const int* item_tok_off,
                         const int* item_slot, int num_items, int heads, int key_dim, int value_dim, float scale,
                         float inv_tau, hipStream_t stream) {
    const int waves = (value_dim + 15) / 16, threads = 64 * waves;
    const int per = 3 * 4 * DQ + 16 * waves;
    const int j = (per + threads - 1) / threads;
    const dim3 grid(heads, num_items);
    // (a chunk of the widest heads takes 128 KB of LDS, more than a launch gets without asking)
#define ST_GLA(J)                                                                                                    \
    {                                                                                                                \
        const size_t bytes = (size_t)(32 / J) * per * sizeof(float);                                                 \
        static bool asked = false;                                                                                   \
        if (bytes > 48 * 1024 && !asked) {                                                                           \
            ST_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(&gla_scan_kernel<T, DQ, J>),                  \
                                         hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024) == hipSuccess,      \
                     "gla_scan: the device refuses %zu bytes of LDS", bytes);                                        \
            asked = true;                                                                                            \
        }                                                                                                            \
        gla_scan_kernel<T, DQ, J><<<grid, threads, bytes, stream>>>(o, (const T*)q, qs, (const T*)k, ks,             \
            (const T*)v, vs, z, state, item_len, item_tok_off, item_slot, heads, key_dim, value_dim, scale, inv_tau);\
    }
    if (j <= 1) ST_GLA(1)
    else if (j <= 2) ST_GLA(2)
    else if (j <= 4) ST_GLA(4)
    else if (j <= 8) ST_GLA(8)
    else ST_GLA(16)
#undef ST_GLA
    ST_LAUNCH_CHECK("gla_scan");
    return 0;
}

template <typename T>
static int launch_gla(float* o, const void* q, int64_t qs, const void* k, int64_t ks, const void* v, int64_t vs,
                      const float* z, float* state, const int* item_len, const int* item_tok_off,
                      const int* item_slot, int num_items, int heads, int key_dim, int value_dim, float scale,
                      float inv_tau, hipStream_t stream) {
    const int dq = (key_dim + 3) / 4;
#define ST_GLA_ARGS o, q, qs, k, ks, v, vs, z, state, item_len, item_tok_off, item_slot, num_items, heads, key_dim, \
                    value_dim, scale, inv_tau, stream
    if (dq <= 4) return launch_gla_dq<T, 4>(ST_GLA_ARGS);
    if (dq <= 8) return launch_gla_dq<T, 8>(ST_GLA_ARGS);
    if (dq <= 12) return launch_gla_dq<T, 12>(ST_GLA_ARGS);
    if (dq <= 16) return launch_gla_dq<T, 16>(ST_GLA_ARGS);
    if (dq <= 24) return launch_gla_dq<T, 24>(ST_GLA_ARGS);
    if (dq <= 32) return launch_gla_dq<T, 32>(ST_GLA_ARGS);
    if (dq <= 48) return launch_gla_dq<T, 48>(ST_GLA_ARGS);
    return launch_gla_dq<T, 64>(ST_GLA_ARGS);
#undef ST_GLA_ARGS
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
                           const void* v, int64_t v_stride, const float* z, float* state,
                           const int* item_len, const int* item_tok_off, const int* item_slot, int num_items,
                           int heads, int key_dim, int value_dim, float scale, float inv_tau, int dtype,
                           hipStream_t stream) {
    ST_CHECK(num_items >= 0 && heads > 0 && key_dim > 0 && value_dim > 0, "gla_scan: bad sizes");
    ST_CHECK(key_dim <= 256 && value_dim <= 256, "gla_scan: up to 256 key and 256 value channels a head, not %d and %d",
             key_dim, value_dim);
    ST_CHECK(num_items <= 65535, "gla_scan: too many items");
    ST_CHECK(o && q && k && v && z && state && item_len && item_tok_off && item_slot, "gla_scan: null operand");
    ST_CHECK(inv_tau > 0.f, "gla_scan: the decay's exponent must be positive");
    ST_CHECK(dtype == kF32 || dtype == kBF16, "gla_scan: unknown dtype %d", dtype);
    if (num_items == 0) return 0;
    if (dtype == kF32)
        return launch_gla<float>(o, q, q_stride, k, k_stride, v, v_stride, z, state, item_len, item_tok_off, item_slot,
                                 num_items, heads, key_dim, value_dim, scale, inv_tau, stream);
    return launch_gla<bf16_t>(o, q, q_stride, k, k_stride, v, v_stride, z, state, item_len, item_tok_off, item_slot,
                              num_items, heads, key_dim, value_dim, scale, inv_tau, stream);
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
