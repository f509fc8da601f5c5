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
// rows are walked in chunks of C: all threads together bring a chunk's q, k, decay logits and v
// from memory into registers, then into LDS as floats, the decay a = exp(log sigmoid(z) / tau)
// computed on the way once an element; then every lane reads what it needs from LDS, a token at
// a time, while the next chunk's loads are in flight.  Every load is issued unconditionally
// (addresses clamped, values cleared when they are stored): a load whose result meets a constant
// at the end of a branch would be waited for on the spot, one after the other.
// LDS row of a token: q [KP] | k [KP] | a [KP] | v [VP], KP = 4 DQ >= key_dim and VP = 16 WAVES
// >= value_dim, the padding zero (a padded key channel then adds nothing).
template <int N> struct Pow2Up { static constexpr int value = N <= 16 ? 16 : N <= 32 ? 32 : N <= 64 ? 64 : N <= 128 ? 128 : 256; };

template <typename T, int DQ, int WAVES>
__global__ __launch_bounds__(64 * WAVES) void gla_scan_kernel(
    float* __restrict__ o, const T* __restrict__ q, int64_t q_stride, const T* __restrict__ k, int64_t k_stride,
    const T* __restrict__ v, int64_t v_stride, const float* __restrict__ z, float* __restrict__ state,
    const int* __restrict__ item_len, const int* __restrict__ item_tok_off, const int* __restrict__ item_slot,
    int heads, int key_dim, int value_dim, float scale, float inv_tau) {
    constexpr int KP = 4 * DQ, VP = 16 * WAVES, THREADS = 64 * WAVES, PER = 3 * KP + VP;
    constexpr int C = PER > 512 ? 16 : 32;                       // rows a chunk: at most 64 KB of LDS
    constexpr int KC = Pow2Up<KP>::value;                        // columns the threads are dealt over
    constexpr int SK = (C * KC + THREADS - 1) / THREADS;         // loads a thread and chunk, per key array
    constexpr int SV = (C * VP + THREADS - 1) / THREADS;         // and of v
    extern __shared__ float lds[];
    const int h = blockIdx.x, item = blockIdx.y;
    const int slot = item_slot[item], n = item_len[item];
    if (slot < 0 || n <= 0) return;                    // a padding item of a batch of fixed size
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6, c16 = lane & 15, g = lane >> 4;
    const int col = wave * 16 + c16;
    const bool col_ok = col < value_dim;
    const int d0 = g * DQ;
    const int row0 = item_tok_off[item];

    float* s_ptr = state + (((int64_t)slot * heads + h) * key_dim + d0) * value_dim + col;
    float S[DQ];
#pragma unroll
    for (int i = 0; i < DQ; ++i) S[i] = (col_ok && d0 + i < key_dim) ? s_ptr[(int64_t)i * value_dim] : 0.f;

    const T* qh = q + (int64_t)row0 * q_stride + (int64_t)h * key_dim;
    const T* kh = k + (int64_t)row0 * k_stride + (int64_t)h * key_dim;
    const T* vh = v + (int64_t)row0 * v_stride + (int64_t)h * value_dim;
    const int64_t z_stride = (int64_t)heads * key_dim;
    const float* zh = z + (int64_t)row0 * z_stride + (int64_t)h * key_dim;

    T sq[SK], sk[SK], sv[SV];
    float sz[SK];
    auto fetch = [&](int r0) {
        const int left = n - r0;                       // rows of this chunk onwards (uniform)
#pragma unroll
        for (int s = 0; s < SK; ++s) {
            if ((s * THREADS) / KC < left) {           // else: a slot wholly behind the item's last row (uniform)
                const int idx = tid + s * THREADS;
                const int r = min(r0 + idx / KC, n - 1), d = min(idx % KC, key_dim - 1);
                sq[s] = qh[(int64_t)r * q_stride + d];
                sk[s] = kh[(int64_t)r * k_stride + d];
                sz[s] = zh[(int64_t)r * z_stride + d];
            }
        }
#pragma unroll
        for (int s = 0; s < SV; ++s) {
            if ((s * THREADS) / VP < left) {
                const int idx = tid + s * THREADS;
                const int r = min(r0 + idx / VP, n - 1), d = min(idx % VP, value_dim - 1);
                sv[s] = vh[(int64_t)r * v_stride + d];
            }
        }
    };
    auto put = [&](int r0) {
        const int left = n - r0;
#pragma unroll
        for (int s = 0; s < SK; ++s) {
            const int idx = tid + s * THREADS;
            const int r = idx / KC, d = idx % KC;
            if ((s * THREADS) / KC < left && r < C && d < KP) {
                const bool ok = d < key_dim && r < left;
                float* dst = lds + r * PER + d;
                const float zz = sz[s];
                // a = sigmoid(z)^(1/tau);  log sigmoid(z) = min(z, 0) - log(1 + exp(-|z|))
                const float a = expf((fminf(zz, 0.f) - log1pf(expf(-fabsf(zz)))) * inv_tau);
                dst[0] = ok ? Elem<T>::load(&sq[s]) : 0.f;
                dst[KP] = ok ? Elem<T>::load(&sk[s]) : 0.f;
                dst[2 * KP] = ok ? a : 0.f;
            }
        }
#pragma unroll
        for (int s = 0; s < SV; ++s) {
            const int idx = tid + s * THREADS;
            const int r = idx / VP, d = idx % VP;
            if ((s * THREADS) / VP < left && r < C) lds[r * PER + 3 * KP + d] = (d < value_dim && r < left) ? Elem<T>::load(&sv[s]) : 0.f;
        }
    };
    float* op = o + ((int64_t)row0 * heads + h) * value_dim + col;
    const int64_t o_stride = (int64_t)heads * value_dim;
    const float* lq = lds + d0;
    const float* lv = lds + 3 * KP + col;

    fetch(0);
    for (int r0 = 0; r0 < n; r0 += C) {
        __syncthreads();                               // the chunk before has been read
        put(r0);
        __syncthreads();
        if (r0 + C < n) fetch(r0 + C);
        const int rows = min(C, n - r0);
        // a row's operands are read from LDS while the row before it is computed
        float4 q4[DQ / 4], k4[DQ / 4], a4[DQ / 4], qn[DQ / 4], kn[DQ / 4], an[DQ / 4];
        float vv, vn;
        auto read = [&](int r, float4* qq, float4* kk, float4* aa, float& v1) {
            const float* row = lq + r * PER;
#pragma unroll
            for (int i = 0; i < DQ / 4; ++i) {
                qq[i] = *reinterpret_cast<const float4*>(row + 4 * i);
                kk[i] = *reinterpret_cast<const float4*>(row + KP + 4 * i);
                aa[i] = *reinterpret_cast<const float4*>(row + 2 * KP + 4 * i);
            }
            v1 = lv[r * PER];
        };
        read(0, q4, k4, a4, vv);
        for (int r = 0; r < rows; ++r) {
            read(min(r + 1, C - 1), qn, kn, an, vn);
            float acc = 0.f;
#pragma unroll
            for (int i = 0; i < DQ / 4; ++i) {
                const int j = 4 * i;
                S[j] = fmaf(a4[i].x, S[j], k4[i].x * vv);         acc = fmaf(S[j], q4[i].x, acc);
                S[j + 1] = fmaf(a4[i].y, S[j + 1], k4[i].y * vv); acc = fmaf(S[j + 1], q4[i].y, acc);
                S[j + 2] = fmaf(a4[i].z, S[j + 2], k4[i].z * vv); acc = fmaf(S[j + 2], q4[i].z, acc);
                S[j + 3] = fmaf(a4[i].w, S[j + 3], k4[i].w * vv); acc = fmaf(S[j + 3], q4[i].w, acc);
            }
            acc = rows4_sum(acc);
            if (g == 0 && col_ok) op[(int64_t)(r0 + r) * o_stride] = acc * scale;
#pragma unroll
            for (int i = 0; i < DQ / 4; ++i) { q4[i] = qn[i]; k4[i] = kn[i]; a4[i] = an[i]; }
            vv = vn;
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
    const int waves = (value_dim + 15) / 16;
    const dim3 grid(heads, num_items);
    // (a chunk takes up to 64 KB of LDS, more than a launch gets without asking)
#define ST_GLA(W)                                                                                                    \
    {                                                                                                                \
        constexpr int per = 12 * DQ + 16 * W;                                                                        \
        constexpr size_t bytes = (size_t)(per > 512 ? 16 : 32) * per * sizeof(float);                                \
        static bool asked = false;                                                                                   \
        if (bytes > 32 * 1024 && !asked) {                                                                           \
            ST_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(&gla_scan_kernel<T, DQ, W>),                  \
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes) == hipSuccess,      \
                     "gla_scan: the device refuses %zu bytes of LDS", bytes);                                        \
            asked = true;                                                                                            \
        }                                                                                                            \
        gla_scan_kernel<T, DQ, W><<<grid, 64 * W, bytes, stream>>>(o, (const T*)q, qs, (const T*)k, ks,              \
            (const T*)v, vs, z, state, item_len, item_tok_off, item_slot, heads, key_dim, value_dim, scale, inv_tau);\
    }
    if (waves <= 1) ST_GLA(1)
    else if (waves <= 2) ST_GLA(2)
    else if (waves <= 4) ST_GLA(4)
    else if (waves <= 8) ST_GLA(8)
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
