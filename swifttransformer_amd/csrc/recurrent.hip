// Gated linear attention: a matrix-valued state per request and head that decays per key channel.
//
//   S_t = diag(a_t) S_(t-1) + k_t v_t^T          S: [key_dim, value_dim], float, one per (slot, head)
//   o_t = scale * S_t^T q_t
//
// One kernel serves whole prompts, portions and single decoded tokens: it loads the state of the
// item's slot, walks over the item's rows in order and stores the state back, so the sum that
// reaches a position is formed in the same order however the tokens were cut into steps.
//
// The columns of S (value channels) never mix, and the rows (key channels) only meet in the dot
// product with q: a wave takes 64 value channels (one a lane) and a part of DQ key channels, keeps
// its DQ x 64 piece of S in registers, and writes its partial dot products to a plane of its own;
// the head norm that follows sums the planes.  So no two waves ever wait for each other, and a
// head is spread over as many compute units as it has parts.  What a wave needs of q, k and the
// decay is the same for all its lanes: the wave brings 32 tokens' worth of them into its own LDS
// with a dozen coalesced loads (the next 32 on their way while these are used) and every lane
// reads them back from there, all lanes one address; v comes as one coalesced load a token.
// Per token a lane does 3 DQ multiply-adds.
// The state, the decay and every sum are float whatever the storage type of q, k and v.
#include "api.h"
#include "common.h"

namespace st {

__global__ __launch_bounds__(256) void decay_gate_out_kernel(float* __restrict__ out, const float* __restrict__ z,
                                                             int64_t n, float inv_tau) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    const float v = z[i];
    out[i] = expf((fminf(v, 0.f) - log1pf(expf(-fabsf(v)))) * inv_tau);
}

// grid (heads * parts, ceil(value_dim / 64), items), one wave a workgroup.  LDS row of a token:
// q [DQ] | k [DQ] | a [DQ] of this wave's part, the part's tail (key channels the head does not
// have) zero.  Loads are issued unconditionally, addresses clamped: a load whose result meets a
// constant at the end of a branch would be waited for on the spot.
template <typename T, int DQ>
__global__ __launch_bounds__(64) void gla_scan_kernel(
    float* __restrict__ o_part, int64_t part_stride, const T* __restrict__ q, int64_t q_stride,
    const T* __restrict__ k, int64_t k_stride, const T* __restrict__ v, int64_t v_stride,
    const float* __restrict__ a, float* __restrict__ state,
    const int* __restrict__ item_len, const int* __restrict__ item_tok_off, const int* __restrict__ item_slot,
    int heads, int parts, int key_dim, int value_dim, float scale) {
    constexpr int C = 32;                              // tokens a chunk
    constexpr int NL = C * DQ / 64;                    // loads a lane, chunk and operand
    __shared__ float lds[C * 3 * DQ];
    const int h = blockIdx.x / parts, part = blockIdx.x - h * parts, item = blockIdx.z;
    const int slot = item_slot[item], n = item_len[item];
    if (slot < 0 || n <= 0) return;                    // a padding item of a batch of fixed size
    const int lane = threadIdx.x;
    const int col = blockIdx.y * 64 + lane;
    const bool col_ok = col < value_dim;
    const int d0 = part * DQ;
    const int dn = min(DQ, key_dim - d0);              // key channels of this part (the last may be short)
    const int row0 = item_tok_off[item];

    float* s_ptr = state + (((int64_t)slot * heads + h) * key_dim + d0) * value_dim + col;
    float S[DQ];
#pragma unroll
    for (int i = 0; i < DQ; ++i) S[i] = (col_ok && i < dn) ? s_ptr[(int64_t)i * value_dim] : 0.f;

    const T* qp = q + (int64_t)row0 * q_stride + (int64_t)h * key_dim + d0;
    const T* kp = k + (int64_t)row0 * k_stride + (int64_t)h * key_dim + d0;
    const int64_t a_stride = (int64_t)heads * key_dim, o_stride = (int64_t)heads * value_dim;
    const float* ap = a + (int64_t)row0 * a_stride + (int64_t)h * key_dim + d0;
    const T* vp = v + (int64_t)row0 * v_stride + (int64_t)h * value_dim + (col_ok ? col : 0);
    float* op = o_part + (int64_t)part * part_stride + (int64_t)row0 * o_stride + (int64_t)h * value_dim + col;

    // lane's places in a chunk's operand block: (token idx / DQ, channel idx % DQ), idx = lane + 64 s
    T sq[NL], sk[NL], sv[C];
    float sa[NL];
    auto fetch = [&](int r0) {
#pragma unroll
        for (int s = 0; s < NL; ++s) {
            const int idx = lane + 64 * s;
            const int64_t r = min(r0 + idx / DQ, n - 1);
            const int d = min(idx % DQ, dn - 1);
            sq[s] = qp[r * q_stride + d];
            sk[s] = kp[r * k_stride + d];
            sa[s] = ap[r * a_stride + d];
        }
        const int left = n - r0;
#pragma unroll
        for (int r = 0; r < C; ++r)
            if (r < left) sv[r] = vp[(int64_t)(r0 + r) * v_stride];       // (uniform; nothing reads the others)
    };
    fetch(0);
    for (int r0 = 0; r0 < n; r0 += C) {
        __syncthreads();                               // the chunk before has been read
#pragma unroll
        for (int s = 0; s < NL; ++s) {
            const int idx = lane + 64 * s;
            const int r = idx / DQ, d = idx % DQ;
            const bool ok = d < dn;
            float* dst = lds + r * (3 * DQ) + d;
            dst[0] = ok ? Elem<T>::load(&sq[s]) : 0.f;
            dst[DQ] = ok ? Elem<T>::load(&sk[s]) : 0.f;
            dst[2 * DQ] = ok ? sa[s] : 0.f;
        }
        float vv[C];
#pragma unroll
        for (int r = 0; r < C; ++r) vv[r] = Elem<T>::load(&sv[r]);
        __syncthreads();
        if (r0 + C < n) fetch(r0 + C);
        const int rows = min(C, n - r0);
#pragma unroll
        for (int r = 0; r < C; ++r) {
            if (r < rows) {                            // (uniform)
                const float* row = lds + r * (3 * DQ);
                float acc = 0.f;
#pragma unroll
                for (int i = 0; i < DQ; i += 4) {
                    const float4 q4 = *reinterpret_cast<const float4*>(row + i);
                    const float4 k4 = *reinterpret_cast<const float4*>(row + DQ + i);
                    const float4 a4 = *reinterpret_cast<const float4*>(row + 2 * DQ + i);
                    S[i] = fmaf(a4.x, S[i], k4.x * vv[r]);         acc = fmaf(S[i], q4.x, acc);
                    S[i + 1] = fmaf(a4.y, S[i + 1], k4.y * vv[r]); acc = fmaf(S[i + 1], q4.y, acc);
                    S[i + 2] = fmaf(a4.z, S[i + 2], k4.z * vv[r]); acc = fmaf(S[i + 2], q4.z, acc);
                    S[i + 3] = fmaf(a4.w, S[i + 3], k4.w * vv[r]); acc = fmaf(S[i + 3], q4.w, acc);
                }
                if (col_ok) op[(int64_t)(r0 + r) * o_stride] = acc * scale;
            }
        }
    }
#pragma unroll
    for (int i = 0; i < DQ; ++i)
        if (col_ok && i < dn) s_ptr[(int64_t)i * value_dim] = S[i];
}

// One wave per (token, head): root-mean-square norm over the head's value channels, the gain, and
// the gate silu(g).
template <typename T>
__global__ __launch_bounds__(256) void gated_head_norm_kernel(
    T* __restrict__ out, const float* __restrict__ o, int parts, int64_t part_stride, const T* __restrict__ g,
    int64_t g_stride, const float* __restrict__ gain, int num_tokens, int heads, int value_dim, float eps) {
    const int lane = threadIdx.x & 63;
    const int64_t unit = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);      // (token, head)
    if (unit >= (int64_t)num_tokens * heads) return;
    const int64_t t = unit / heads;
    const int h = (int)(unit - t * heads);
    const float* op = o + unit * value_dim;
    const T* gp = g + t * g_stride + (int64_t)h * value_dim;
    T* dst = out + unit * value_dim;
    // the planes of partial results are summed in their order; up to 4 values a lane stay in registers
    float x[4];
    float ss = 0.f;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        const int j = lane + 64 * u;
        float sum = 0.f;
        if (j < value_dim)
            for (int p = 0; p < parts; ++p) sum += op[(int64_t)p * part_stride + j];
        x[u] = sum;
        ss = fmaf(sum, sum, ss);
    }
    ss = wave_sum(ss);
    const float r = 1.f / sqrtf(ss / (float)value_dim + eps);
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        const int j = lane + 64 * u;
        if (j >= value_dim) continue;
        const float gv = Elem<T>::load(gp + j);
        Elem<T>::store(dst + j, x[u] * r * gain[j] * (gv / (1.f + expf(-gv))));
    }
}

template <typename T, int DQ>
static int launch_gla(float* o_part, int64_t part_stride, const void* q, int64_t qs, const void* k, int64_t ks,
                      const void* v, int64_t vs, const float* a, float* state, const int* item_len,
                      const int* item_tok_off, const int* item_slot, int num_items, int heads, int key_dim,
                      int value_dim, float scale, hipStream_t stream) {
    const int parts = (key_dim + DQ - 1) / DQ;
    const dim3 grid(heads * parts, (value_dim + 63) / 64, num_items);
    gla_scan_kernel<T, DQ><<<grid, 64, 0, stream>>>(o_part, part_stride, (const T*)q, qs, (const T*)k, ks,
        (const T*)v, vs, a, state, item_len, item_tok_off, item_slot, heads, parts, key_dim, value_dim, scale);
    ST_LAUNCH_CHECK("gla_scan");
    return 0;
}

}  // namespace st

using namespace st;

extern "C" int st_decay_gate(float* out, const float* z, int64_t n, float inv_tau, hipStream_t stream) {
    ST_CHECK(n >= 0 && ((z && out) || n == 0), "decay_gate: bad operands");
    ST_CHECK(inv_tau > 0.f, "decay_gate: the exponent must be positive");
    if (n == 0) return 0;
    decay_gate_out_kernel<<<(unsigned)((n + 255) / 256), 256, 0, stream>>>(out, z, n, inv_tau);
    ST_LAUNCH_CHECK("decay_gate");
    return 0;
}

extern "C" int st_gla_scan_parts(int key_dim, int part_dim) {
    return part_dim > 0 ? (key_dim + part_dim - 1) / part_dim : 0;
}

extern "C" int st_gla_scan(float* o_part, int64_t part_stride, int part_dim, const void* q, int64_t q_stride,
                           const void* k, int64_t k_stride, const void* v, int64_t v_stride, const float* a,
                           float* state, const int* item_len, const int* item_tok_off, const int* item_slot,
                           int num_items, int heads, int key_dim, int value_dim, float scale, int dtype,
                           hipStream_t stream) {
    ST_CHECK(num_items >= 0 && heads > 0 && key_dim > 0 && value_dim > 0, "gla_scan: bad sizes");
    ST_CHECK(part_dim == 4 || part_dim == 8 || part_dim == 16, "gla_scan: parts of 4, 8 or 16 key channels, not %d", part_dim);
    const int parts = (key_dim + part_dim - 1) / part_dim;
    ST_CHECK((int64_t)heads * parts <= 0x7fffffff && num_items <= 65535 && (value_dim + 63) / 64 <= 65535,
             "gla_scan: too many heads, items or value channels");
    ST_CHECK(o_part && q && k && v && a && state && item_len && item_tok_off && item_slot, "gla_scan: null operand");
    ST_CHECK(dtype == kF32 || dtype == kBF16, "gla_scan: unknown dtype %d", dtype);
    if (num_items == 0) return 0;
#define ST_ARGS o_part, part_stride, q, q_stride, k, k_stride, v, v_stride, a, state, item_len, item_tok_off, \
                item_slot, num_items, heads, key_dim, value_dim, scale, stream
    if (dtype == kF32) {
        if (part_dim == 4) return launch_gla<float, 4>(ST_ARGS);
        if (part_dim == 8) return launch_gla<float, 8>(ST_ARGS);
        return launch_gla<float, 16>(ST_ARGS);
    }
    if (part_dim == 4) return launch_gla<bf16_t, 4>(ST_ARGS);
    if (part_dim == 8) return launch_gla<bf16_t, 8>(ST_ARGS);
    return launch_gla<bf16_t, 16>(ST_ARGS);
#undef ST_ARGS
}

extern "C" int st_gated_head_norm(void* out, const float* o, int parts, int64_t part_stride, const void* g,
                                  int64_t g_stride, const float* gain, int num_tokens, int heads, int value_dim,
                                  float eps, int dtype, hipStream_t stream) {
    ST_CHECK(num_tokens >= 0 && heads > 0 && value_dim > 0 && value_dim <= 256 && parts >= 1,
             "gated_head_norm: bad sizes (up to 256 value channels a head)");
    ST_CHECK(out && o && g && gain, "gated_head_norm: null operand");
    ST_CHECK(eps > 0.f, "gated_head_norm: eps must be positive");
    if (num_tokens == 0) return 0;
    const int64_t units = (int64_t)num_tokens * heads;
    const unsigned grid = (unsigned)((units + 3) / 4);
    if (dtype == kF32)
        gated_head_norm_kernel<float><<<grid, 256, 0, stream>>>((float*)out, o, parts, part_stride, (const float*)g,
                                                                g_stride, gain, num_tokens, heads, value_dim, eps);
    else if (dtype == kBF16)
        gated_head_norm_kernel<bf16_t><<<grid, 256, 0, stream>>>((bf16_t*)out, o, parts, part_stride, (const bf16_t*)g,
                                                                 g_stride, gain, num_tokens, heads, value_dim, eps);
    else ST_CHECK(false, "gated_head_norm: unknown dtype %d", dtype);
    ST_LAUNCH_CHECK("gated_head_norm");
    return 0;
}
