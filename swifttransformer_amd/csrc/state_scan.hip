// Recurrent mixers with a matrix state S [key channels x value channels] a head and one scalar
// decay a head and token, for batches of portions of sequences.  Two recurrences share one kernel:
//
//   additive (state-space duality):  S <- a_t S + (b_t k_t) v_t^T;          o_t = S^T q_t + D v_t
//   delta rule:                      S <- a_t S;  u = b_t (v_t - S^T k_t);
//                                    S <- S + k_t u^T;                      o_t = S^T q_t
//
// a_t (the decay) and b_t (the step size, or the write strength) are float [T, heads] made by
// `recurrence_gates`; q, k, v are float rows; the state is float, lives in the request's slot and is
// loaded before and stored after the item's rows, so prompts, portions and single tokens take the
// same route and a position's sums are formed in the same order however the tokens were cut.
//
// Launch: a workgroup a (head, block of 64 value channels, item); lane = value channel, wave = a
// part of 16 key channels, whose column of the state stays in registers.  The waves' partial dot
// products meet in LDS: one barrier a token for the additive form, two for the delta rule (its
// write needs S^T k over all key channels first).  Operands are staged through LDS a chunk of
// tokens at a time.
#include "api.h"
#include "common.h"

namespace st {

constexpr int kScanPart = 16;        // key channels a wave
constexpr int kScanMaxParts = 16;    // up to 256 key channels

__device__ inline float softplus_f(float x) { return x > 20.f ? x : log1pf(expf(x)); }

// mode 0: raw [T, heads]: a = softplus(raw + bias) (step size), b = exp(-exp(a_log) * a) (decay)
// mode 1: raw [T, 2 * heads] = write logits | decay logits:
//         a = sigmoid(raw[:, :heads]), b = exp(-exp(a_log) * softplus(raw[:, heads:] + bias))
__global__ __launch_bounds__(256) void recurrence_gates_kernel(
    float* __restrict__ out_a, float* __restrict__ out_b, const float* __restrict__ raw, int64_t raw_stride,
    const float* __restrict__ a_log, const float* __restrict__ bias, int64_t n, int heads, int mode) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    const int64_t t = i / heads;
    const int h = (int)(i - t * heads);
    const float* r = raw + t * raw_stride;
    if (mode == 0) {
        const float dt = softplus_f(r[h] + bias[h]);
        out_a[i] = dt;
        out_b[i] = expf(-expf(a_log[h]) * dt);
    } else {
        out_a[i] = 1.f / (1.f + expf(-r[h]));
        out_b[i] = expf(-expf(a_log[h]) * softplus_f(r[heads + h] + bias[h]));
    }
}

// x[t, h, :] <- x[t, h, :] / sqrt(sum x^2 + eps) * scale, float rows, a wave a (row, head)
__global__ __launch_bounds__(256) void unit_norm_kernel(float* __restrict__ x, int64_t stride, int64_t units,
                                                        int heads, int dim, float eps, float scale) {
    const int64_t u = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (u >= units) return;
    const int lane = threadIdx.x & 63;
    const int64_t t = u / heads;
    const int h = (int)(u - t * heads);
    float* p = x + t * stride + (int64_t)h * dim;
    float ss = 0.f;
    for (int j = lane; j < dim; j += 64) ss = fmaf(p[j], p[j], ss);
    ss = wave_sum(ss);
    const float r = scale / sqrtf(ss + eps);
    for (int j = lane; j < dim; j += 64) p[j] *= r;
}

// Operands of `chunk` tokens at a time are staged in LDS, q [chunk, key_dim] | k [chunk, key_dim] |
// v [chunk, 64] | a [chunk] | b [chunk], so that the walk over the tokens waits for LDS only.
// floats a thread carries from memory to LDS for a chunk: what its register budget allows
constexpr int scan_regs(int max_parts) { return max_parts >= 16 ? 6 : max_parts >= 8 ? 16 : 32; }

template <int MODE, int MAXPARTS>
__global__ __launch_bounds__(64 * MAXPARTS) void state_scan_kernel(
    float* __restrict__ out, const float* __restrict__ q, int64_t q_stride, const float* __restrict__ k,
    int64_t k_stride, const float* __restrict__ v, int64_t v_stride, const float* __restrict__ ga,
    const float* __restrict__ gb, const float* __restrict__ skip, float* __restrict__ state, int64_t slot_stride,
    const int* __restrict__ item_len, const int* __restrict__ item_tok_off, const int* __restrict__ item_slot,
    int heads, int qk_heads, int key_dim, int value_dim, int chunk) {
    extern __shared__ __attribute__((aligned(16))) float staged[];   // a chunk's operands, then its results [chunk, 64]
    __shared__ float red[2][kScanMaxParts][64];
    const int head = blockIdx.x, item = blockIdx.z;
    const int tid = threadIdx.x, lane = tid & 63, part = tid >> 6;
    const int nthreads = blockDim.x, parts = nthreads >> 6;
    const int col0 = blockIdx.y * 64, col = col0 + lane;
    const bool live = col < value_dim;
    const int slot = item_slot[item], n = item_len[item];
    if (slot < 0 || n <= 0) return;                     // uniform over the workgroup
    const int64_t row0 = item_tok_off[item];
    const int qk_head = head / (heads / qk_heads);
    const int k0 = part * kScanPart;
    float S[kScanPart];
    float* sp = state + (int64_t)slot * slot_stride + ((int64_t)head * key_dim + k0) * value_dim + col;
#pragma unroll
    for (int i = 0; i < kScanPart; ++i)
        S[i] = (live && k0 + i < key_dim) ? sp[(int64_t)i * value_dim] : 0.f;
    const float d_skip = skip ? skip[head] : 0.f;
    const float* qp = q + row0 * q_stride + (int64_t)qk_head * key_dim;
    const float* kp = k + row0 * k_stride + (int64_t)qk_head * key_dim;
    const float* vp = v + row0 * v_stride + (int64_t)head * value_dim + col0;
    const float* ap = ga + row0 * heads + head;
    const float* bp = gb + row0 * heads + head;
    float* op = out + row0 * ((int64_t)heads * value_dim) + (int64_t)head * value_dim + col0;
    const int kdp = kScanPart * parts;                  // a row of q or k in LDS: padded with zeros to whole parts
    const int nq = chunk * kdp, nv = chunk * 64;
    // A chunk's operands go to LDS through registers: all of a thread's loads are issued before any is
    // stored, so that a chunk costs one trip to memory, not one an element.  Rows beyond the item's end
    // are zeros.
    const int per_buf = 2 * nq + nv + 2 * chunk;
    float* res = staged + per_buf;
    const int chunks = (n + chunk - 1) / chunk;
    for (int c = 0; c < chunks; ++c) {
        const float* buf = staged;
        const int t0 = c * chunk;
        constexpr int kRegs = scan_regs(MAXPARTS);
        float pre[kRegs];
#pragma unroll
        for (int i = 0; i < kRegs; ++i) {
            const int idx = tid + i * nthreads;
            const float* src = nullptr;
            if (idx < 2 * nq) {
                const int j = idx < nq ? idx : idx - nq;
                const int r = j / kdp, cc = j - r * kdp;
                if (t0 + r < n && cc < key_dim) src = idx < nq ? qp + (int64_t)(t0 + r) * q_stride + cc : kp + (int64_t)(t0 + r) * k_stride + cc;
            } else if (idx < 2 * nq + nv) {
                const int j = idx - 2 * nq, r = j >> 6, cc = j & 63;
                if (t0 + r < n && col0 + cc < value_dim) src = vp + (int64_t)(t0 + r) * v_stride + cc;
            } else if (idx < per_buf) {
                const int j = idx - 2 * nq - nv;
                const int r = j < chunk ? j : j - chunk;
                if (t0 + r < n) src = (j < chunk ? ap : bp) + (int64_t)(t0 + r) * heads;
            }
            pre[i] = src ? *src : 0.f;
        }
        __syncthreads();                     // the chunk before has been walked by every wave
#pragma unroll
        for (int i = 0; i < kRegs; ++i) {
            const int idx = tid + i * nthreads;
            if (idx < per_buf) staged[idx] = pre[i];
        }
        __syncthreads();
        const int rows = min(chunk, n - c * chunk);
        for (int r = 0; r < rows; ++r) {
            const int t = c * chunk + r;
            float cq[kScanPart], ck[kScanPart];
            {
                const float4* q4 = reinterpret_cast<const float4*>(buf + r * kdp + k0);
                const float4* k4 = reinterpret_cast<const float4*>(buf + nq + r * kdp + k0);
#pragma unroll
                for (int i = 0; i < kScanPart / 4; ++i) {
                    const float4 a4 = q4[i], b4 = k4[i];
                    cq[4 * i] = a4.x; cq[4 * i + 1] = a4.y; cq[4 * i + 2] = a4.z; cq[4 * i + 3] = a4.w;
                    ck[4 * i] = b4.x; ck[4 * i + 1] = b4.y; ck[4 * i + 2] = b4.z; ck[4 * i + 3] = b4.w;
                }
            }
            const float cv = buf[2 * nq + r * 64 + lane];
            const float ca = buf[2 * nq + nv + r], cb = buf[2 * nq + nv + chunk + r];
            float acc = 0.f;
            if (MODE == 0) {
                // ca: the step size, cb: the decay
                const float w = ca * cv;
#pragma unroll
                for (int i = 0; i < kScanPart; ++i) {
                    S[i] = fmaf(cb, S[i], ck[i] * w);
                    acc = fmaf(S[i], cq[i], acc);
                }
                red[t & 1][part][lane] = acc;
                __syncthreads();
                if (part == 0) {
                    float sum = 0.f;
                    for (int p = 0; p < parts; ++p) sum += red[t & 1][p][lane];
                    res[r * 64 + lane] = fmaf(d_skip, cv, sum);
                }
            } else {
                // ca: the write strength, cb: the decay
#pragma unroll
                for (int i = 0; i < kScanPart; ++i) acc = fmaf(S[i], ck[i], acc);
                red[0][part][lane] = acc;
                __syncthreads();
                float read = 0.f;
                for (int p = 0; p < parts; ++p) read += red[0][p][lane];
                const float u = ca * (cv - cb * read);
                acc = 0.f;
#pragma unroll
                for (int i = 0; i < kScanPart; ++i) {
                    S[i] = fmaf(cb, S[i], ck[i] * u);
                    acc = fmaf(S[i], cq[i], acc);
                }
                red[1][part][lane] = acc;
                __syncthreads();
                if (part == 0) {
                    float sum = 0.f;
                    for (int p = 0; p < parts; ++p) sum += red[1][p][lane];
                    res[r * 64 + lane] = sum;
                }
            }
        }
        // the chunk's results leave together: a store a token would make every barrier wait for memory
        __syncthreads();
        for (int j = tid; j < rows * 64; j += nthreads) {
            const int r = j >> 6, cc = j & 63;
            if (col0 + cc < value_dim) op[(int64_t)(t0 + r) * heads * value_dim + cc] = res[j];
        }
    }
    if (live) {
#pragma unroll
        for (int i = 0; i < kScanPart; ++i)
            if (k0 + i < key_dim) sp[(int64_t)i * value_dim] = S[i];
    }
}

// out[t, g, j] = val * rsqrt(mean_j(val^2) + eps) * gain * (gate_first ? 1 : silu(gate)),
// val = o[t, g, j] * (gate_first ? silu(gate[t, g, j]) : 1); a workgroup a (row, group)
template <typename T>
__global__ __launch_bounds__(256) void gated_group_norm_kernel(
    T* __restrict__ out, const float* __restrict__ o, const T* __restrict__ gate, int64_t gate_stride,
    const float* __restrict__ gain, int groups, int width, int gain_per_group, int gate_first, float eps) {
    __shared__ float red[16];
    const int64_t t = blockIdx.x / groups;
    const int g = blockIdx.x - (int)t * groups;
    const float* op = o + (t * groups + g) * width;
    const T* gp = gate + t * gate_stride + (int64_t)g * width;
    const float* wp = gain + (gain_per_group ? (int64_t)g * width : 0);
    T* dst = out + (t * groups + g) * width;
    float ss = 0.f;
    for (int j = threadIdx.x; j < width; j += 256) {
        float val = op[j];
        if (gate_first) {
            const float z = Elem<T>::load(gp + j);
            val *= z / (1.f + expf(-z));
        }
        ss = fmaf(val, val, ss);
    }
    ss = block_sum(ss, red);
    const float r = 1.f / sqrtf(ss / (float)width + eps);
    for (int j = threadIdx.x; j < width; j += 256) {
        const float z = Elem<T>::load(gp + j);
        const float s = z / (1.f + expf(-z));
        const float val = op[j] * r * wp[j] * s;
        Elem<T>::store(dst + j, val);
    }
}

}  // namespace st

using namespace st;

extern "C" int st_recurrence_gates(float* out_a, float* out_b, const float* raw, int64_t raw_stride,
                                   const float* a_log, const float* bias, int num_tokens, int heads, int mode,
                                   hipStream_t stream) {
    ST_CHECK(num_tokens >= 0 && heads > 0 && (mode == 0 || mode == 1), "recurrence_gates: bad sizes or mode");
    if (num_tokens == 0) return 0;
    ST_CHECK(out_a && out_b && raw && a_log && bias, "recurrence_gates: null operand");
    const int64_t n = (int64_t)num_tokens * heads;
    recurrence_gates_kernel<<<(unsigned)((n + 255) / 256), 256, 0, stream>>>(out_a, out_b, raw, raw_stride, a_log,
                                                                           bias, n, heads, mode);
    ST_LAUNCH_CHECK("recurrence_gates");
    return 0;
}

extern "C" int st_unit_norm(float* x, int64_t stride, int num_tokens, int heads, int dim, float eps, float scale,
                            hipStream_t stream) {
    ST_CHECK(num_tokens >= 0 && heads > 0 && dim > 0, "unit_norm: bad sizes");
    if (num_tokens == 0) return 0;
    ST_CHECK(x, "unit_norm: null operand");
    const int64_t units = (int64_t)num_tokens * heads;
    unit_norm_kernel<<<(unsigned)((units + 3) / 4), 256, 0, stream>>>(x, stride, units, heads, dim, eps, scale);
    ST_LAUNCH_CHECK("unit_norm");
    return 0;
}

extern "C" int st_state_scan(float* out, const float* q, int64_t q_stride, const float* k, int64_t k_stride,
                             const float* v, int64_t v_stride, const float* gate_a, const float* gate_b,
                             const float* skip, float* state, int64_t slot_stride, const int* item_len,
                             const int* item_tok_off, const int* item_slot, int num_items, int heads, int qk_heads,
                             int key_dim, int value_dim, int mode, hipStream_t stream) {
    ST_CHECK(num_items >= 0 && heads > 0 && qk_heads > 0 && heads % qk_heads == 0 && key_dim > 0 && value_dim > 0,
             "state_scan: bad sizes");
    ST_CHECK(key_dim <= kScanPart * kScanMaxParts, "state_scan: up to %d key channels a head, not %d",
             kScanPart * kScanMaxParts, key_dim);
    ST_CHECK(mode == 0 || mode == 1, "state_scan: mode 0 (additive) or 1 (delta rule)");
    ST_CHECK(num_items <= 65535 && (value_dim + 63) / 64 <= 65535, "state_scan: too many items or value channels");
    if (num_items == 0) return 0;
    ST_CHECK(out && q && k && v && gate_a && gate_b && state && item_len && item_tok_off && item_slot,
             "state_scan: null operand");
    const int parts = (key_dim + kScanPart - 1) / kScanPart;
    const dim3 grid(heads, (value_dim + 63) / 64, num_items);
    // tokens a chunk: what 32 KB of LDS and the threads' staging registers hold
    const int max_parts = parts <= 1 ? 1 : parts <= 2 ? 2 : parts <= 4 ? 4 : parts <= 8 ? 8 : 16;
    int chunk = 64;
    const int kdp = kScanPart * parts;
    while (chunk > 1 && (4 * chunk * (2 * kdp + 66 + 64) > 40 * 1024 ||
                         chunk * (2 * kdp + 66) > scan_regs(max_parts) * 64 * parts))
        chunk >>= 1;
    const size_t lds = (size_t)4 * chunk * (2 * kdp + 66 + 64);
#define ST_SCAN(MODE, MP)                                                                                         \
    state_scan_kernel<MODE, MP><<<grid, 64 * parts, lds, stream>>>(out, q, q_stride, k, k_stride, v, v_stride,    \
        gate_a, gate_b, skip, state, slot_stride, item_len, item_tok_off, item_slot, heads, qk_heads, key_dim,    \
        value_dim, chunk)
#define ST_SCAN_MODE(MP) do { if (mode == 0) ST_SCAN(0, MP); else ST_SCAN(1, MP); } while (0)
    switch (max_parts) {
        case 1: ST_SCAN_MODE(1); break;
        case 2: ST_SCAN_MODE(2); break;
        case 4: ST_SCAN_MODE(4); break;
        case 8: ST_SCAN_MODE(8); break;
        default: ST_SCAN_MODE(16); break;
    }
#undef ST_SCAN_MODE
#undef ST_SCAN
    ST_LAUNCH_CHECK("state_scan");
    return 0;
}

extern "C" int st_gated_group_norm(void* out, const float* o, const void* gate, int64_t gate_stride,
                                   const float* gain, int num_tokens, int groups, int width, int gain_per_group,
                                   int gate_first, float eps, int dtype, hipStream_t stream) {
    ST_CHECK(num_tokens >= 0 && groups > 0 && width > 0, "gated_group_norm: bad sizes");
    ST_CHECK(eps > 0.f, "gated_group_norm: eps must be positive");
    if (num_tokens == 0) return 0;
    ST_CHECK(out && o && gate && gain, "gated_group_norm: null operand");
    ST_CHECK((int64_t)num_tokens * groups <= 0x7fffffff, "gated_group_norm: too many rows");
    const unsigned grid = (unsigned)(num_tokens * groups);
    if (dtype == kF32)
        gated_group_norm_kernel<float><<<grid, 256, 0, stream>>>((float*)out, o, (const float*)gate, gate_stride,
                                                                 gain, groups, width, gain_per_group, gate_first, eps);
    else if (dtype == kBF16)
        gated_group_norm_kernel<bf16_t><<<grid, 256, 0, stream>>>((bf16_t*)out, o, (const bf16_t*)gate, gate_stride,
                                                                  gain, groups, width, gain_per_group, gate_first, eps);
    else ST_CHECK(false, "gated_group_norm: unknown dtype %d", dtype);
    ST_LAUNCH_CHECK("gated_group_norm");
    return 0;
}
