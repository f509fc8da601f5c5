// A short causal convolution over time with one filter a channel, for batches of portions of
// sequences: what lies before a portion's first row comes from the request's state slot, which
// holds the inputs at the last taps - 1 positions.
//
//   y[t, c] = act((x[t, c] if add_input) + bias[c] + sum_{j < taps} w[c, j] * x(position p_t - (taps - 1) + j, c))
//
// The input rows are float or in the storage type, with any row stride (a slice of a product's
// output); the state is float with any stride between slots (a part of a larger state of the
// request).  A row depends on earlier rows of the same launch only through x, which the kernel
// does not write; the state is moved on by a second kernel after all rows have read it.  Sums are float.
#include "api.h"
#include "common.h"
#include "activation.h"

namespace st {

constexpr int kMaxTaps = 8;

template <typename TI, typename TO>
__global__ __launch_bounds__(256) void token_conv_kernel(
    TO* __restrict__ out, const TI* __restrict__ x, int64_t x_stride, const float* __restrict__ w,
    const float* __restrict__ bias, const float* __restrict__ state, int64_t slot_stride,
    const int* __restrict__ token_item, const int* __restrict__ item_tok_off, const int* __restrict__ item_slot,
    int channels, int taps, int add_input, int activation) {
    const int t = blockIdx.x;
    const int c = blockIdx.y * 256 + threadIdx.x;
    if (c >= channels) return;
    const int item = token_item[t];
    const int slot = item >= 0 ? item_slot[item] : -1;
    if (slot < 0) {                                  // a padding row of a batch of fixed size
        Elem<TO>::store(out + (int64_t)t * channels + c, 0.f);
        return;
    }
    const int r = t - item_tok_off[item];            // row within the item's portion
    const int hist = taps - 1;
    const float* st_c = state + (int64_t)slot * slot_stride + c;
    const TI* x_c = x + (int64_t)t * x_stride + c;
    float acc = add_input ? Elem<TI>::load(x_c) : 0.f;
    if (bias) acc += bias[c];
    for (int j = 0; j < taps; ++j) {
        const int back = hist - j;                   // rows back from this one
        const float v = (r - back >= 0) ? Elem<TI>::load(x_c - (int64_t)back * x_stride)
                                        : st_c[(int64_t)(hist + r - back) * channels];
        acc = fmaf(w[(int64_t)c * taps + j], v, acc);
    }
    Elem<TO>::store(out + (int64_t)t * channels + c, apply_activation(activation, acc));
}

// One thread per (item, channel): the new state is the last taps - 1 of (old state, the item's rows).
template <typename TI>
__global__ __launch_bounds__(256) void token_conv_state_kernel(
    float* __restrict__ state, int64_t slot_stride, const TI* __restrict__ x, int64_t x_stride,
    const int* __restrict__ item_len, const int* __restrict__ item_tok_off, const int* __restrict__ item_slot,
    int channels, int taps) {
    const int item = blockIdx.x;
    const int c = blockIdx.y * 256 + threadIdx.x;
    if (c >= channels) return;
    const int slot = item_slot[item], n = item_len[item];
    if (slot < 0 || n <= 0) return;
    const int hist = taps - 1;
    float* st_c = state + (int64_t)slot * slot_stride + c;
    const TI* x_c = x + (int64_t)item_tok_off[item] * x_stride + c;
    float keep[kMaxTaps];
#pragma unroll
    for (int i = 0; i < kMaxTaps; ++i) {
        if (i >= hist) break;
        const int p = n - hist + i;                  // row of the portion, negative: still in the old state
        keep[i] = p >= 0 ? Elem<TI>::load(x_c + (int64_t)p * x_stride) : st_c[(int64_t)(hist + p) * channels];
    }
#pragma unroll
    for (int i = 0; i < kMaxTaps; ++i) {
        if (i >= hist) break;
        st_c[(int64_t)i * channels] = keep[i];
    }
}

}  // namespace st

using namespace st;

extern "C" int st_token_conv(void* out, const void* x, int64_t x_stride, int in_dtype, const float* w,
                             const float* bias, const float* state, int64_t slot_stride, const int* token_item,
                             const int* item_tok_off, const int* item_slot, int num_tokens, int channels, int taps,
                             int add_input, int activation, int out_dtype, hipStream_t stream) {
    ST_CHECK(num_tokens >= 0 && channels > 0, "token_conv: bad sizes T=%d C=%d", num_tokens, channels);
    ST_CHECK(taps >= 1 && taps <= kMaxTaps, "token_conv: 1 to %d taps, not %d", kMaxTaps, taps);
    ST_CHECK(out && x && w && token_item && item_tok_off && item_slot && (state || taps == 1), "token_conv: null operand");
    ST_CHECK(out != x, "token_conv: the result cannot take its input's place");
    ST_CHECK(activation_known(activation), "token_conv: activation %d has no kernel", activation);
    ST_CHECK((in_dtype == kF32 || in_dtype == kBF16) && (out_dtype == kF32 || out_dtype == kBF16),
             "token_conv: unknown dtype %d -> %d", in_dtype, out_dtype);
    if (num_tokens == 0) return 0;
    const dim3 grid(num_tokens, (channels + 255) / 256);
#define ST_CONV(TI, TO)                                                                                      \
    token_conv_kernel<TI, TO><<<grid, 256, 0, stream>>>((TO*)out, (const TI*)x, x_stride, w, bias, state,   \
        slot_stride, token_item, item_tok_off, item_slot, channels, taps, add_input, activation)
    if (in_dtype == kF32 && out_dtype == kF32) ST_CONV(float, float);
    else if (in_dtype == kF32) ST_CONV(float, bf16_t);
    else if (out_dtype == kF32) ST_CONV(bf16_t, float);
    else ST_CONV(bf16_t, bf16_t);
#undef ST_CONV
    ST_LAUNCH_CHECK("token_conv");
    return 0;
}

extern "C" int st_token_conv_state(float* state, int64_t slot_stride, const void* x, int64_t x_stride, int in_dtype,
                                   const int* item_len, const int* item_tok_off, const int* item_slot, int num_items,
                                   int channels, int taps, hipStream_t stream) {
    ST_CHECK(num_items >= 0 && channels > 0, "token_conv_state: bad sizes");
    ST_CHECK(taps >= 1 && taps <= kMaxTaps, "token_conv_state: 1 to %d taps, not %d", kMaxTaps, taps);
    ST_CHECK(in_dtype == kF32 || in_dtype == kBF16, "token_conv_state: unknown dtype %d", in_dtype);
    if (num_items == 0 || taps == 1) return 0;
    ST_CHECK(state && x && item_len && item_tok_off && item_slot, "token_conv_state: null operand");
    const dim3 grid(num_items, (channels + 255) / 256);
    if (in_dtype == kF32)
        token_conv_state_kernel<float><<<grid, 256, 0, stream>>>(state, slot_stride, (const float*)x, x_stride,
                                                                 item_len, item_tok_off, item_slot, channels, taps);
    else
        token_conv_state_kernel<bf16_t><<<grid, 256, 0, stream>>>(state, slot_stride, (const bf16_t*)x, x_stride,
                                                                  item_len, item_tok_off, item_slot, channels, taps);
    ST_LAUNCH_CHECK("token_conv_state");
    return 0;
}
