// A short causal convolution over time with one filter a channel, for batches of portions of
// sequences: what lies before a portion's first row comes from the request's state slot, which
// holds the inputs at the last taps - 1 positions.
//
//   y[t, c] = (x[t, c] if add_input) + sum_{j < taps} w[c, j] * x(position p_t - (taps - 1) + j, c)
//
// A row depends on earlier rows of the same launch only through x, which the kernel does not
// write; the state is moved on by a second kernel after all rows have read it.  Sums are float.
#include "api.h"
#include "common.h"

namespace st {

constexpr int kMaxTaps = 8;

template <typename TO>
__global__ __launch_bounds__(256) void token_conv_kernel(
    TO* __restrict__ out, const float* __restrict__ x, const float* __restrict__ w,
    const float* __restrict__ state, const int* __restrict__ token_item,
    const int* __restrict__ item_tok_off, const int* __restrict__ item_slot,
    int channels, int taps, int add_input) {
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
    const float* st_c = state + ((int64_t)slot * hist) * channels + c;
    const float* x_c = x + (int64_t)t * channels + c;
    float acc = add_input ? x_c[0] : 0.f;
    for (int j = 0; j < taps; ++j) {
        const int back = hist - j;                   // rows back from this one
        const float v = (r - back >= 0) ? x_c[-(int64_t)back * channels]
                                        : st_c[(int64_t)(hist + r - back) * channels];
        acc = fmaf(w[(int64_t)c * taps + j], v, acc);
    }
    Elem<TO>::store(out + (int64_t)t * channels + c, acc);
}

// One thread per (item, channel): the new state is the last taps - 1 of (old state, the item's rows).
__global__ __launch_bounds__(256) void token_conv_state_kernel(
    float* __restrict__ state, const float* __restrict__ x, const int* __restrict__ item_len,
    const int* __restrict__ item_tok_off, const int* __restrict__ item_slot, int channels, int taps) {
    const int item = blockIdx.x;
    const int c = blockIdx.y * 256 + threadIdx.x;
    if (c >= channels) return;
    const int slot = item_slot[item], n = item_len[item];
    if (slot < 0 || n <= 0) return;
    const int hist = taps - 1;
    float* st_c = state + ((int64_t)slot * hist) * channels + c;
    const float* x_c = x + (int64_t)item_tok_off[item] * channels + c;
    float keep[kMaxTaps];
#pragma unroll
    for (int i = 0; i < kMaxTaps; ++i) {
        if (i >= hist) break;
        const int p = n - hist + i;                  // row of the portion, negative: still in the old state
        keep[i] = p >= 0 ? x_c[(int64_t)p * channels] : st_c[(int64_t)(hist + p) * channels];
    }
#pragma unroll
    for (int i = 0; i < kMaxTaps; ++i) {
        if (i >= hist) break;
        st_c[(int64_t)i * channels] = keep[i];
    }
}

}  // namespace st

using namespace st;

extern "C" int st_token_conv(void* out, const float* x, const float* w, const float* state, const int* token_item,
                             const int* item_tok_off, const int* item_slot, int num_tokens, int channels, int taps,
                             int add_input, int out_dtype, hipStream_t stream) {
    ST_CHECK(num_tokens >= 0 && channels > 0, "token_conv: bad sizes T=%d C=%d", num_tokens, channels);
    ST_CHECK(taps >= 1 && taps <= kMaxTaps, "token_conv: 1 to %d taps, not %d", kMaxTaps, taps);
    ST_CHECK(out && x && w && token_item && item_tok_off && item_slot && (state || taps == 1), "token_conv: null operand");
    ST_CHECK(out != (const void*)x, "token_conv: the result cannot take its input's place");
    if (num_tokens == 0) return 0;
    const dim3 grid(num_tokens, (channels + 255) / 256);
    if (out_dtype == kF32)
        token_conv_kernel<float><<<grid, 256, 0, stream>>>((float*)out, x, w, state, token_item, item_tok_off,
                                                           item_slot, channels, taps, add_input);
    else if (out_dtype == kBF16)
        token_conv_kernel<bf16_t><<<grid, 256, 0, stream>>>((bf16_t*)out, x, w, state, token_item, item_tok_off,
                                                            item_slot, channels, taps, add_input);
    else ST_CHECK(false, "token_conv: unknown dtype %d", out_dtype);
    ST_LAUNCH_CHECK("token_conv");
    return 0;
}

extern "C" int st_token_conv_state(float* state, const float* x, const int* item_len, const int* item_tok_off,
                                   const int* item_slot, int num_items, int channels, int taps, hipStream_t stream) {
    ST_CHECK(num_items >= 0 && channels > 0, "token_conv_state: bad sizes");
    ST_CHECK(taps >= 1 && taps <= kMaxTaps, "token_conv_state: 1 to %d taps, not %d", kMaxTaps, taps);
    if (num_items == 0 || taps == 1) return 0;
    ST_CHECK(state && x && item_len && item_tok_off && item_slot, "token_conv_state: null operand");
    const dim3 grid(num_items, (channels + 255) / 256);
    token_conv_state_kernel<<<grid, 256, 0, stream>>>(state, x, item_len, item_tok_off, item_slot, channels, taps);
    ST_LAUNCH_CHECK("token_conv_state");
    return 0;
}
