// A residual stream kept in several copies (hyper-connections): x [tokens][copies][width], float32.
//   xrt_streams_open    every copy of a token starts as the token's embedding row
//   xrt_streams_read    what a sublayer reads: u = sum over the copies s of in[s] * x_s, then u / sqrt(mean(u^2) + eps) * gain in the
//                       element type of the product that follows (gain null: u itself); only `rows` of the tokens, if given
//   xrt_streams_write   what a sublayer y [tokens][width] (float32) leaves: all copies at once from the old ones,
//                       x_t <- sum over s of mix[s][t] * x_s + out[t] * y; and, if asked for, the next sublayer's read of the new
//                       copies in the same pass over the token
// A workgroup a token. Sums over the copies run in the copies' order; all arithmetic is float32.
#include "common.h"
#include "xrt_hip.h"

namespace {

constexpr int STREAM_THREADS = 1024;         // the most threads of a workgroup; rows narrower than 2048 take 256
constexpr int MOST_COPIES = XRT_MOST_STREAMS;

__device__ __forceinline__ float gain_at(const void* p, int dtype, int i) {
    return dtype == XRT_F32 ? ((const float*)p)[i] : to_float(((const bf16*)p)[i]);
}
__device__ __forceinline__ void store_as(void* p, int dtype, long i, float v) {
    if (dtype == XRT_F32) ((float*)p)[i] = v; else ((bf16*)p)[i] = from_float<bf16>(v);
}

__global__ void __launch_bounds__(STREAM_THREADS) streams_open_kernel(const float* __restrict__ x, float* __restrict__ streams, int width, int copies) {
    const long t = blockIdx.x;
    for (int c = threadIdx.x; c < width; c += blockDim.x) {
        const float v = x[t * width + c];
        for (int s = 0; s < copies; ++s) streams[(t * copies + s) * width + c] = v;
    }
}

// the norm of the row u that lies in LDS (squares: this thread's share of the sum of its squares), written to out row `to`
__device__ __forceinline__ void write_normed(const float* u, float squares, int width, const void* gain, int gain_dtype, float eps, void* out,
                                             int out_dtype, long to, float* scratch) {
    if (gain == nullptr) {
        for (int c = threadIdx.x; c < width; c += blockDim.x) store_as(out, out_dtype, to * width + c, u[c]);
        return;
    }
    const float inv = 1.0f / sqrtf(block_sum(squares, scratch) / (float)width + eps);
    for (int c = threadIdx.x; c < width; c += blockDim.x) store_as(out, out_dtype, to * width + c, u[c] * inv * gain_at(gain, gain_dtype, c));
}

__global__ void __launch_bounds__(STREAM_THREADS) streams_read_kernel(const float* __restrict__ streams, int copies, const float* __restrict__ in,
                                                                     const void* __restrict__ gain, int gain_dtype, float eps, void* __restrict__ out,
                                                                     int out_dtype, const int* __restrict__ rows, int width) {
    extern __shared__ float u[];
    __shared__ float scratch[32];
    const long t = rows != nullptr ? rows[blockIdx.x] : blockIdx.x;
    float squares = 0.f;
    for (int c = threadIdx.x; c < width; c += blockDim.x) {
        float sum = 0.f;
        for (int s = 0; s < copies; ++s) sum = fmaf(in[s], streams[(t * copies + s) * width + c], sum);
        u[c] = sum;
        squares = fmaf(sum, sum, squares);
    }
    write_normed(u, squares, width, gain, gain_dtype, eps, out, out_dtype, blockIdx.x, scratch);
}

__global__ void __launch_bounds__(STREAM_THREADS) streams_write_kernel(float* __restrict__ streams, int copies, const float* __restrict__ mix,
                                                                      const float* __restrict__ out_weights, const float* __restrict__ y, int width,
                                                                      const float* __restrict__ next_in, const void* __restrict__ gain, int gain_dtype,
                                                                      float eps, void* __restrict__ normed, int normed_dtype) {
    extern __shared__ float u[];
    __shared__ float scratch[32];
    __shared__ float weights[MOST_COPIES * MOST_COPIES + 2 * MOST_COPIES];
    float* mixes = weights;                                    // [from][to]
    float* outs = weights + MOST_COPIES * MOST_COPIES;
    float* ins = outs + MOST_COPIES;
    for (int i = threadIdx.x; i < copies * copies; i += blockDim.x) mixes[i] = mix[i];
    for (int i = threadIdx.x; i < copies; i += blockDim.x) { outs[i] = out_weights[i]; ins[i] = next_in != nullptr ? next_in[i] : 0.f; }
    __syncthreads();
    const long t = blockIdx.x;
    float squares = 0.f;
    for (int c = threadIdx.x; c < width; c += blockDim.x) {
        float old[MOST_COPIES];
#pragma unroll
        for (int s = 0; s < MOST_COPIES; ++s) old[s] = s < copies ? streams[(t * copies + s) * width + c] : 0.f;
        const float add = y[t * width + c];
        float read = 0.f;
#pragma unroll
        for (int to = 0; to < MOST_COPIES; ++to) {
            if (to < copies) {
                float sum = 0.f;
#pragma unroll
                for (int s = 0; s < MOST_COPIES; ++s)
                    if (s < copies) sum = fmaf(mixes[s * copies + to], old[s], sum);
                sum = fmaf(outs[to], add, sum);
                streams[(t * copies + to) * width + c] = sum;
                read = fmaf(ins[to], sum, read);
            }
        }
        if (next_in != nullptr) {
            u[c] = read;
            squares = fmaf(read, read, squares);
        }
    }
    if (next_in != nullptr) write_normed(u, squares, width, gain, gain_dtype, eps, normed, normed_dtype, t, scratch);
}

int threads_for(int width) { return width >= 2048 ? STREAM_THREADS : 256; }

}  // namespace

extern "C" int xrt_streams_open(const float* x, float* streams, long tokens, int width, int copies, void* stream) {
    XRT_REQUIRE(x && streams && tokens >= 0 && tokens < (1L << 31) && width > 0 && copies > 0 && copies <= MOST_COPIES,
                "streams_open: bad operands (%ld tokens, width %d, %d copies of up to %d)", tokens, width, copies, MOST_COPIES);
    if (tokens == 0) return 0;
    streams_open_kernel<<<(unsigned)tokens, threads_for(width), 0, (hipStream_t)stream>>>(x, streams, width, copies);
    XRT_LAUNCH_CHECK("streams_open");
    return 0;
}

extern "C" int xrt_streams_read(const float* streams, int copies, const float* in, const void* gain, int gain_dtype, float eps, void* out,
                                int out_dtype, const int* rows, long n_rows, int width, void* stream) {
    XRT_REQUIRE(streams && in && out && n_rows >= 0 && n_rows < (1L << 31) && width > 0 && width <= 16384 && copies > 0 && copies <= MOST_COPIES,
                "streams_read: bad operands (%ld rows, width %d of up to 16384, %d copies of up to %d)", n_rows, width, copies, MOST_COPIES);
    XRT_REQUIRE((out_dtype == XRT_F32 || out_dtype == XRT_BF16) && (gain_dtype == XRT_F32 || gain_dtype == XRT_BF16), "streams_read: unknown dtype");
    if (n_rows == 0) return 0;
    streams_read_kernel<<<(unsigned)n_rows, threads_for(width), (size_t)width * sizeof(float), (hipStream_t)stream>>>(streams, copies, in, gain, gain_dtype,
                                                                                                                eps, out, out_dtype, rows, width);
    XRT_LAUNCH_CHECK("streams_read");
    return 0;
}

extern "C" int xrt_streams_write(float* streams, int copies, const float* mix, const float* out_weights, const float* y, long tokens, int width,
                                 const float* next_in, const void* gain, int gain_dtype, float eps, void* normed, int normed_dtype, void* stream) {
    XRT_REQUIRE(streams && mix && out_weights && y && tokens >= 0 && tokens < (1L << 31) && width > 0 && width <= 16384 && copies > 0 &&
                copies <= MOST_COPIES, "streams_write: bad operands (%ld tokens, width %d of up to 16384, %d copies of up to %d)", tokens, width,
                copies, MOST_COPIES);
    XRT_REQUIRE(next_in == nullptr || normed != nullptr, "streams_write: the next sublayer's read needs a place to go");
    XRT_REQUIRE(next_in == nullptr || ((normed_dtype == XRT_F32 || normed_dtype == XRT_BF16) && (gain_dtype == XRT_F32 || gain_dtype == XRT_BF16)),
                "streams_write: unknown dtype");
    if (tokens == 0) return 0;
    streams_write_kernel<<<(unsigned)tokens, threads_for(width), next_in != nullptr ? (size_t)width * sizeof(float) : 0, (hipStream_t)stream>>>(
        streams, copies, mix, out_weights, y, width, next_in, gain, gain_dtype, eps, normed, normed_dtype);
    XRT_LAUNCH_CHECK("streams_write");
    return 0;
}
