// A host program with no Python and no torch in it: allocates with the HIP runtime, calls every entry point of the
// portable payload format and of the CUDA extension's byte format through the C ABI of include/lbc.h on a stream of
// its own, and compares every byte with the scalar C oracles (oracle/codec_scalar.c, oracle/cuda_wire_scalar.c,
// oracle/cuda_wire_general_scalar.c, linked from oracle/_build).  Built by __graft_entry__.build(), run by
// tests/test_abi_client.py on the GPU box.  Prints "OK <checks>" or the first mismatch.
// `abi_client ring-host-cost` instead measures what the calls of one rank's ring schedule cost a native caller: the
// host time of 15 consecutive lbc_ring_step calls (the launches of a W=8 ring on one 200 MiB fp32 bucket) and the time
// the device takes for them back to back - the floor under any submission loop written above this ABI.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>

#include <chrono>
#include <vector>

#include "../../include/lbc.h"

extern "C" {
void lbo_quantize_f32(const float *x, int64_t n, int group_size, int8_t *codes, float *scales);
void lbo_dequantize_f32(const int8_t *codes, const float *scales, int64_t n, int group_size, float *out);
void lbo_reduce_f32(const int8_t *const *codes, const float *const *scales, int world, int64_t n, int group_size,
                    float divisor, float *out);
void lbo_ef_step_f32(const float *grad, const float *residual_in, int64_t n, int group_size, int8_t *codes, float *scales,
                     float *residual_out, float *restored_out);
// the byte format of the reference's CUDA extension (oracle/cuda_wire_scalar.c, oracle/cuda_wire_general_scalar.c)
void lbw_quantize(const void *x, const void *residual, int dtype, int64_t numel, int g, int compact, int bit, uint8_t *payload);
void lbw_dequantize(const uint8_t *payload, int64_t numel, int g, int compact, int dtype, int op, int bit, void *out);
void lbw_reduce(const uint8_t *const *payloads, int world, int64_t numel, int g, int compact, int dtype, float inv_divisor,
                int use_fma, const void *prepared, void *out, void *residual);
void lbg_quantize(const void *x, int dtype, int64_t numel, int g, int bit, int kind, int topk, int stochastic, uint64_t seed,
                  uint64_t offset, int compact, uint8_t *payload);
void lbg_dequantize(const uint8_t *payload, int64_t numel, int g, int bit, int kind, int topk, int compact, int dtype, int op,
                    void *out);
}

#define HIP_OK(call)                                                                       \
    do {                                                                                   \
        hipError_t status_ = (call);                                                       \
        if (status_ != hipSuccess) {                                                       \
            printf("FAIL %s: %s\n", #call, hipGetErrorString(status_));                    \
            return 2;                                                                      \
        }                                                                                  \
    } while (0)

#define LBC_OK_OR_FAIL(call)                                                               \
    do {                                                                                   \
        int status_ = (call);                                                              \
        if (status_ != LBC_OK) {                                                           \
            printf("FAIL %s -> %d: %s\n", #call, status_, lbc_last_error());               \
            return 3;                                                                      \
        }                                                                                  \
    } while (0)

static uint32_t lcg(uint32_t &state) {
    state = state * 1664525u + 1013904223u;
    return state;
}

// roughly normal values of standard deviation `sigma` (sum of four uniforms), with a few large outliers
static void fill(std::vector<float> &x, uint32_t seed, float sigma) {
    uint32_t s = seed;
    for (size_t i = 0; i < x.size(); ++i) {
        float u = 0.0f;
        for (int k = 0; k < 4; ++k) u += static_cast<float>(lcg(s) >> 8) * (1.0f / 16777216.0f) - 0.5f;
        x[i] = u * 1.7320508f * sigma;
        if ((lcg(s) & 1023u) == 0u) x[i] *= 100.0f;
    }
}

static uint16_t to_bf16(float f) {   // round to nearest even; the inputs here are finite
    uint32_t bits;
    memcpy(&bits, &f, 4);
    return static_cast<uint16_t>((bits + 0x7FFFu + ((bits >> 16) & 1u)) >> 16);
}

// Every entry point of the CUDA extension's byte format, on whole groups, against its scalar C restatement.
static int wire_format_checks(hipStream_t stream, long &checks) {
    const int world = 4, g = 64;
    const int64_t n = 64 * 4 * 750;   // whole groups, whole shards
    std::vector<std::vector<float>> x(world, std::vector<float>(n));
    for (int r = 0; r < world; ++r) fill(x[r], 4321u + 31u * r, 2e-3f * (r + 1));
    std::vector<uint16_t> half(n);
    for (int64_t i = 0; i < n; ++i) half[i] = to_bf16(x[0][i]);
    void *d_x = nullptr, *d_out = nullptr;
    HIP_OK(hipMalloc(&d_x, n * sizeof(float)));
    HIP_OK(hipMalloc(&d_out, n * sizeof(float)));
    const int64_t room = n + n / g * 16 + 256;   // the largest payload here: 8-bit codes and four fp32 words a group
    std::vector<uint8_t *> d_payload(world, nullptr);
    for (int r = 0; r < world; ++r) HIP_OK(hipMalloc(&d_payload[r], room));
    std::vector<uint8_t> got(room), want(room);
    std::vector<float> out(n), want_out(n);

    // quantize + pack and decode: fp32 and bf16, interleaved and appended scales, 8 and 4 bits
    for (int dtype : {LBC_F32, LBC_BF16}) {
        const void *host = dtype == LBC_F32 ? static_cast<const void *>(x[0].data()) : static_cast<const void *>(half.data());
        const size_t item = dtype == LBC_F32 ? 4 : 2;
        HIP_OK(hipMemcpyAsync(d_x, host, n * item, hipMemcpyHostToDevice, stream));
        for (int compact : {1, 0}) {
            for (int bit : {8, 4}) {
                const int64_t bytes = lbc_wire_payload_nbytes(n, g, dtype, bit);
                if (bytes <= 0 || bytes > room) {
                    printf("FAIL payload size %lld\n", static_cast<long long>(bytes));
                    return 20;
                }
                LBC_OK_OR_FAIL(lbc_wire_quant_pack(d_x, nullptr, dtype, n, g, bit, compact, d_payload[0], LBC_ACCESS_AUTO, stream));
                LBC_OK_OR_FAIL(lbc_wire_dequant(d_payload[0], n, g, bit, compact, d_out, dtype, LBC_REDUCE_NONE, LBC_ACCESS_AUTO, stream));
                HIP_OK(hipMemcpyAsync(got.data(), d_payload[0], bytes, hipMemcpyDeviceToHost, stream));
                HIP_OK(hipMemcpyAsync(out.data(), d_out, n * item, hipMemcpyDeviceToHost, stream));
                HIP_OK(hipStreamSynchronize(stream));
                lbw_quantize(host, nullptr, dtype, n, g, compact, bit, want.data());
                lbw_dequantize(want.data(), n, g, compact, dtype, 0, bit, want_out.data());
                if (memcmp(got.data(), want.data(), bytes) != 0 || memcmp(out.data(), want_out.data(), n * item) != 0) {
                    printf("FAIL wire format: dtype %d compact %d bit %d differs from the oracle\n", dtype, compact, bit);
                    return 21;
                }
                checks += 2;
            }
        }
    }

    // the payloads of four ranks (fp32, interleaved scales), their fused mean, and one ring step on them
    const int64_t bytes = lbc_wire_payload_nbytes(n, g, LBC_F32, 8);
    std::vector<std::vector<uint8_t>> host_payload(world, std::vector<uint8_t>(bytes));
    std::vector<const uint8_t *> d_ptrs(world), h_ptrs(world);
    for (int r = 0; r < world; ++r) {
        HIP_OK(hipMemcpyAsync(d_x, x[r].data(), n * sizeof(float), hipMemcpyHostToDevice, stream));
        LBC_OK_OR_FAIL(lbc_wire_quant_pack(d_x, nullptr, LBC_F32, n, g, 8, 1, d_payload[r], LBC_ACCESS_AUTO, stream));
        HIP_OK(hipStreamSynchronize(stream));
        lbw_quantize(x[r].data(), nullptr, LBC_F32, n, g, 1, 8, host_payload[r].data());
        d_ptrs[r] = d_payload[r];
        h_ptrs[r] = host_payload[r].data();
    }
    LBC_OK_OR_FAIL(lbc_wire_dequant_reduce(d_ptrs.data(), world, n, g, 1, 0.25f, 1, d_out, LBC_F32, nullptr, nullptr,
                                           LBC_ACCESS_AUTO, stream));
    HIP_OK(hipMemcpyAsync(out.data(), d_out, n * sizeof(float), hipMemcpyDeviceToHost, stream));
    HIP_OK(hipStreamSynchronize(stream));
    lbw_reduce(h_ptrs.data(), world, n, g, 1, LBC_F32, 0.25f, 1, nullptr, want_out.data(), nullptr);
    if (memcmp(out.data(), want_out.data(), n * sizeof(float)) != 0) {
        printf("FAIL wire format: fused mean differs from the oracle\n");
        return 22;
    }
    ++checks;
    uint8_t *d_send = nullptr;
    HIP_OK(hipMalloc(&d_send, room));
    HIP_OK(hipMemcpyAsync(d_out, x[0].data(), n * sizeof(float), hipMemcpyHostToDevice, stream));
    LBC_OK_OR_FAIL(lbc_wire_ring_step(d_payload[1], d_out, LBC_F32, n, g, 1, LBC_REDUCE_SUM, 1.0f, d_send, LBC_ACCESS_AUTO, stream));
    HIP_OK(hipMemcpyAsync(out.data(), d_out, n * sizeof(float), hipMemcpyDeviceToHost, stream));
    HIP_OK(hipMemcpyAsync(got.data(), d_send, bytes, hipMemcpyDeviceToHost, stream));
    HIP_OK(hipStreamSynchronize(stream));
    want_out = x[0];
    lbw_dequantize(host_payload[1].data(), n, g, 1, LBC_F32, 1, 8, want_out.data());
    lbw_quantize(want_out.data(), nullptr, LBC_F32, n, g, 1, 8, want.data());
    if (memcmp(out.data(), want_out.data(), n * sizeof(float)) != 0 || memcmp(got.data(), want.data(), bytes) != 0) {
        printf("FAIL wire format: ring step differs from the oracle\n");
        return 23;
    }
    checks += 2;

    // the bucket as four chunks in one launch, and the chunks decoded back in one launch
    const int64_t shard = n / world, shard_bytes = lbc_wire_payload_nbytes(shard, g, LBC_F32, 8);
    const int64_t stride = (shard_bytes + 255) / 256 * 256;
    uint8_t *d_rows = nullptr;
    HIP_OK(hipMalloc(&d_rows, world * stride));
    HIP_OK(hipMemcpyAsync(d_x, x[0].data(), n * sizeof(float), hipMemcpyHostToDevice, stream));
    LBC_OK_OR_FAIL(lbc_wire_quant_pack_chunks(d_x, nullptr, LBC_F32, n, world, g, 8, 1, d_rows, stride, LBC_ACCESS_AUTO, stream));
    LBC_OK_OR_FAIL(lbc_wire_dequant_chunks(d_rows, stride, world, shard, n, g, 8, 1, d_out, LBC_F32, LBC_REDUCE_NONE,
                                           LBC_ACCESS_AUTO, stream));
    std::vector<uint8_t> rows(world * stride);
    HIP_OK(hipMemcpyAsync(rows.data(), d_rows, world * stride, hipMemcpyDeviceToHost, stream));
    HIP_OK(hipMemcpyAsync(out.data(), d_out, n * sizeof(float), hipMemcpyDeviceToHost, stream));
    HIP_OK(hipStreamSynchronize(stream));
    for (int d = 0; d < world; ++d) {
        lbw_quantize(x[0].data() + d * shard, nullptr, LBC_F32, shard, g, 1, 8, want.data());
        lbw_dequantize(want.data(), shard, g, 1, LBC_F32, 0, 8, want_out.data() + d * shard);
        if (memcmp(rows.data() + d * stride, want.data(), shard_bytes) != 0) {
            printf("FAIL wire format: payload of chunk %d differs from the oracle\n", d);
            return 24;
        }
    }
    if (memcmp(out.data(), want_out.data(), n * sizeof(float)) != 0) {
        printf("FAIL wire format: decoded chunks differ from the oracle\n");
        return 24;
    }
    checks += 2;

    // the general policies: two outliers, stochastic rounding, a code book
    struct Policy { int dtype, bit, kind, topk, stochastic; };
    const Policy policies[] = {{LBC_F32, 8, LBC_QUANT_LINEAR, 2, 0}, {LBC_F32, 8, LBC_QUANT_LINEAR, 0, 1},
                               {LBC_BF16, 4, LBC_QUANT_NORMAL, 0, 0}, {LBC_BF16, 4, LBC_QUANT_E2M1, 1, 1}};
    for (const Policy &p : policies) {
        const void *host = p.dtype == LBC_F32 ? static_cast<const void *>(x[0].data()) : static_cast<const void *>(half.data());
        const size_t item = p.dtype == LBC_F32 ? 4 : 2;
        const uint64_t seed = 0x1234567887654321ULL, offset = 12;
        const int64_t size = lbc_wire_general_payload_nbytes(n, g, p.dtype, p.bit, p.topk);
        if (size <= 0 || size > room) {
            printf("FAIL general payload size %lld\n", static_cast<long long>(size));
            return 25;
        }
        HIP_OK(hipMemcpyAsync(d_x, host, n * item, hipMemcpyHostToDevice, stream));
        LBC_OK_OR_FAIL(lbc_wire_quant_general(d_x, p.dtype, n, g, p.bit, p.kind, p.topk, p.stochastic, seed, offset, 1,
                                              d_payload[0], stream));
        LBC_OK_OR_FAIL(lbc_wire_dequant_general(d_payload[0], n, g, p.bit, p.kind, p.topk, 1, d_out, p.dtype, LBC_REDUCE_NONE, stream));
        HIP_OK(hipMemcpyAsync(got.data(), d_payload[0], size, hipMemcpyDeviceToHost, stream));
        HIP_OK(hipMemcpyAsync(out.data(), d_out, n * item, hipMemcpyDeviceToHost, stream));
        HIP_OK(hipStreamSynchronize(stream));
        lbg_quantize(host, p.dtype, n, g, p.bit, p.kind, p.topk, p.stochastic, seed, offset, 1, want.data());
        lbg_dequantize(want.data(), n, g, p.bit, p.kind, p.topk, 1, p.dtype, 0, want_out.data());
        if (memcmp(got.data(), want.data(), size) != 0 || memcmp(out.data(), want_out.data(), n * item) != 0) {
            printf("FAIL wire format: policy (dtype %d, %d bit, kind %d, top-%d, stochastic %d) differs from the oracle\n", p.dtype,
                   p.bit, p.kind, p.topk, p.stochastic);
            return 26;
        }
        checks += 2;
    }
    return 0;
}

static int ring_host_cost() {
    const int64_t n = 6553600, groups = n / 64;   // a 200 MiB fp32 bucket over 8 ranks
    const int buckets = 12, launches = 15;
    int8_t *recv_codes, *send_codes;
    float *recv_scales, *send_scales, *chunk;
    hipStream_t stream;
    HIP_OK(hipStreamCreate(&stream));
    HIP_OK(hipMalloc(&recv_codes, n));
    HIP_OK(hipMalloc(&send_codes, n));
    HIP_OK(hipMalloc(&recv_scales, groups * sizeof(float)));
    HIP_OK(hipMalloc(&send_scales, groups * sizeof(float)));
    HIP_OK(hipMalloc(&chunk, n * sizeof(float)));
    HIP_OK(hipMemset(recv_codes, 1, n));
    HIP_OK(hipMemset(recv_scales, 0, groups * sizeof(float)));
    HIP_OK(hipMemset(chunk, 0, n * sizeof(float)));
    for (int rep = 0; rep < 5; ++rep) {           // the first repetition warms up
        const auto begin = std::chrono::steady_clock::now();
        for (int i = 0; i < buckets * launches; ++i)
            LBC_OK_OR_FAIL(lbc_ring_step(recv_codes, recv_scales, chunk, LBC_F32, n, 64, LBC_REDUCE_SUM, 1.0f, send_codes,
                                         send_scales, LBC_ACCESS_AUTO, stream));
        const auto enqueued = std::chrono::steady_clock::now();
        HIP_OK(hipStreamSynchronize(stream));
        const auto done = std::chrono::steady_clock::now();
        if (rep > 0)
            printf("%d calls of lbc_ring_step (6,553,600 fp32): host %.1f us (%.2f us a call), device %.1f us\n", launches,
                   std::chrono::duration<double, std::micro>(enqueued - begin).count() / buckets,
                   std::chrono::duration<double, std::micro>(enqueued - begin).count() / (buckets * launches),
                   std::chrono::duration<double, std::micro>(done - begin).count() / buckets);
    }
    return 0;
}

int main(int argc, char **argv) {
    if (argc > 1 && strcmp(argv[1], "ring-host-cost") == 0) return ring_host_cost();
    if (lbc_abi_version() != LBC_ABI_VERSION) {
        printf("FAIL abi version %d, header %d\n", lbc_abi_version(), LBC_ABI_VERSION);
        return 1;
    }
    const int world = 4, g = 64;
    const int64_t n = 64 * 3000 + 37;   // ragged tail
    const int64_t groups = (n + g - 1) / g, padded = groups * g;
    hipStream_t stream;
    HIP_OK(hipStreamCreate(&stream));

    std::vector<std::vector<float>> x(world, std::vector<float>(n));
    std::vector<std::vector<int8_t>> want_codes(world, std::vector<int8_t>(padded));
    std::vector<std::vector<float>> want_scales(world, std::vector<float>(groups));
    float *d_x = nullptr, *d_out = nullptr;
    std::vector<int8_t *> d_codes(world, nullptr);
    std::vector<float *> d_scales(world, nullptr);
    HIP_OK(hipMalloc(&d_x, n * sizeof(float)));
    HIP_OK(hipMalloc(&d_out, n * sizeof(float)));
    long checks = 0;
    for (int r = 0; r < world; ++r) {
        fill(x[r], 1234u + 17u * r, 1e-3f * (r + 1));
        lbo_quantize_f32(x[r].data(), n, g, want_codes[r].data(), want_scales[r].data());
        HIP_OK(hipMalloc(&d_codes[r], padded));
        HIP_OK(hipMalloc(&d_scales[r], groups * sizeof(float)));
        HIP_OK(hipMemcpyAsync(d_x, x[r].data(), n * sizeof(float), hipMemcpyHostToDevice, stream));
        LBC_OK_OR_FAIL(lbc_quant_pack(d_x, LBC_F32, nullptr, LBC_NONE, n, g, d_codes[r], d_scales[r], nullptr, LBC_NONE,
                                      nullptr, LBC_NONE, nullptr, LBC_NONE, LBC_ACCESS_AUTO, stream));
        std::vector<int8_t> codes(padded);
        std::vector<float> scales(groups);
        HIP_OK(hipMemcpyAsync(codes.data(), d_codes[r], padded, hipMemcpyDeviceToHost, stream));
        HIP_OK(hipMemcpyAsync(scales.data(), d_scales[r], groups * sizeof(float), hipMemcpyDeviceToHost, stream));
        HIP_OK(hipStreamSynchronize(stream));
        if (memcmp(codes.data(), want_codes[r].data(), padded) != 0) {
            printf("FAIL codes of payload %d differ from the oracle\n", r);
            return 4;
        }
        if (memcmp(scales.data(), want_scales[r].data(), groups * sizeof(float)) != 0) {
            printf("FAIL scales of payload %d differ from the oracle\n", r);
            return 4;
        }
        checks += 2;
    }

    // fused dequant-reduce (mean) of the four payloads, fixed rank order
    std::vector<const int8_t *> code_ptrs(d_codes.begin(), d_codes.end());
    std::vector<const float *> scale_ptrs(d_scales.begin(), d_scales.end());
    LBC_OK_OR_FAIL(lbc_dequant_reduce(code_ptrs.data(), scale_ptrs.data(), world, n, g, static_cast<float>(world), d_out,
                                      LBC_F32, nullptr, nullptr, LBC_ACCESS_CACHED, stream));
    std::vector<float> got(n), want(n);
    HIP_OK(hipMemcpyAsync(got.data(), d_out, n * sizeof(float), hipMemcpyDeviceToHost, stream));
    HIP_OK(hipStreamSynchronize(stream));
    std::vector<const int8_t *> host_codes(world);
    std::vector<const float *> host_scales(world);
    for (int r = 0; r < world; ++r) {
        host_codes[r] = want_codes[r].data();
        host_scales[r] = want_scales[r].data();
    }
    lbo_reduce_f32(host_codes.data(), host_scales.data(), world, n, g, static_cast<float>(world), want.data());
    if (memcmp(got.data(), want.data(), n * sizeof(float)) != 0) {
        printf("FAIL reduced mean differs from the oracle\n");
        return 5;
    }
    ++checks;

    // one ring step: out += decode(payload 1), then quantize the sum; against decode + add + quantize on the host
    std::vector<float> chunk(x[0]);
    HIP_OK(hipMemcpyAsync(d_out, chunk.data(), n * sizeof(float), hipMemcpyHostToDevice, stream));
    int8_t *d_send_codes = nullptr;
    float *d_send_scales = nullptr;
    HIP_OK(hipMalloc(&d_send_codes, padded));
    HIP_OK(hipMalloc(&d_send_scales, groups * sizeof(float)));
    LBC_OK_OR_FAIL(lbc_ring_step(d_codes[1], d_scales[1], d_out, LBC_F32, n, g, LBC_REDUCE_SUM, 1.0f, d_send_codes,
                                 d_send_scales, LBC_ACCESS_STREAM, stream));
    std::vector<int8_t> send_codes(padded), want_send_codes(padded);
    std::vector<float> send_scales(groups), want_send_scales(groups);
    HIP_OK(hipMemcpyAsync(got.data(), d_out, n * sizeof(float), hipMemcpyDeviceToHost, stream));
    HIP_OK(hipMemcpyAsync(send_codes.data(), d_send_codes, padded, hipMemcpyDeviceToHost, stream));
    HIP_OK(hipMemcpyAsync(send_scales.data(), d_send_scales, groups * sizeof(float), hipMemcpyDeviceToHost, stream));
    HIP_OK(hipStreamSynchronize(stream));
    for (int64_t i = 0; i < n; ++i) {
        volatile float decoded = static_cast<float>(want_codes[1][i]) * want_scales[1][i / g];
        want[i] = chunk[i] + decoded;
    }
    lbo_quantize_f32(want.data(), n, g, want_send_codes.data(), want_send_scales.data());
    if (memcmp(got.data(), want.data(), n * sizeof(float)) != 0 || memcmp(send_codes.data(), want_send_codes.data(), padded) != 0 ||
        memcmp(send_scales.data(), want_send_scales.data(), groups * sizeof(float)) != 0) {
        printf("FAIL ring step differs from the oracle\n");
        return 6;
    }
    checks += 3;

    // decode of one payload
    LBC_OK_OR_FAIL(lbc_dequant(d_codes[0], d_scales[0], n, g, d_out, LBC_F32, LBC_REDUCE_NONE, LBC_ACCESS_AUTO, stream));
    HIP_OK(hipMemcpyAsync(got.data(), d_out, n * sizeof(float), hipMemcpyDeviceToHost, stream));
    HIP_OK(hipStreamSynchronize(stream));
    lbo_dequantize_f32(want_codes[0].data(), want_scales[0].data(), n, g, want.data());
    if (memcmp(got.data(), want.data(), n * sizeof(float)) != 0) {
        printf("FAIL decoded payload differs from the oracle\n");
        return 8;
    }
    ++checks;

    // error-feedback step: quantize x + residual, residual updated in place, the decoded value as a second output;
    // then the same residual once more from lbc_ef_update
    std::vector<float> residual(n), want_residual(n), want_restored(n), prepared(n);
    fill(residual, 99u, 1e-5f);
    for (int64_t i = 0; i < n; ++i) {
        volatile float sum = x[0][i] + residual[i];
        prepared[i] = sum;
    }
    std::vector<int8_t> ef_codes(padded), want_ef_codes(padded);
    std::vector<float> ef_scales(groups), want_ef_scales(groups);
    lbo_ef_step_f32(x[0].data(), residual.data(), n, g, want_ef_codes.data(), want_ef_scales.data(), want_residual.data(),
                    want_restored.data());
    float *d_residual = nullptr, *d_restored = nullptr, *d_prepared = nullptr, *d_prepared_out = nullptr;
    HIP_OK(hipMalloc(&d_residual, n * sizeof(float)));
    HIP_OK(hipMalloc(&d_restored, n * sizeof(float)));
    HIP_OK(hipMalloc(&d_prepared, n * sizeof(float)));
    HIP_OK(hipMalloc(&d_prepared_out, n * sizeof(float)));
    HIP_OK(hipMemcpyAsync(d_x, x[0].data(), n * sizeof(float), hipMemcpyHostToDevice, stream));
    HIP_OK(hipMemcpyAsync(d_residual, residual.data(), n * sizeof(float), hipMemcpyHostToDevice, stream));
    HIP_OK(hipMemcpyAsync(d_prepared, prepared.data(), n * sizeof(float), hipMemcpyHostToDevice, stream));
    LBC_OK_OR_FAIL(lbc_quant_pack(d_x, LBC_F32, d_residual, LBC_F32, n, g, d_send_codes, d_send_scales, d_residual, LBC_F32,
                                  d_restored, LBC_F32, d_prepared_out, LBC_F32, LBC_ACCESS_AUTO, stream));
    std::vector<float> got_residual(n), got_restored(n), got_prepared(n);
    HIP_OK(hipMemcpyAsync(got_prepared.data(), d_prepared_out, n * sizeof(float), hipMemcpyDeviceToHost, stream));
    HIP_OK(hipMemcpyAsync(ef_codes.data(), d_send_codes, padded, hipMemcpyDeviceToHost, stream));
    HIP_OK(hipMemcpyAsync(ef_scales.data(), d_send_scales, groups * sizeof(float), hipMemcpyDeviceToHost, stream));
    HIP_OK(hipMemcpyAsync(got_residual.data(), d_residual, n * sizeof(float), hipMemcpyDeviceToHost, stream));
    HIP_OK(hipMemcpyAsync(got_restored.data(), d_restored, n * sizeof(float), hipMemcpyDeviceToHost, stream));
    HIP_OK(hipStreamSynchronize(stream));
    if (memcmp(ef_codes.data(), want_ef_codes.data(), padded) != 0 ||
        memcmp(ef_scales.data(), want_ef_scales.data(), groups * sizeof(float)) != 0 ||
        memcmp(got_residual.data(), want_residual.data(), n * sizeof(float)) != 0 ||
        memcmp(got_restored.data(), want_restored.data(), n * sizeof(float)) != 0 ||
        memcmp(got_prepared.data(), prepared.data(), n * sizeof(float)) != 0) {
        printf("FAIL error-feedback step differs from the oracle\n");
        return 9;
    }
    checks += 5;
    LBC_OK_OR_FAIL(lbc_ef_update(d_prepared, LBC_F32, d_restored, LBC_F32, d_residual, LBC_F32, n, LBC_ACCESS_AUTO, stream));
    HIP_OK(hipMemcpyAsync(got_residual.data(), d_residual, n * sizeof(float), hipMemcpyDeviceToHost, stream));
    HIP_OK(hipStreamSynchronize(stream));
    if (memcmp(got_residual.data(), want_residual.data(), n * sizeof(float)) != 0) {
        printf("FAIL residual update differs from the oracle\n");
        return 9;
    }
    ++checks;

    // the bucket as `world` chunks in one launch, and the chunks decoded back in one launch
    const int64_t shard = (n + world - 1) / world, shard_groups = (shard + g - 1) / g, shard_padded = shard_groups * g;
    const int64_t stride = (shard_padded + shard_groups * 4 + 255) / 256 * 256;
    uint8_t *d_rows = nullptr;
    HIP_OK(hipMalloc(&d_rows, world * stride));
    HIP_OK(hipMemsetAsync(d_rows, 0xEE, world * stride, stream));
    LBC_OK_OR_FAIL(lbc_quant_pack_chunks(d_x, LBC_F32, nullptr, LBC_NONE, n, world, g, d_rows, stride, nullptr, LBC_NONE, nullptr,
                                         LBC_NONE, nullptr, LBC_NONE, LBC_ACCESS_AUTO, stream));
    LBC_OK_OR_FAIL(lbc_dequant_chunks(d_rows, stride, world, shard, n, g, d_out, LBC_F32, LBC_ACCESS_AUTO, stream));
    std::vector<uint8_t> rows(world * stride);
    HIP_OK(hipMemcpyAsync(rows.data(), d_rows, world * stride, hipMemcpyDeviceToHost, stream));
    HIP_OK(hipMemcpyAsync(got.data(), d_out, n * sizeof(float), hipMemcpyDeviceToHost, stream));
    HIP_OK(hipStreamSynchronize(stream));
    std::vector<std::vector<int8_t>> chunk_codes(world, std::vector<int8_t>(shard_padded));
    std::vector<std::vector<float>> chunk_scales(world, std::vector<float>(shard_groups));
    for (int d = 0; d < world; ++d) {
        std::vector<float> piece(shard, 0.0f);   // the bucket counts as zero padded to world * shard
        for (int64_t i = 0; i < shard && d * shard + i < n; ++i) piece[i] = x[0][d * shard + i];
        lbo_quantize_f32(piece.data(), shard, g, chunk_codes[d].data(), chunk_scales[d].data());
        if (memcmp(rows.data() + d * stride, chunk_codes[d].data(), shard_padded) != 0 ||
            memcmp(rows.data() + d * stride + shard_padded, chunk_scales[d].data(), shard_groups * sizeof(float)) != 0) {
            printf("FAIL payload of chunk %d differs from the oracle\n", d);
            return 10;
        }
        std::vector<float> decoded(shard);
        lbo_dequantize_f32(chunk_codes[d].data(), chunk_scales[d].data(), shard, g, decoded.data());
        for (int64_t i = 0; i < shard && d * shard + i < n; ++i) want[d * shard + i] = decoded[i];
        ++checks;
    }
    if (memcmp(got.data(), want.data(), n * sizeof(float)) != 0) {
        printf("FAIL decoded chunks differ from the oracle\n");
        return 10;
    }
    ++checks;

    // reduce (mean) and requantize in one launch: the payload of quantize(reduce(payloads))
    LBC_OK_OR_FAIL(lbc_dequant_reduce_quant(code_ptrs.data(), scale_ptrs.data(), world, n, g, static_cast<float>(world), LBC_F32,
                                            d_send_codes, d_send_scales, LBC_ACCESS_AUTO, stream));
    HIP_OK(hipMemcpyAsync(send_codes.data(), d_send_codes, padded, hipMemcpyDeviceToHost, stream));
    HIP_OK(hipMemcpyAsync(send_scales.data(), d_send_scales, groups * sizeof(float), hipMemcpyDeviceToHost, stream));
    HIP_OK(hipStreamSynchronize(stream));
    lbo_reduce_f32(host_codes.data(), host_scales.data(), world, n, g, static_cast<float>(world), want.data());
    lbo_quantize_f32(want.data(), n, g, want_send_codes.data(), want_send_scales.data());
    if (memcmp(send_codes.data(), want_send_codes.data(), padded) != 0 ||
        memcmp(send_scales.data(), want_send_scales.data(), groups * sizeof(float)) != 0) {
        printf("FAIL reduce + requantize differs from the oracle\n");
        return 11;
    }
    checks += 2;

    // quantize of one bucket (as chunks) and reduce of another bucket's payloads in one launch
    const int64_t even = 64 * world * 40, even_shard = even / world, even_groups = even_shard / g;
    const int64_t even_stride = (even_shard + even_groups * 4 + 255) / 256 * 256, reduce_n = 64 * 100;
    HIP_OK(hipMemsetAsync(d_rows, 0xEE, world * stride, stream));
    LBC_OK_OR_FAIL(lbc_quant_pack_chunks_and_dequant_reduce(d_x, LBC_F32, nullptr, LBC_NONE, even, world, g, d_rows, even_stride,
                                                            nullptr, LBC_NONE, code_ptrs.data(), scale_ptrs.data(), world, reduce_n,
                                                            static_cast<float>(world), d_out, LBC_F32, nullptr, nullptr,
                                                            LBC_ACCESS_AUTO, stream));
    HIP_OK(hipMemcpyAsync(rows.data(), d_rows, world * even_stride, hipMemcpyDeviceToHost, stream));
    HIP_OK(hipMemcpyAsync(got.data(), d_out, reduce_n * sizeof(float), hipMemcpyDeviceToHost, stream));
    HIP_OK(hipStreamSynchronize(stream));
    for (int d = 0; d < world; ++d) {
        lbo_quantize_f32(x[0].data() + d * even_shard, even_shard, g, chunk_codes[d].data(), chunk_scales[d].data());
        if (memcmp(rows.data() + d * even_stride, chunk_codes[d].data(), even_shard) != 0 ||
            memcmp(rows.data() + d * even_stride + even_shard, chunk_scales[d].data(), even_groups * sizeof(float)) != 0) {
            printf("FAIL shared launch: payload of chunk %d differs from the oracle\n", d);
            return 12;
        }
    }
    lbo_reduce_f32(host_codes.data(), host_scales.data(), world, reduce_n, g, static_cast<float>(world), want.data());
    if (memcmp(got.data(), want.data(), reduce_n * sizeof(float)) != 0) {
        printf("FAIL shared launch: reduced shard differs from the oracle\n");
        return 12;
    }
    checks += 2;

    // three stages of a bucket stream in one launch: chunked quantize of one bucket, reduce + requantize of the payloads
    // that arrived for another, decode of a third one's gathered shard payloads
    uint8_t *d_gathered = nullptr;
    float *d_decoded = nullptr;
    HIP_OK(hipMalloc(&d_gathered, world * even_stride));
    HIP_OK(hipMalloc(&d_decoded, even * sizeof(float)));
    HIP_OK(hipMemcpyAsync(d_gathered, d_rows, world * even_stride, hipMemcpyDeviceToDevice, stream));   // verified above
    HIP_OK(hipMemsetAsync(d_rows, 0xEE, world * even_stride, stream));
    HIP_OK(hipMemsetAsync(d_send_codes, 0xEE, padded, stream));
    {
        lbc_quant_chunks_stage quant_stage{};
        quant_stage.x = d_x;
        quant_stage.x_dtype = LBC_F32;
        quant_stage.residual_dtype = quant_stage.new_residual_dtype = LBC_NONE;
        quant_stage.numel = even;
        quant_stage.world = world;
        quant_stage.payloads = d_rows;
        quant_stage.payload_stride = even_stride;
        lbc_reduce_quant_stage reduce_stage{};
        reduce_stage.codes = code_ptrs.data();
        reduce_stage.scales = scale_ptrs.data();
        reduce_stage.world = world;
        reduce_stage.numel = reduce_n;
        reduce_stage.divisor = static_cast<float>(world);
        reduce_stage.mid_dtype = LBC_F32;
        reduce_stage.out_codes = d_send_codes;
        reduce_stage.out_scales = d_send_scales;
        lbc_dequant_chunks_stage decode_stage{};
        decode_stage.payloads = d_gathered;
        decode_stage.payload_stride = even_stride;
        decode_stage.world = world;
        decode_stage.shard_numel = even_shard;
        decode_stage.total_numel = even;
        decode_stage.out = d_decoded;
        decode_stage.out_dtype = LBC_F32;
        LBC_OK_OR_FAIL(lbc_bucket_pipeline_step(&quant_stage, &reduce_stage, &decode_stage, g, LBC_ACCESS_AUTO, stream));
        // a decode into the tensor the quantize reads: the stages of one launch are not ordered, so this is refused
        lbc_dequant_chunks_stage clash = decode_stage;
        clash.out = d_x;
        if (lbc_bucket_pipeline_step(&quant_stage, nullptr, &clash, g, LBC_ACCESS_AUTO, stream) != LBC_EINVAL) {
            printf("FAIL pipeline step: stages that write into each other were not refused\n");
            return 13;
        }
        ++checks;
    }
    HIP_OK(hipMemcpyAsync(rows.data(), d_rows, world * even_stride, hipMemcpyDeviceToHost, stream));
    HIP_OK(hipMemcpyAsync(send_codes.data(), d_send_codes, reduce_n, hipMemcpyDeviceToHost, stream));
    HIP_OK(hipMemcpyAsync(send_scales.data(), d_send_scales, reduce_n / g * sizeof(float), hipMemcpyDeviceToHost, stream));
    HIP_OK(hipMemcpyAsync(got.data(), d_decoded, even * sizeof(float), hipMemcpyDeviceToHost, stream));
    HIP_OK(hipStreamSynchronize(stream));
    lbo_quantize_f32(want.data(), reduce_n, g, want_send_codes.data(), want_send_scales.data());   // want: the mean of reduce_n
    for (int d = 0; d < world; ++d) {
        if (memcmp(rows.data() + d * even_stride, chunk_codes[d].data(), even_shard) != 0 ||
            memcmp(rows.data() + d * even_stride + even_shard, chunk_scales[d].data(), even_groups * sizeof(float)) != 0) {
            printf("FAIL pipeline step: payload of chunk %d differs from the oracle\n", d);
            return 13;
        }
        std::vector<float> decoded(even_shard);
        lbo_dequantize_f32(chunk_codes[d].data(), chunk_scales[d].data(), even_shard, g, decoded.data());
        if (memcmp(got.data() + d * even_shard, decoded.data(), even_shard * sizeof(float)) != 0) {
            printf("FAIL pipeline step: decoded shard %d differs from the oracle\n", d);
            return 13;
        }
    }
    if (memcmp(send_codes.data(), want_send_codes.data(), reduce_n) != 0 ||
        memcmp(send_scales.data(), want_send_scales.data(), reduce_n / g * sizeof(float)) != 0) {
        printf("FAIL pipeline step: reduce + requantize differs from the oracle\n");
        return 13;
    }
    checks += 3;

    // contract: a bad argument is refused with a message, an unsupported group size is "unsupported", not an error
    if (lbc_quant_pack(d_x, LBC_F32, nullptr, LBC_NONE, -1, g, d_codes[0], d_scales[0], nullptr, LBC_NONE, nullptr, LBC_NONE,
                       nullptr, LBC_NONE, LBC_ACCESS_AUTO, stream) != LBC_EINVAL || strstr(lbc_last_error(), "numel") == nullptr) {
        printf("FAIL negative numel was not refused\n");
        return 7;
    }
    if (lbc_quant_pack(d_x, LBC_F32, nullptr, LBC_NONE, n, 48, d_codes[0], d_scales[0], nullptr, LBC_NONE, nullptr, LBC_NONE,
                       nullptr, LBC_NONE, LBC_ACCESS_AUTO, stream) != LBC_UNSUPPORTED) {
        printf("FAIL group size 48 should be unsupported\n");
        return 7;
    }
    checks += 2;
    if (const int status = wire_format_checks(stream, checks)) return status;
    printf("OK %ld\n", checks);
    return 0;
}
