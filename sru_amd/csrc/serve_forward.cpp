// A caller of the C ABI with no Python and no torch in the process: the role the
// reference's TorchScript demo (sru/csrc/main_test_cpp.cpp:8-52) plays for its operators.
// Runs one forward scan without state store (the serving variant) on inputs generated
// from a fixed integer recipe, and writes h and c_last to a file for a checker to compare.
//
//   serve_forward L B d dirs k padded out_file
//
// Input recipe (exact in float, so a checker can rebuild it bit for bit):
//   value(i, salt) = ((uint32)(i * 2654435761 + salt * 40503) >> 8 & 0xffff) / 65536 - 0.5
//   U = 2 * value(i, 1), x = 2 * value(i, 2), weight_c = value(i, 3), bias = value(i, 4),
//   c_init = value(i, 5); scale_x = 1.5; with padded = 1, sequence b keeps L - (b * 3) % (L / 2)
//   steps and the rest is padding (right-padded).
// Output file: h as L*B*D' floats, then c_last as B*D' floats.
#include <hip/hip_runtime_api.h>

#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "sru_amd.h"

#define HIP_OK(call)                                                                    \
    do {                                                                                \
        hipError_t e_ = (call);                                                         \
        if (e_ != hipSuccess) {                                                         \
            std::fprintf(stderr, "%s failed: %s\n", #call, hipGetErrorString(e_));      \
            return 2;                                                                   \
        }                                                                               \
    } while (0)

static float value(uint64_t i, uint32_t salt) {
    const uint32_t h = (uint32_t)(i * 2654435761u + salt * 40503u);
    return (float)((h >> 8) & 0xffffu) / 65536.0f - 0.5f;
}

template <typename T>
static int to_device(const std::vector<T> &host, void **dev) {
    HIP_OK(hipMalloc(dev, host.size() * sizeof(T)));
    HIP_OK(hipMemcpy(*dev, host.data(), host.size() * sizeof(T), hipMemcpyHostToDevice));
    return 0;
}

int main(int argc, char **argv) {
    if (argc != 8) {
        std::fprintf(stderr, "usage: %s L B d dirs k padded out_file\n", argv[0]);
        return 64;
    }
    const int64_t L = std::atoll(argv[1]), B = std::atoll(argv[2]), d = std::atoll(argv[3]);
    const int dirs = std::atoi(argv[4]), k = std::atoi(argv[5]), padded = std::atoi(argv[6]);
    if (L <= 0 || B <= 0 || d <= 0 || dirs < 1 || dirs > 2 || (k != 3 && k != 4)) {
        std::fprintf(stderr, "bad sizes\n");
        return 64;
    }
    if (sru_amd_abi_version() != SRU_AMD_ABI_VERSION) {
        std::fprintf(stderr, "library ABI %d, header ABI %d\n", sru_amd_abi_version(), SRU_AMD_ABI_VERSION);
        return 3;
    }
    const int64_t Dp = d * dirs, cells = L * B * Dp;

    std::vector<float> U(cells * k), x(cells), wc(2 * Dp), bias(2 * Dp), c0(B * Dp), scale(1, 1.5f);
    std::vector<uint8_t> pad(L * B, 0);
    for (size_t i = 0; i < U.size(); ++i) U[i] = 2.0f * value(i, 1);
    for (size_t i = 0; i < x.size(); ++i) x[i] = 2.0f * value(i, 2);
    for (size_t i = 0; i < wc.size(); ++i) wc[i] = value(i, 3);
    for (size_t i = 0; i < bias.size(); ++i) bias[i] = value(i, 4);
    for (size_t i = 0; i < c0.size(); ++i) c0[i] = value(i, 5);
    if (padded)
        for (int64_t b = 0; b < B; ++b) {
            const int64_t keep = L - (L >= 2 ? (b * 3) % (L / 2) : 0);
            for (int64_t t = keep; t < L; ++t) pad[t * B + b] = 1;
        }

    void *dU, *dx, *dwc, *dbias, *dc0, *dscale, *dpad, *dh, *dcl;
    if (to_device(U, &dU) || to_device(x, &dx) || to_device(wc, &dwc) || to_device(bias, &dbias) ||
        to_device(c0, &dc0) || to_device(scale, &dscale) || to_device(pad, &dpad))
        return 2;
    HIP_OK(hipMalloc(&dh, cells * sizeof(float)));
    HIP_OK(hipMalloc(&dcl, B * Dp * sizeof(float)));
    hipStream_t stream;
    HIP_OK(hipStreamCreate(&stream));

    sru_amd_shape s = {};
    s.length = L;
    s.batch = B;
    s.hidden = d;
    s.dirs = dirs;
    s.k = k;
    s.activation_type = 0;
    s.skip_type = k == 3 ? 1 : 2;
    s.is_custom = 0;
    s.dtype = SRU_AMD_F32;
    s.state_interval = 0;

    // a caller mistake comes back as a status code with a message, nothing is launched
    const float *fbias = static_cast<const float *>(dbias), *fc0 = static_cast<const float *>(dc0);
    const float *fscale = static_cast<const float *>(dscale);
    const uint8_t *bpad = static_cast<const uint8_t *>(dpad);
    float *fcl = static_cast<float *>(dcl);
    int rc = sru_amd_forward(&s, nullptr, dx, dwc, fbias, fc0, nullptr, nullptr, fscale, dh, nullptr, fcl, stream);
    if (rc != SRU_AMD_ERR_NULL_POINTER) {
        std::fprintf(stderr, "expected a NULL-pointer refusal, got %d (%s)\n", rc, sru_amd_status_string(rc));
        return 4;
    }

    rc = sru_amd_forward(&s, dU, k == 3 ? dx : nullptr, dwc, fbias, fc0, /*mask_c*/ nullptr,
                         padded ? bpad : nullptr, k == 3 ? fscale : nullptr, dh,
                         /*c: not kept when serving*/ nullptr, fcl, stream);
    if (rc != SRU_AMD_OK) {
        std::fprintf(stderr, "sru_amd_forward: %s\n", sru_amd_status_string(rc));
        return 5;
    }
    HIP_OK(hipStreamSynchronize(stream));

    std::vector<float> h(cells), cl(B * Dp);
    HIP_OK(hipMemcpy(h.data(), dh, h.size() * sizeof(float), hipMemcpyDeviceToHost));
    HIP_OK(hipMemcpy(cl.data(), dcl, cl.size() * sizeof(float), hipMemcpyDeviceToHost));
    std::FILE *f = std::fopen(argv[7], "wb");
    if (!f || std::fwrite(h.data(), sizeof(float), h.size(), f) != h.size() ||
        std::fwrite(cl.data(), sizeof(float), cl.size(), f) != cl.size() || std::fclose(f) != 0) {
        std::fprintf(stderr, "cannot write %s\n", argv[7]);
        return 6;
    }
    std::printf("serve_forward ok: L=%lld B=%lld d=%lld dirs=%d k=%d padded=%d\n", (long long)L, (long long)B,
                (long long)d, dirs, k, padded);
    for (void *q : {dU, dx, dwc, dbias, dc0, dscale, dpad, dh, dcl}) HIP_OK(hipFree(q));
    HIP_OK(hipStreamDestroy(stream));
    return 0;
}
