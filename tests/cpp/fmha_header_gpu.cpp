// GPU check of include/flashck/fmha/fmha_fwd.h with real device pointers: reads a problem file written by
// tests/test_gpu_cpp_header.py, runs it through the header API (the typed layer a C++ caller of the reference's header
// interface would use) and writes the output for the test to compare with the oracle.
//
// usage: fmha_header_gpu <fp16|bf16> <fwd|decode|prefill> <in.bin> <out.bin>
// file: int64 header[16], then the arrays in the order the op reads them (sizes follow from the header)
#include "flashck/fmha/fmha_fwd.h"

#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#define HIP_OK(x)                                                                      \
    do {                                                                               \
        hipError_t e_ = (x);                                                           \
        if (e_ != hipSuccess) {                                                        \
            std::printf("%s failed: %s\n", #x, hipGetErrorString(e_));                 \
            std::exit(2);                                                              \
        }                                                                              \
    } while (0)

struct File {
    std::FILE* f;
    explicit File(const char* path, const char* mode) : f(std::fopen(path, mode))
    {
        if (!f) {
            std::printf("cannot open %s\n", path);
            std::exit(2);
        }
    }
    ~File() { std::fclose(f); }
    void read(void* dst, size_t bytes)
    {
        if (std::fread(dst, 1, bytes, f) != bytes) {
            std::printf("short read\n");
            std::exit(2);
        }
    }
};

// one array: read from the file into device memory
template <typename E>
static E* upload(File& in, size_t count)
{
    std::vector<E> host(count);
    in.read(host.data(), count * sizeof(E));
    E* dev = nullptr;
    HIP_OK(hipMalloc(&dev, count * sizeof(E) + 16));
    HIP_OK(hipMemcpy(dev, host.data(), count * sizeof(E), hipMemcpyHostToDevice));
    return dev;
}

template <typename E>
static void download(const char* path, const E* dev, size_t count)
{
    std::vector<E> host(count);
    HIP_OK(hipDeviceSynchronize());
    HIP_OK(hipMemcpy(host.data(), dev, count * sizeof(E), hipMemcpyDeviceToHost));
    File out(path, "wb");
    std::fwrite(host.data(), sizeof(E), count, out.f);
}

template <typename T>
static int run_fwd(File& in, const int64_t* h, const char* out_path)
{
    namespace n = flashck::naive;
    // header: B sq sk Hq Hk D mask_type window_left window_right
    const int64_t B = h[0], sq = h[1], sk = h[2], Hq = h[3], Hk = h[4], D = h[5];
    T* q = upload<T>(in, B * sq * Hq * D);
    T* k = upload<T>(in, B * sk * Hk * D);
    T* v = upload<T>(in, B * sk * Hk * D);
    T* o = nullptr;
    HIP_OK(hipMalloc(&o, B * sq * Hq * D * sizeof(T)));
    T* r = n::fmha_fwd<T>(q, k, v, o, B, sq, sk, Hq, Hk, D, D, 0.f, {h[7], h[8]}, (uint32_t)h[6]);
    if (r != o) return 1;
    download(out_path, o, B * sq * Hq * D);
    return 0;
}

template <typename T>
static int run_decode(File& in, const int64_t* h, const char* out_path)
{
    namespace n = flashck::naive;
    // header: B Hq Hk D pages page_size table_stride num_splits (0: the heuristic)
    const int64_t B = h[0], Hq = h[1], Hk = h[2], D = h[3], pages = h[4], P = h[5], stride = h[6];
    T* q = upload<T>(in, B * Hq * D);
    T* kc = upload<T>(in, pages * P * Hk * D);
    T* vc = upload<T>(in, pages * P * Hk * D);
    int32_t* sl = upload<int32_t>(in, B);
    int32_t* bt = upload<int32_t>(in, B * stride);
    // a workspace for the largest split count the heuristic can return; lse_acc sits behind o_acc for the count used
    float* ws = nullptr;
    HIP_OK(hipMalloc(&ws, fck_fmha_splitkv_workspace_bytes(B, Hq, 1, D, 128)));
    // the split count is needed to lay the workspace out, so ask the heuristic the way the header does
    const int64_t ns = h[7] > 0 ? h[7] : fck_fmha_num_splits_heuristic(B, Hq, Hk, 1, stride * P, D, 0);
    float* o_acc = ws;
    float* lse_acc = ws + B * Hq * ns * D;
    const int used = n::fmha_fwd_splitkv<T>(q, kc, vc, o_acc, lse_acc, sl, bt, B, 1, Hq, Hk, D, D, h[7], B * stride, P);
    if (used != ns) {
        std::printf("split count %d, expected %ld\n", used, (long)ns);
        return 1;
    }
    T* o = nullptr;
    HIP_OK(hipMalloc(&o, B * Hq * D * sizeof(T)));
    n::fmha_fwd_splitkv_combine<T>(lse_acc, o_acc, o, B, 1, Hq, D, ns);
    download(out_path, o, B * Hq * D);
    return 0;
}

template <typename T>
static int run_prefill(File& in, const int64_t* h, const char* out_path)
{
    namespace n = flashck::naive;
    // header: B total_q Hq Hk D pages page_size n_indices max_seqlen_q
    const int64_t B = h[0], tq = h[1], Hq = h[2], Hk = h[3], D = h[4], pages = h[5], P = h[6], nidx = h[7], maxq = h[8];
    T* q = upload<T>(in, tq * Hq * D);
    T* kc = upload<T>(in, pages * P * Hk * D);
    T* vc = upload<T>(in, pages * P * Hk * D);
    int32_t* cu = upload<int32_t>(in, B + 1);
    int32_t* indptr = upload<int32_t>(in, B + 1);
    int32_t* indices = upload<int32_t>(in, nidx);
    int32_t* last = upload<int32_t>(in, B);
    T* o = nullptr;
    HIP_OK(hipMalloc(&o, tq * Hq * D * sizeof(T)));
    n::fmha_batch_prefill<T>(q, kc, vc, o, cu, indptr, indices, last, pages, P, B, Hq, Hk, D, D, maxq);
    download(out_path, o, tq * Hq * D);
    return 0;
}

int main(int argc, char** argv)
{
    if (argc != 5) {
        std::printf("usage: %s <fp16|bf16> <fwd|decode|prefill> <in.bin> <out.bin>\n", argv[0]);
        return 2;
    }
    const bool fp16 = !std::strcmp(argv[1], "fp16");
    File in(argv[3], "rb");
    int64_t h[16];
    in.read(h, sizeof(h));
    try {
        if (!std::strcmp(argv[2], "fwd")) return fp16 ? run_fwd<_Float16>(in, h, argv[4]) : run_fwd<unsigned short>(in, h, argv[4]);
        if (!std::strcmp(argv[2], "decode")) return fp16 ? run_decode<_Float16>(in, h, argv[4]) : run_decode<unsigned short>(in, h, argv[4]);
        if (!std::strcmp(argv[2], "prefill")) return fp16 ? run_prefill<_Float16>(in, h, argv[4]) : run_prefill<unsigned short>(in, h, argv[4]);
    } catch (const std::exception& e) {
        std::printf("exception: %s\n", e.what());
        return 1;
    }
    return 2;
}
