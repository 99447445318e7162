// Timing harness for librocm_wmma_gemm_<arch>.so, driven through the runtime loader
// exactly as an application would use it.
//
//   gemm_bench --type f16_f16 --shapes 4096,4096,4096:8192,8192,8192 --layouts all
//              [--reps 20] [--warmup 3] [--batch_count 1]
//              [--variant V --swizzle S --split_k K]   force one compiled variant
//              [--rocblas] [--hipblaslt]               also time rocblas_gemm_ex / hipblasLtMatmul
//                                                      (through libvendor_gemm.so)
//              [--data cyclic|random]
//              [--names]   also print each result under the reference's benchmark name,
//                          "{A:m_layout::...,B:...,C:...,m:M,n:N,k:K}/manual_time ...", in
//                          the column order its report generator parses
//                          (reference docs/generate_report.py:36-58)
//
// Measures what the reference's benchmarks measure (reference
// benchmark/gemm/bench_half_half.cpp:78-114): hipEvent time around each enqueue,
// TFLOP/s = 2*M*N*K*batch / t, reported per shape and layout; "--shapes M,N,K:..."
// and "--batch_count" keep the reference's spelling (:182-235).  Layout triples are
// written A,B,C with r/c, e.g. "rcr" = A row-major, B column-major, C row-major.
#include <dlfcn.h>
#include <hip/hip_runtime.h>
#include <rocm_wmma_gemm/kernel_loader.hpp>
#include <rocm_wmma_gemm_c.h>

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include <vendor_gemm/vendor_gemm.h>

// The type pair a binary times when --type is not given: the Makefile builds this file
// once per pair under the reference's benchmark names (reference benchmark/gemm/
// bench_half_half.cpp, bench_float_half.cpp, bench_bf16_bf16.cpp, bench_float_bf16.cpp)
// and once as gemm_bench.
#ifndef GEMM_BENCH_DEFAULT_TYPE
#define GEMM_BENCH_DEFAULT_TYPE "f16_f16"
#endif

#define CHECK(x)                                                                                   \
    do                                                                                             \
    {                                                                                              \
        hipError_t e_ = (x);                                                                       \
        if(e_ != hipSuccess)                                                                       \
        {                                                                                          \
            std::fprintf(stderr, "%s:%d %s: %s\n", __FILE__, __LINE__, #x, hipGetErrorString(e_)); \
            std::exit(2);                                                                          \
        }                                                                                          \
    } while(0)

namespace
{

struct shape
{
    size_t m, n, k;
};

// Fill 16-bit elements: cyclic {0.1, 0.125, 0.15, 0.175, 0.2} as the reference's
// benchmarks do (reference benchmark/bench.hpp:37-52), or hashed uniform [-1, 1).
__global__ void fill16(unsigned short* p, size_t n, int bf16, int random, unsigned seed)
{
    for(size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
        i += (size_t)gridDim.x * blockDim.x)
    {
        float v;
        if(random)
        {
            unsigned h = (unsigned)i * 2654435761u ^ seed;
            h ^= h >> 16;
            h *= 0x85ebca6bu;
            h ^= h >> 13;
            h *= 0xc2b2ae35u;
            h ^= h >> 16;
            v = (float)(h >> 8) * (2.0f / 16777216.0f) - 1.0f;
        }
        else
        {
            const float cyc[5] = {0.1f, 0.125f, 0.15f, 0.175f, 0.2f};
            v                  = cyc[i % 5];
        }
        if(bf16)
        {
            unsigned u = __float_as_uint(v);
            u += 0x7fffu + ((u >> 16) & 1u);
            p[i] = (unsigned short)(u >> 16);
        }
        else
        {
            _Float16 h = (_Float16)v;
            p[i]       = __builtin_bit_cast(unsigned short, h);
        }
    }
}

std::vector<shape> parse_shapes(const std::string& s)
{
    std::vector<shape> out;
    size_t             pos = 0;
    while(pos < s.size())
    {
        size_t      end = s.find(':', pos);
        std::string tok = s.substr(pos, end == std::string::npos ? std::string::npos : end - pos);
        shape       sh{};
        if(std::sscanf(tok.c_str(), "%zu,%zu,%zu", &sh.m, &sh.n, &sh.k) != 3)
        {
            std::fprintf(stderr, "bad shape '%s' (want M,N,K)\n", tok.c_str());
            std::exit(2);
        }
        out.push_back(sh);
        if(end == std::string::npos)
            break;
        pos = end + 1;
    }
    return out;
}

std::vector<std::string> parse_layouts(const std::string& s)
{
    if(s == "all")
        return {"rrr", "rrc", "rcr", "rcc", "crr", "crc", "ccr", "ccc"};
    std::vector<std::string> out;
    size_t                   pos = 0;
    while(pos < s.size())
    {
        size_t end = s.find(',', pos);
        out.push_back(s.substr(pos, end == std::string::npos ? std::string::npos : end - pos));
        if(end == std::string::npos)
            break;
        pos = end + 1;
    }
    for(auto& l : out)
        if(l.size() != 3 || l.find_first_not_of("rc") != std::string::npos)
        {
            std::fprintf(stderr, "bad layout '%s' (want three of r/c in A,B,C order)\n", l.c_str());
            std::exit(2);
        }
    return out;
}

int type_index(const std::string& t)
{
    const char* names[4] = {"f16_f16", "f32_f16", "bf16_bf16", "f32_bf16"};
    for(int i = 0; i < 4; ++i)
        if(t == names[i])
            return i;
    std::fprintf(stderr, "bad type '%s'\n", t.c_str());
    std::exit(2);
}

} // namespace

int main(int argc, char** argv)
{
    std::string type = GEMM_BENCH_DEFAULT_TYPE, shapes_arg = "4096,4096,4096", layouts_arg = "rcr",
                data = "random";
    int    reps = 20, warmup = 3, variant = -1, swizzle = 4, split_k = 1;
    size_t batch = 1;
    bool   with_rocblas = false, with_hipblaslt = false;
    bool   names        = false;
    for(int i = 1; i < argc; ++i)
    {
        auto next = [&](const char* flag) -> const char* {
            if(i + 1 >= argc)
            {
                std::fprintf(stderr, "%s needs a value\n", flag);
                std::exit(2);
            }
            return argv[++i];
        };
        std::string a = argv[i];
        if(a == "--type")
            type = next("--type");
        else if(a == "--shapes")
            shapes_arg = next("--shapes");
        else if(a == "--layouts")
            layouts_arg = next("--layouts");
        else if(a == "--reps")
            reps = std::atoi(next("--reps"));
        else if(a == "--warmup")
            warmup = std::atoi(next("--warmup"));
        else if(a == "--batch_count")
            batch = std::strtoull(next("--batch_count"), nullptr, 10);
        else if(a == "--variant")
            variant = std::atoi(next("--variant"));
        else if(a == "--swizzle")
            swizzle = std::atoi(next("--swizzle"));
        else if(a == "--split_k")
            split_k = std::atoi(next("--split_k"));
        else if(a == "--data")
            data = next("--data");
        else if(a == "--rocblas")
            with_rocblas = true;
        else if(a == "--hipblaslt")
            with_hipblaslt = true;
        else if(a == "--names")
            names = true;
        else
        {
            std::fprintf(stderr, "unknown argument %s\n", a.c_str());
            return 2;
        }
    }
    const int  tidx    = type_index(type);
    const bool bf16    = tidx >= 2;
    const bool c_is_32 = tidx == 1 || tidx == 3;
    const auto shapes  = parse_shapes(shapes_arg);
    const auto layouts = parse_layouts(layouts_arg);

    hipDeviceProp_t prop;
    CHECK(hipGetDeviceProperties(&prop, 0));
    const double peak_tf = prop.multiProcessorCount * 4.0 * 1024.0 * 2.4e9 / 1e12;
    std::printf("# device %s, %d CUs, reported clock %d MHz; peak denominator = CUs*4*1024*2.4GHz = %.1f TFLOP/s\n",
                prop.gcnArchName, prop.multiProcessorCount, prop.clockRate / 1000, peak_tf);

    rocm_wmma_gemm::loader loader;
    using run_variant_fn = int (*)(int, int, int, int, void*, void*, void*, size_t, size_t, size_t,
                                   size_t, int, int, int, void*);
    auto run_variant = reinterpret_cast<run_variant_fn>(
        dlsym(loader.native_handle(), "rocm_wmma_gemm_run_variant"));
    using select_fn = int (*)(size_t, size_t, size_t, size_t, int, int, int, int, int*, int*);
    auto select = reinterpret_cast<select_fn>(
        dlsym(loader.native_handle(), "rocm_wmma_gemm_select_batched"));
    using entry_fn = rocm_wmma_gemm::loader::entry_fn;
    const char* entry_names[4] = {"rocm_wmma_gemm_f16_f16", "rocm_wmma_gemm_f32_f16",
                                  "rocm_wmma_gemm_bf16_bf16", "rocm_wmma_gemm_f32_bf16"};
    auto entry = reinterpret_cast<entry_fn>(dlsym(loader.native_handle(), entry_names[tidx]));
    if(!entry || (variant >= 0 && !run_variant))
    {
        std::fprintf(stderr, "library lacks a needed symbol\n");
        return 2;
    }

    if((with_rocblas || with_hipblaslt) && vendor_gemm_init() != 0)
    {
        std::fprintf(stderr, "vendor_gemm_init failed\n");
        return 2;
    }

    hipStream_t stream;
    CHECK(hipStreamCreate(&stream));
    hipEvent_t e0, e1;
    CHECK(hipEventCreate(&e0));
    CHECK(hipEventCreate(&e1));

    std::printf("%-10s %-22s %-4s %8s %6s %10s %10s %8s %8s\n", "type", "M,N,K", "ABC", "variant",
                "split", "median_ms", "min_ms", "TFLOP/s", "%peak");
    for(const shape& sh : shapes)
    {
        const size_t a_elems = sh.m * sh.k * batch, b_elems = sh.k * sh.n * batch,
                     c_elems = sh.m * sh.n * batch;
        void *A, *B, *C;
        CHECK(hipMalloc(&A, a_elems * 2));
        CHECK(hipMalloc(&B, b_elems * 2));
        CHECK(hipMalloc(&C, c_elems * (c_is_32 ? 4 : 2)));
        fill16<<<2048, 256, 0, stream>>>((unsigned short*)A, a_elems, bf16, data == "random", 0x1234u);
        fill16<<<2048, 256, 0, stream>>>((unsigned short*)B, b_elems, bf16, data == "random", 0x9876u);
        CHECK(hipStreamSynchronize(stream));
        for(const std::string& lay : layouts)
        {
            const int la = lay[0] == 'c', lb = lay[1] == 'c', lc = lay[2] == 'c';
            int       sel_swz = swizzle, sel_sk = split_k, sel_var = variant;
            if(variant < 0 && select)
                sel_var = select(sh.m, sh.n, sh.k, batch, tidx, lc, la, lb, &sel_swz, &sel_sk);
            auto call = [&]() {
                if(variant >= 0)
                {
                    int rc = run_variant(tidx, variant, swizzle, split_k, C, A, B, sh.m, sh.n, sh.k,
                                         batch, lc, la, lb, &stream);
                    if(rc != 0)
                    {
                        std::fprintf(stderr, "run_variant failed: %d\n", rc);
                        std::exit(3);
                    }
                }
                else
                    entry(C, A, B, sh.m, sh.n, sh.k, batch, lc, la, lb, &stream);
            };
            for(int w = 0; w < warmup; ++w)
                call();
            CHECK(hipStreamSynchronize(stream));
            CHECK(hipGetLastError());
            std::vector<float> ms(reps);
            for(int r = 0; r < reps; ++r)
            {
                CHECK(hipEventRecord(e0, stream));
                call();
                CHECK(hipEventRecord(e1, stream));
                CHECK(hipEventSynchronize(e1));
                CHECK(hipEventElapsedTime(&ms[r], e0, e1));
            }
            std::sort(ms.begin(), ms.end());
            const double med = ms[reps / 2], mn = ms[0];
            const double tf  = 2.0 * sh.m * sh.n * sh.k * batch / (med * 1e-3) / 1e12;
            char         dims[64];
            std::snprintf(dims, sizeof dims, "%zu,%zu,%zu", sh.m, sh.n, sh.k);
            std::printf("%-10s %-22s %-4s %8d %6d %10.4f %10.4f %8.1f %7.1f%%\n", type.c_str(), dims,
                        lay.c_str(), sel_var, sel_sk, med, mn, tf, 100.0 * tf / peak_tf);
            if(names)
            {
                // name/manual_time  time  cpu  iterations  avg_tflops  bytes_per_second
                const double gib_s = ((double)(sh.m * sh.k + sh.k * sh.n) * 2 + (double)sh.m * sh.n * (c_is_32 ? 4 : 2))
                                     * batch / (med * 1e-3) / (1024.0 * 1024.0 * 1024.0);
                std::printf("{A:m_layout::%s,B:m_layout::%s,C:m_layout::%s,m:%zu,n:%zu,k:%zu}/manual_time"
                            " %10.3f ms %10.3f ms %8d %10.4f %12.4fGi/s\n",
                            la ? "col_major" : "row_major", lb ? "col_major" : "row_major",
                            lc ? "col_major" : "row_major", sh.m, sh.n, sh.k, med, med, reps, tf, gib_s);
            }
            std::fflush(stdout);
            for(int backend = 0; backend < 2; ++backend)
            {
                if(!(backend == VENDOR_GEMM_ROCBLAS ? with_rocblas : with_hipblaslt))
                    continue;
                auto blas_call = [&]() {
                    const int rc = vendor_gemm(backend, tidx, C, A, B, sh.m, sh.n, sh.k, batch, lc, la, lb, &stream);
                    if(rc != 0)
                    {
                        std::fprintf(stderr, "vendor_gemm failed: %d\n", rc);
                        std::exit(3);
                    }
                };
                for(int w = 0; w < warmup; ++w)
                    blas_call();
                CHECK(hipStreamSynchronize(stream));
                for(int r = 0; r < reps; ++r)
                {
                    CHECK(hipEventRecord(e0, stream));
                    blas_call();
                    CHECK(hipEventRecord(e1, stream));
                    CHECK(hipEventSynchronize(e1));
                    CHECK(hipEventElapsedTime(&ms[r], e0, e1));
                }
                std::sort(ms.begin(), ms.end());
                const double btf = 2.0 * sh.m * sh.n * sh.k * batch / (ms[reps / 2] * 1e-3) / 1e12;
                std::printf("%-10s %-22s %-4s %8s %6s %10.4f %10.4f %8.1f %7.1f%%\n",
                            backend == VENDOR_GEMM_ROCBLAS ? "rocblas" : "hipblaslt", dims, lay.c_str(), "-", "-",
                            ms[reps / 2], ms[0], btf, 100.0 * btf / peak_tf);
                std::fflush(stdout);
            }
        }
        CHECK(hipFree(A));
        CHECK(hipFree(B));
        CHECK(hipFree(C));
    }
    return 0;
}
