// Drop-in check: a C++ client written against the rocm_wmma_gemm loader interface
// (loader.gemm<layout_C, layout_A, layout_B>(C, A, B, M, N, K[, batch], stream)),
// run for all four type pairs and all eight layout triples, compared with a host
// triple loop.  The same source is compiled twice: once against this repository's
// include/rocm_wmma_gemm/kernel_loader.hpp and once against the reference's own
// header where it lies, to show that the reference's loader opens and drives
// librocm_wmma_gemm_gfx950.so unchanged.
#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>
#include <rocm_wmma_gemm/kernel_loader.hpp>

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <vector>

using rocm_wmma_gemm::m_layout;

#define CHECK(x)                                                                      \
    do                                                                                \
    {                                                                                 \
        hipError_t e_ = (x);                                                          \
        if(e_ != hipSuccess)                                                          \
        {                                                                             \
            std::fprintf(stderr, "%s:%d %s\n", __FILE__, __LINE__, hipGetErrorString(e_)); \
            std::exit(2);                                                             \
        }                                                                             \
    } while(0)

template<class T>
float to_f(T v)
{
    return static_cast<float>(v);
}
template<>
float to_f(__hip_bfloat16 v)
{
    return __bfloat162float(v);
}
template<class T>
T from_f(float v)
{
    return static_cast<T>(v);
}
template<>
__hip_bfloat16 from_f(float v)
{
    return __float2bfloat16(v);
}

static size_t at(size_t i, size_t j, size_t m, size_t n, m_layout l)
{
    return l == m_layout::row_major ? i * n + j : j * m + i;
}

template<m_layout LC, m_layout LA, m_layout LB, class T, class U>
int one_case(rocm_wmma_gemm::loader& loader, size_t M, size_t N, size_t K, size_t batch,
             hipStream_t& stream)
{
    std::vector<U> A(M * K * batch), B(K * N * batch);
    std::vector<T> C(M * N * batch);
    unsigned       s = 12345u;
    auto           rnd = [&]() {
        s = s * 1664525u + 1013904223u;
        return (float)((int)(s >> 20) % 17 - 8) / 8.0f; // multiples of 1/8 in [-1, 1]
    };
    for(auto& v : A)
        v = from_f<U>(rnd());
    for(auto& v : B)
        v = from_f<U>(rnd());
    U *dA, *dB;
    T* dC;
    CHECK(hipMalloc(&dA, A.size() * sizeof(U)));
    CHECK(hipMalloc(&dB, B.size() * sizeof(U)));
    CHECK(hipMalloc(&dC, C.size() * sizeof(T)));
    CHECK(hipMemcpy(dA, A.data(), A.size() * sizeof(U), hipMemcpyHostToDevice));
    CHECK(hipMemcpy(dB, B.data(), B.size() * sizeof(U), hipMemcpyHostToDevice));
    if(batch == 1)
        loader.gemm<LC, LA, LB>(dC, dA, dB, M, N, K, stream);
    else
        loader.gemm<LC, LA, LB>(dC, dA, dB, M, N, K, batch, stream);
    CHECK(hipPeekAtLastError());
    CHECK(hipStreamSynchronize(stream));
    CHECK(hipMemcpy(C.data(), dC, C.size() * sizeof(T), hipMemcpyDeviceToHost));
    int bad = 0;
    for(size_t b = 0; b < batch; ++b)
        for(size_t i = 0; i < M; ++i)
            for(size_t j = 0; j < N; ++j)
            {
                float acc = 0.0f; // sums of multiples of 1/64 below 2^24/64: exact in fp32
                for(size_t k = 0; k < K; ++k)
                    acc += to_f(A[b * M * K + at(i, k, M, K, LA)]) * to_f(B[b * K * N + at(k, j, K, N, LB)]);
                const float got  = to_f(C[b * M * N + at(i, j, M, N, LC)]);
                const float want = to_f(from_f<T>(acc));
                if(got != want)
                    ++bad;
            }
    CHECK(hipFree(dA));
    CHECK(hipFree(dB));
    CHECK(hipFree(dC));
    return bad;
}

template<class T, class U>
int all_layouts(rocm_wmma_gemm::loader& loader, const char* name, hipStream_t& stream)
{
    constexpr m_layout R = m_layout::row_major, Cm = m_layout::col_major;
    int bad = 0;
    const size_t M = 192, N = 320, K = 136;
    bad += one_case<R, R, R, T, U>(loader, M, N, K, 1, stream);
    bad += one_case<R, R, Cm, T, U>(loader, M, N, K, 1, stream);
    bad += one_case<R, Cm, R, T, U>(loader, M, N, K, 1, stream);
    bad += one_case<R, Cm, Cm, T, U>(loader, M, N, K, 1, stream);
    bad += one_case<Cm, R, R, T, U>(loader, M, N, K, 1, stream);
    bad += one_case<Cm, R, Cm, T, U>(loader, M, N, K, 1, stream);
    bad += one_case<Cm, Cm, R, T, U>(loader, M, N, K, 1, stream);
    bad += one_case<Cm, Cm, Cm, T, U>(loader, M, N, K, 1, stream);
    bad += one_case<R, R, Cm, T, U>(loader, 256, 256, 256, 3, stream); // batched, tile-aligned
    std::printf("%-10s %s (%d mismatching elements)\n", name, bad ? "FAIL" : "PASS", bad);
    return bad;
}

int main()
{
    rocm_wmma_gemm::loader loader; // probes device 0, dlopens the per-arch library
    hipStream_t            stream;
    CHECK(hipStreamCreate(&stream));
    int bad = 0;
    bad += all_layouts<half, half>(loader, "f16_f16", stream);
    bad += all_layouts<float, half>(loader, "f32_f16", stream);
    bad += all_layouts<__hip_bfloat16, __hip_bfloat16>(loader, "bf16_bf16", stream);
    bad += all_layouts<float, __hip_bfloat16>(loader, "f32_bf16", stream);
    CHECK(hipStreamDestroy(stream));
    std::printf("%s\n", bad ? "DROP-IN CHECK FAILED" : "DROP-IN CHECK PASSED");
    return bad ? 1 : 0;
}
