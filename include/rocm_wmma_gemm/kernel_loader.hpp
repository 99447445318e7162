// Header-only runtime loader: finds the shared library built for the GPU in the
// machine and forwards typed gemm() calls through its C ABI.
//
// Interface parity: reference rocm_wmma_gemm/include/rocm_wmma_gemm/kernel_loader.hpp:51-182
// (same class name, same gemm<layout_C, layout_A, layout_B>() arities, same library
// naming "librocm_wmma_gemm_<arch>.so", same search order and error type).
#ifndef ROCM_WMMA_GEMM_KERNEL_LOADER_HPP
#define ROCM_WMMA_GEMM_KERNEL_LOADER_HPP

#include <dlfcn.h>
#include <hip/hip_runtime.h>
#include <rocm_wmma_gemm/kernel/common.hpp>
#include <stdexcept>
#include <string>
#include <type_traits>

namespace rocm_wmma_gemm
{

class loader
{
public:
    // (C, A, B, M, N, K, batch, layout_c, layout_a, layout_b, hipStream_t*)
    using entry_fn
        = void (*)(void*, void*, void*, size_t, size_t, size_t, size_t, int, int, int, void*);

    // Probes device 0 for its architecture name and opens the matching library.
    loader() : loader(detect_arch()) {}

    // Opens the library of a named architecture (e.g. "gfx950") without probing.
    explicit loader(const std::string& arch)
    {
        const std::string file = "librocm_wmma_gemm_" + arch + ".so";
        std::string       why;
#ifdef ROCM_WMMA_GEMM_LIB_DIR
        lib_ = try_open(std::string(ROCM_WMMA_GEMM_LIB_DIR) + "/" + file, why);
#endif
        if(lib_ == nullptr)
        {
            lib_ = try_open(file, why);
        }
        if(lib_ == nullptr)
        {
            throw std::runtime_error("rocm_wmma_gemm::loader: could not open " + file + ": " + why);
        }
        try
        {
            entries_[0] = symbol("rocm_wmma_gemm_f16_f16");
            entries_[1] = symbol("rocm_wmma_gemm_f32_f16");
            entries_[2] = symbol("rocm_wmma_gemm_bf16_bf16");
            entries_[3] = symbol("rocm_wmma_gemm_f32_bf16");
        }
        catch(...)
        {
            dlclose(lib_);
            lib_ = nullptr;
            throw;
        }
    }

    ~loader()
    {
        if(lib_ != nullptr)
        {
            dlclose(lib_);
        }
    }

    loader(const loader&)            = delete;
    loader& operator=(const loader&) = delete;
    loader(loader&&)                 = delete;
    loader& operator=(loader&&)      = delete;

    template<m_layout layout_C, m_layout layout_A, m_layout layout_B, class T, class U>
    void gemm(T* C, U* A, U* B, size_t M, size_t N, size_t K, hipStream_t& stream)
    {
        gemm<layout_C, layout_A, layout_B>(C, A, B, M, N, K, size_t{1}, stream);
    }

    template<m_layout layout_C, m_layout layout_A, m_layout layout_B, class T, class U>
    void gemm(
        T* C, U* A, U* B, size_t M, size_t N, size_t K, size_t batch_count, hipStream_t& stream)
    {
        constexpr int slot = type_slot<T, U>();
        static_assert(slot >= 0, "Unsupported type pair for rocm_wmma_gemm::loader");
        entries_[slot](C,
                       A,
                       B,
                       M,
                       N,
                       K,
                       batch_count,
                       static_cast<int>(layout_C),
                       static_cast<int>(layout_A),
                       static_cast<int>(layout_B),
                       &stream);
    }

    // Raw access for callers that bind further symbols of the library.
    void* native_handle() const
    {
        return lib_;
    }

private:
    template<class T, class U>
    static constexpr int type_slot()
    {
        if(std::is_same_v<T, half> && std::is_same_v<U, half>)
            return 0;
        if(std::is_same_v<T, float> && std::is_same_v<U, half>)
            return 1;
        if(std::is_same_v<T, __hip_bfloat16> && std::is_same_v<U, __hip_bfloat16>)
            return 2;
        if(std::is_same_v<T, float> && std::is_same_v<U, __hip_bfloat16>)
            return 3;
        return -1;
    }

    static std::string detect_arch()
    {
        hipDeviceProp_t props{};
        if(hipGetDeviceProperties(&props, 0) != hipSuccess)
        {
            throw std::runtime_error("rocm_wmma_gemm::loader: hipGetDeviceProperties failed");
        }
        // "gfx950:sramecc+:xnack-" -> "gfx950"
        std::string name = props.gcnArchName;
        return name.substr(0, name.find(':'));
    }

    static void* try_open(const std::string& path, std::string& why)
    {
        void* h = dlopen(path.c_str(), RTLD_NOW | RTLD_LOCAL);
        if(h == nullptr)
        {
            const char* e = dlerror();
            why           = e ? e : "unknown dlopen error";
        }
        return h;
    }

    entry_fn symbol(const char* name) const
    {
        dlerror();
        void* p = dlsym(lib_, name);
        if(p == nullptr)
        {
            const char* e = dlerror();
            throw std::runtime_error(std::string("rocm_wmma_gemm::loader: symbol not found: ") + name
                                     + " (" + (e ? e : "null symbol") + ")");
        }
        return reinterpret_cast<entry_fn>(p);
    }

    void*    lib_        = nullptr;
    entry_fn entries_[4] = {nullptr, nullptr, nullptr, nullptr};
};

} // namespace rocm_wmma_gemm

#endif // ROCM_WMMA_GEMM_KERNEL_LOADER_HPP
