// C wrappers around the reference's own CPU functions, for validating tab_oracle.c.
//
// TEST INFRASTRUCTURE ONLY.  This translation unit contains no reference code: the build
// recipe (oracle/Makefile, target _ref/libtab_ref.so) compiles it together with
//   - /root/reference/TAB_CPU.h           (im2row templates, popcnt64 macro), included
//     from where it lies, and
//   - the bodies of the named functions of /root/reference/TAB_CPU.cpp, which the recipe
//     extracts into a temporary file (REF_EXTRACT) outside the repository, because the
//     file as a whole is not valid C++ (undeclared identifiers at TAB_CPU.cpp:213,222,
//     522-530,608,632) and cannot be compiled as shipped.
// Only the resulting shared object is kept (oracle/_ref/, git-ignored).
#define GCC 1
#include <cstdint>
#include <cstring>
#include <vector>
#include "TAB_CPU.h"
#include REF_EXTRACT

extern "C" {

// TAB_CPU.cpp:242-328.  y is [M][N] int32.
void ref_gemm_tnn(int64_t *a, int64_t *b, int M, int N, int K, int32_t *y)
{
    std::vector<int> r = TNNGEMM_baseline(a, b, M, N, K);
    std::memcpy(y, r.data(), sizeof(int) * r.size());
}
void ref_gemm_tbn(int64_t *a, int64_t *b, int M, int N, int K, int32_t *y)
{
    std::vector<int> r = TBNGEMM_baseline(a, b, M, N, K);
    std::memcpy(y, r.data(), sizeof(int) * r.size());
}
void ref_gemm_btn(int64_t *a, int64_t *b, int32_t *btn, int M, int N, int K, int32_t *y)
{
    std::vector<int> r = BTNGEMM_baseline(a, b, btn, M, N, K);
    std::memcpy(y, r.data(), sizeof(int) * r.size());
}
void ref_gemm_bnn(int64_t *a, int64_t *b, int M, int N, int K, int NUM, int32_t *y)
{
    std::vector<int> r = BNNGEMM_baseline(a, b, M, N, K, NUM);
    std::memcpy(y, r.data(), sizeof(int) * r.size());
}

// TAB_CPU.cpp:332-383, the CPU-only types 4 (DoReFa 2-bit) and 5 (RTN).
void ref_gemm_drf(int64_t *a, int64_t *b, int M, int N, int K, int32_t *y)
{
    std::vector<int> r = DRFGEMM_baseline(a, b, M, N, K);
    std::memcpy(y, r.data(), sizeof(int) * r.size());
}
void ref_gemm_rtn(int64_t *a, int64_t *b, int M, int N, int K, int32_t *y)
{
    std::vector<int> r = RTNGEMM_baseline(a, b, M, N, K);
    std::memcpy(y, r.data(), sizeof(int) * r.size());
}

// TAB_CPU.h:27-63.  x is [N][H][W][D] packed words (already padded); rows is
// [N*OH*OW][KH*KW*D].  The routine copies exactly three kernel rows, so KH must be 3.
void ref_img2row_3x3(int64_t *x, int N, int D, int H, int W, int KH, int KW, int s1, int s2,
                     int64_t *rows)
{
    std::vector<int64_t> r = Parallel_Img2Row_NHWCB_3x3<int64_t>(x, N, D, H, W, KH, KW, s1, s2);
    std::memcpy(rows, r.data(), sizeof(int64_t) * r.size());
}

// TAB_CPU.cpp:20-124 / 137-206.  x is NCHW fp32; out is the spatially pre-padded
// [N][H+2p1][W+2p2][PC][planes] buffer.  The caller is responsible for the input layout
// these routines actually read (they advance to the next 64-channel block before
// reading, TAB_CPU.cpp:59,92,171,189).
void ref_ternarize_nchw(float *x, int p1, int p2, float *ths, int N, int C, int H, int W,
                        int64_t *out)
{
    std::vector<int64_t> r = Parallel_Ternarize_NCHWB_to_NHWCB(x, p1, p2, ths, N, C, H, W);
    std::memcpy(out, r.data(), sizeof(int64_t) * r.size());
}
void ref_binarize_nchw(const float *x, int p1, int p2, int N, int C, int H, int W, int64_t *out)
{
    std::vector<int64_t> r = Parallel_Binarize_NCHW_to_NHWC(x, p1, p2, N, C, H, W);
    std::memcpy(out, r.data(), sizeof(int64_t) * r.size());
}

}  // extern "C"
