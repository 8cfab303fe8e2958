// Timing harness with the reference's command line (src/gemm/benchmark.cc:27-38):
//
//     benchmark type M N K lda ldb ldc [transA transB dtype batch alpha beta]
//
//   type 0: the per-shape table's pick (the reference's mode 0 ran its hand-written kernel)
//   type 1: sweep every tile config and report the fastest (src/gemm/benchmark.cc:89-109 did this over
//           the 23 Tensile kernels)
//   type 2: in the reference this timed rocBLAS; this library has no third-party GEMM to compare with
//           and says so
//   transA/transB: N or T (default N T, the reference's only layout); dtype: s (fp32), h (fp16) or
//   d (fp64, the reference's element type); alpha, beta default to the reference's -1 and 1
//   (src/gemm/benchmark.cc:20).
//
// TFLOP/s = 1e-12 * 2*M*N*K*batch / t (src/gemm/benchmark.cc:98), t from a blocking-sync event pair on the
// null stream (src/gemm/common.h:4-18) around `reps` launches after one warm-up.  The reference timed one
// launch that included loading the code object (src/gemm/driver.h:41); kernels here are linked in.
// Efficiency is printed against MI355X's published dense matrix peak for the element type.
#include <cstring>
#include <vector>

#include "common.h"
#include "gemm.h"

static double peak_tflops(int dtype) { return dtype == MMBO_F16 ? 2500.0 : dtype == MMBO_F64 ? 78.6 : 157.3; }

int main(int argc, char **argv)
{
    if (argc < 8) {
        std::fprintf(stderr, "usage: %s type M N K lda ldb ldc [transA transB dtype batch alpha beta]\n", argv[0]);
        return 2;
    }
    const int type = std::atoi(argv[1]);
    const size_t M = std::strtoull(argv[2], NULL, 10), N = std::strtoull(argv[3], NULL, 10),
                 K = std::strtoull(argv[4], NULL, 10);
    const size_t lda = std::strtoull(argv[5], NULL, 10), ldb = std::strtoull(argv[6], NULL, 10),
                 ldc = std::strtoull(argv[7], NULL, 10);
    const int ta = argc > 8 && (argv[8][0] == 'T' || argv[8][0] == 't') ? MMBO_OP_T : MMBO_OP_N;
    const int tb = argc > 9 ? ((argv[9][0] == 'T' || argv[9][0] == 't') ? MMBO_OP_T : MMBO_OP_N) : MMBO_OP_T;
    const char dch = argc > 10 ? argv[10][0] : 's';
    const int dtype = (dch == 'h' || dch == 'H') ? MMBO_F16 : (dch == 'd' || dch == 'D') ? MMBO_F64 : MMBO_F32;
    const int batch = argc > 11 ? std::atoi(argv[11]) : 1;
    const double alpha_d = argc > 12 ? std::atof(argv[12]) : -1.0, beta_d = argc > 13 ? std::atof(argv[13]) : 1.0;
    const float alpha_f = (float)alpha_d, beta_f = (float)beta_d;
    // the C ABI reads the scalars in double for fp64 and in float otherwise
    const void *alpha = dtype == MMBO_F64 ? (const void *)&alpha_d : (const void *)&alpha_f;
    const void *beta = dtype == MMBO_F64 ? (const void *)&beta_d : (const void *)&beta_f;
    if (type == 2) {
        std::printf("type 2 (third-party BLAS comparison) is not part of this library\n");
        return 0;
    }

    const size_t esz = dtype == MMBO_F16 ? 2 : dtype == MMBO_F64 ? 8 : 4;
    const size_t a_elems = lda * (ta ? M : K), b_elems = ldb * (tb ? K : N), c_elems = ldc * N;
    // host fill like the reference's (src/gemm/benchmark.cc:45-53: rand() in [0,1], A then B then C)
    std::vector<unsigned char> hA(a_elems * batch * esz), hB(b_elems * batch * esz), hC(c_elems * batch * esz);
    auto fill = [&](std::vector<unsigned char> &buf, size_t count) {
        for (size_t i = 0; i < count; ++i) {
            float v = (float)std::rand() / (float)RAND_MAX;
            if (dtype == MMBO_F64) {
                double d = (double)std::rand() / (double)RAND_MAX;
                std::memcpy(&buf[i * 8], &d, 8);
            } else if (dtype == MMBO_F16) {
                _Float16 h = (_Float16)v;
                std::memcpy(&buf[i * 2], &h, 2);
            } else {
                std::memcpy(&buf[i * 4], &v, 4);
            }
        }
    };
    fill(hA, a_elems * batch);
    fill(hB, b_elems * batch);
    fill(hC, c_elems * batch);
    void *dA, *dB, *dC;
    HIP_CHECK(hipMalloc(&dA, hA.size() + 16));
    HIP_CHECK(hipMalloc(&dB, hB.size() + 16));
    HIP_CHECK(hipMalloc(&dC, hC.size() + 16));
    HIP_CHECK(hipMemcpy(dA, hA.data(), hA.size(), hipMemcpyHostToDevice));
    HIP_CHECK(hipMemcpy(dB, hB.data(), hB.size(), hipMemcpyHostToDevice));
    HIP_CHECK(hipMemcpy(dC, hC.data(), hC.size(), hipMemcpyHostToDevice));

    auto call = [&](int id) {
        return mmbo_gemm_strided_batched(dtype, ta, tb, M, N, K, alpha, dA, lda, (long long)a_elems, dB, ldb,
                                         (long long)b_elems, beta, dC, ldc, (long long)c_elems, batch, id, NULL);
    };
    auto time_config = [&](int id, float *seconds) {
        int rc = call(id);                       // warm-up, also tells whether the config applies
        if (rc != MMBO_OK) return rc;
        const int reps = 10;
        float t = 0.0f;
        hipEvent_t e0, e1;
        GPU_TIMER_START(t, e0, e1);
        for (int r = 0; r < reps; ++r) call(id);
        GPU_TIMER_END(t, e0, e1);
        *seconds = t / reps;
        return (int)MMBO_OK;
    };
    const char *tn = ta ? "T" : "N", *tbn = tb ? "T" : "N", *dn = dtype == MMBO_F16 ? "hgemm" : dtype == MMBO_F64 ? "dgemm" : "sgemm";
    const double flops = 2.0 * (double)M * N * K * batch;
    if (type == 0) {
        int id = mmbo_select_config(dtype, ta, tb, M, N, K, batch);
        if (id < 0) MMBO_CHECK(-id);
        float t = 0.0f;
        MMBO_CHECK(time_config(id, &t));
        mmbo_config_desc d;
        MMBO_CHECK(mmbo_config_info(dtype, id, &d));
        double tf = 1e-12 * flops / t;
        std::printf("%s(%s%s): kernel, m, n, k, lda, ldb, time, tflops, efficiency = %d (%s), %zu, %zu, %zu, %zu, %zu, %.6f, %.3f, %.2f%%\n",
                    dn, tn, tbn, id, d.name, M, N, K, lda, ldb, t, tf, tf / peak_tflops(dtype) * 100.0);
    } else {
        double best = 0.0;
        int best_id = -1;
        float best_t = 0.0f;
        for (int id = 0; id < mmbo_num_configs(dtype); ++id) {
            float t = 0.0f;
            int rc = time_config(id, &t);
            if (rc == MMBO_ERR_INVALID_CONFIG) continue;      // config does not apply to this shape
            MMBO_CHECK(rc);
            double tf = 1e-12 * flops / t;
            if (tf > best) { best = tf; best_id = id; best_t = t; }
        }
        mmbo_config_desc d;
        MMBO_CHECK(mmbo_config_info(dtype, best_id, &d));
        std::printf("%s(%s%s): kernel, m, n, k, lda, ldb, time, tflops, efficiency = %d (%s), %zu, %zu, %zu, %zu, %zu, %.6f, %.3f, %.2f%%\n",
                    dn, tn, tbn, best_id, d.name, M, N, K, lda, ldb, best_t, best, best / peak_tflops(dtype) * 100.0);
    }
    HIP_CHECK(hipFree(dA));
    HIP_CHECK(hipFree(dB));
    HIP_CHECK(hipFree(dC));
    return 0;
}
