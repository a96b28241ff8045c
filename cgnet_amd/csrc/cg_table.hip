// Clebsch-Gordan table on the device: one thread per table entry, Racah sum in double.
#include <vector>

#include "common.h"

namespace cgnet {
namespace {

struct TableTriple {
    int l, l1, l2;
    int offset;   // first float of this triple's (2l+1) x (2l2+1) table
};

// log(n!) for n < nfact, built per block in LDS from lgamma
__device__ __forceinline__ double racah_sum(const double* lf, int l1, int m1, int l2, int m2, int l, int m) {
    const int k_lo = max(0, max(l2 - m1 - l, l1 + m2 - l));
    const int k_hi = min(l1 + l2 - l, min(l1 - m1, l2 + m2));
    double head = 0.5 * (log(2.0 * l + 1.0) + lf[l + l1 - l2] + lf[l - l1 + l2] + lf[l1 + l2 - l] -
                         lf[l1 + l2 + l + 1] + lf[l + m] + lf[l - m] + lf[l1 - m1] + lf[l1 + m1] +
                         lf[l2 - m2] + lf[l2 + m2]);
    double acc = 0.0;
    for (int k = k_lo; k <= k_hi; ++k) {
        double tail = lf[k] + lf[l1 + l2 - l - k] + lf[l1 - m1 - k] + lf[l2 + m2 - k] +
                      lf[l - l2 + m1 + k] + lf[l - l1 - m2 + k];
        double term = exp(head - tail);
        acc += (k & 1) ? -term : term;
    }
    return acc;
}

__global__ void __launch_bounds__(256) cg_table_kernel(float* __restrict__ cg,
                                                        const TableTriple* __restrict__ triples,
                                                        int nfact) {
    extern __shared__ double lf[];
    for (int n = threadIdx.x; n < nfact; n += blockDim.x) lf[n] = lgamma((double)n + 1.0);
    __syncthreads();
    const TableTriple t = triples[blockIdx.x];
    const int M = 2 * t.l + 1, M2 = 2 * t.l2 + 1;
    for (int e = threadIdx.x; e < M * M2; e += blockDim.x) {
        const int m = e / M2 - t.l, m2 = e % M2 - t.l2;
        const int m1 = m - m2;
        float v = 0.f;
        if (m1 >= -t.l1 && m1 <= t.l1) v = (float)racah_sum(lf, t.l1, m1, t.l2, m2, t.l, m);
        cg[t.offset + e] = v;
    }
}

}  // namespace
}  // namespace cgnet

extern "C" int cgnet_sparse_precomputeCG(float* d_CG, int L, const int* h_llls, int nllls,
                                         const int* h_CG_offsets, void* stream) {
    using namespace cgnet;
    clear_error();
    CGNET_REQUIRE(L >= 0 && L <= kMaxL, CGNET_ERR_UNSUPPORTED, "lmax=%d outside [0, %d]", L, kMaxL);
    CGNET_REQUIRE(nllls >= 0, CGNET_ERR_ARG, "nllls=%d is negative", nllls);
    if (nllls == 0) return CGNET_OK;
    CGNET_REQUIRE(d_CG && h_llls && h_CG_offsets, CGNET_ERR_ARG, "null pointer argument");
    std::vector<TableTriple> tr(nllls);
    const int n1 = L + 1;
    for (int i = 0; i < nllls; ++i) {
        const int c = h_llls[i];
        CGNET_REQUIRE(c >= 0 && c < n1 * n1 * n1, CGNET_ERR_ARG, "llls[%d]=%d is not a triple code for lmax=%d", i, c, L);
        TableTriple t{c / (n1 * n1), (c / n1) % n1, c % n1, h_CG_offsets[i]};
        CGNET_REQUIRE(t.l1 >= t.l2 && t.l1 - t.l2 <= t.l && t.l <= t.l1 + t.l2, CGNET_ERR_ARG,
                      "triple %d = (l=%d, l1=%d, l2=%d) violates l1>=l2 or the triangle rule", i, t.l, t.l1, t.l2);
        CGNET_REQUIRE(h_CG_offsets[i] >= 0 &&
                      h_CG_offsets[i + 1] - h_CG_offsets[i] == (2 * t.l + 1) * (2 * t.l2 + 1),
                      CGNET_ERR_ARG, "CG_offsets[%d..%d] does not span (2l+1)(2l2+1) entries", i, i + 1);
        tr[i] = t;
    }
    hipStream_t s = (hipStream_t)stream;
    TableTriple* d_tr = nullptr;
    CGNET_HIP(hipMallocAsync((void**)&d_tr, sizeof(TableTriple) * nllls, s));
    CGNET_HIP(hipMemcpyAsync(d_tr, tr.data(), sizeof(TableTriple) * nllls, hipMemcpyHostToDevice, s));
    const int nfact = 3 * L + 2;   // largest argument is l1 + l2 + l + 1
    CGNET_LAUNCH(cg_table_kernel, dim3(nllls), dim3(256), sizeof(double) * nfact, s, d_CG, d_tr, nfact);
    CGNET_HIP(hipGetLastError());
    // the host vector must outlive the async copy
    CGNET_HIP(hipStreamSynchronize(s));
    CGNET_HIP(hipFreeAsync(d_tr, s));
    return CGNET_OK;
}
