// K split over several workgroups per tile, for products with few tiles and a long K (a [256, 4096] output has 64 tiles
// of 128 x 128 for 256 CUs): split z multiplies its share of K into the fp32 array partial[z][M][N] of a caller-provided
// workspace, on the 128 x 128, 256 x 128 or 512 x 128 tile kernel, and a second kernel adds the arrays, the bias, and rounds to
// the output type.
// (included from gemm_impl.h, inside namespace mase, after gemm_mid.h and gemm_wide.h)

struct SplitPlan {
    int splits;  // 1: do not split
    int k_len;   // k per split, a multiple of 128
    int kind;    // 0: 128 x 128 tiles, 1: 256 x 128 tiles, 2: 512 x 128 tiles
    int64_t workspace_bytes(int M, int N) const { return splits > 1 ? (int64_t)splits * M * N * 4 : 0; }
};

// Estimated time of one 128-k macro step of a 128 x 128 tile, in us, by the share of the CUs that have a workgroup
// (measured: 0.6 with a handful of workgroups, 1.1 at a quarter of the CUs, 1.6 with all of them busy: L2 bandwidth).
inline double split_step_us(int64_t wgs, int cus) {
    const double share = wgs >= cus ? 1.0 : (double)wgs / cus;
    if (share <= 1.0 / 32) return 0.6;
    if (share <= 0.25) return 1.1;
    return 1.1 + 0.5 * (share - 0.25) / 0.75;
}

// The same plan for the size query and the launch: it depends on the shape and the CU count only.  Every candidate
// (tile kind, number of splits) is priced as rounds x macro steps per split x step time x (1.0 / 1.4 / 2.05 for 128 / 256 /
// 512-row tiles), plus, when split, 4 us for the second launch and the partial sums written and read once at 4.7 TB/s
// (K = 1024 in two splits of a [512, 4096] output was 24 us against 16 us unsplit); the cheapest wins, and if that is
// an unsplit one the plan says so.
inline SplitPlan plan_split_k(int M, int N, int K, int cus, bool allow_tall = true) {
    SplitPlan p{1, K, 0};
    // up to 64 rows the weight-streaming kernels are as fast or faster (64 x 4096 x 4096: 14.5 us against 20.4 us split)
    if (M <= 64 || N % 128 != 0 || K % 128 != 0 || cus <= 0) return p;
    const int nmac = K / 128;
    const int64_t n128 = N / 128;
    const double mn_mb = (double)M * N * 4.0 / 1e6;
    auto price = [&](int rows, double rel, int mac_per, int splits) {
        const int64_t wgs = (int64_t)((M + rows - 1) / rows) * n128 * splits;
        const double rounds = (double)((wgs + cus - 1) / cus);
        return rounds * mac_per * rel * split_step_us(wgs, cus) + (splits > 1 ? 4.0 + (2.0 * splits + 0.5) * mn_mb * 0.21 : 0.0);
    };
    double best = price(128, 1.0, nmac, 1);
    if (M > 128) best = std::min(best, price(256, 1.4, nmac, 1));
    if (M >= 512) best = std::min(best, price(512, 2.05, nmac, 1));
    for (int kind = 0; kind < 3; ++kind) {
        if (kind == 1 && M <= 256) continue;                       // a 256-row tile would be mostly empty rows
        if (kind == 2 && (M < 512 || !allow_tall)) continue;
        const int rows = 128 << kind;
        const double rel = kind == 0 ? 1.0 : kind == 1 ? 1.4 : 2.05;
        const int64_t tiles = (int64_t)((M + rows - 1) / rows) * n128;
        if (tiles * 2 > cus) continue;                             // a second workgroup per tile would not find a free CU
        int most = (int)(cus / tiles);
        // macro steps per split at least: 4, and 24 on the larger tiles, whose longer prologue and larger fp32 tile only pay
        // over a long run (512 x 4096 x 4096: 38 us on 256 x 128 tiles in four splits of 8 against 34 us on 128 x 128 tiles
        // in two of 16)
        const int least = kind == 0 ? 4 : 24;
        if (most > nmac / least) most = nmac / least;
        if (most > 16) most = 16;
        for (int want = 2; want <= most; ++want) {
            if (kind == 2 && nmac % want != 0) continue;           // the 512 x 128 kernel walks equal shares only
            const int mac_per = (nmac + want - 1) / want;
            const int splits = (nmac + mac_per - 1) / mac_per;     // no empty split
            const double t = price(rows, rel, mac_per, splits);
            if (t < best) {
                best = t;
                p.splits = splits;
                p.k_len = mac_per * 128;
                p.kind = kind;
            }
        }
    }
    return p;
}

template <int DT_OUT>
__global__ __launch_bounds__(256) void split_k_reduce_kernel(const float* __restrict__ partial, int splits, int64_t mn, int N,
                                                             const void* __restrict__ bias, int bias_dtype, void* __restrict__ y) {
    // a lane adds four consecutive outputs of every split (N % 4 == 0: they share a row)
    const int64_t o = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
    if (o >= mn) return;
    float4 acc = *reinterpret_cast<const float4*>(partial + o);
    for (int z = 1; z < splits; ++z) {
        const float4 v = *reinterpret_cast<const float4*>(partial + (size_t)z * mn + o);
        acc.x += v.x; acc.y += v.y; acc.z += v.z; acc.w += v.w;
    }
    float r[4] = {acc.x, acc.y, acc.z, acc.w};
    if (bias) {
        const int n = (int)(o % N);
#pragma unroll
        for (int t = 0; t < 4; ++t) r[t] += load_bias(bias, bias_dtype, n + t);
    }
    store_out4<DT_OUT>(y, o, r, (reinterpret_cast<uintptr_t>(y) & 15) == 0, 4);
}

template <class FW, int DT_OUT>
int launch_gemm_split_k(const void* a_dense, const uint8_t* w_scales, const uint8_t* w_elements, const void* bias, int bias_dtype,
                        void* y, int M, int N, int K, const SplitPlan& plan, void* workspace, hipStream_t s) {
    const int64_t mn = (int64_t)M * N;
    if (plan.kind == 0) {
        auto kern = mxfp_gemm_mid_kernel<FW, F32, 2>;
        static std::atomic<uint64_t> lds_allowed{0};
        if (int rc = allow_dynamic_lds(reinterpret_cast<const void*>(kern), MD_LDS_BYTES, lds_allowed)) return rc;
        const int tiles_m = (M + MD_M - 1) / MD_M;
        hipLaunchKernelGGL(kern, dim3((unsigned)(tiles_m * (N / MD_N)), (unsigned)plan.splits), dim3(512), MD_LDS_BYTES, s,
                           static_cast<const uint16_t*>(a_dense), w_scales, w_elements, static_cast<const void*>(nullptr), 0, workspace,
                           M, N, K, tiles_m, plan.k_len, mn * 4, GemmBatch{0, 0, 0, 0});
    } else if (plan.kind == 1) {
        auto kern = mxfp_gemm_wide_kernel<FW, F32>;
        static std::atomic<uint64_t> lds_allowed{0};
        if (int rc = allow_dynamic_lds(reinterpret_cast<const void*>(kern), WD_LDS_BYTES, lds_allowed)) return rc;
        const int tiles_m = (M + WD_M - 1) / WD_M;
        hipLaunchKernelGGL(kern, dim3((unsigned)(tiles_m * (N / WD_N)), (unsigned)plan.splits), dim3(WD_THREADS), WD_LDS_BYTES, s,
                           static_cast<const uint16_t*>(a_dense), w_scales, w_elements, static_cast<const void*>(nullptr), 0, workspace,
                           M, N, K, tiles_m, plan.k_len, mn * 4, GemmBatch{0, 0, 0, 0});
    } else {
        const bool sc4 = plan.k_len % 512 == 0;
        auto kern = sc4 ? mxfp_gemm_tall_kernel<FW, F32, true> : mxfp_gemm_tall_kernel<FW, F32, false>;
        static std::atomic<uint64_t> lds_allowed[2] = {{0}, {0}};
        if (int rc = allow_dynamic_lds(reinterpret_cast<const void*>(kern), U_LDS_BYTES, lds_allowed[sc4])) return rc;
        const int tiles_m = (M + UM - 1) / UM;
        const int walks = tiles_m * (N / UN) * plan.splits;          // at most one per CU (the plan splits only then)
        hipLaunchKernelGGL(kern, dim3((unsigned)((walks + 7) / 8 * 8)), dim3(kGemmThreads), U_LDS_BYTES, s,
                           static_cast<const uint16_t*>(a_dense), w_scales, w_elements, static_cast<const void*>(nullptr), 0, workspace,
                           M, N, K, tiles_m, N / UN, plan.splits, mn * 4, GemmBatch{0, 0, 0, 0}, 0);
    }
    if (int rc = check_launch("mxfp_gemm")) return rc;
    hipLaunchKernelGGL(split_k_reduce_kernel<DT_OUT>, dim3((unsigned)((mn / 4 + 255) / 256)), dim3(256), 0, s,
                       static_cast<const float*>(workspace), plan.splits, mn, N, bias, bias_dtype, y);
    return check_launch("mxfp_gemm");
}
