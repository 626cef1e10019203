// Microbenchmark of the generated tile step (attn_pipe_gen.h) on its own: 8 waves per workgroup run
// the two halves of the step on tiles that stay in LDS, one barrier per step as in the kernel, and
// report shader cycles (s_memtime) and nanoseconds (s_memrealtime, 100 MHz) per step.  Optionally
// every step also issues the wave's four direct-to-LDS tile loads from a 32 MiB buffer that stays in
// the memory-side cache.  Three timing variants of the blocks (gen_pipe_step.py: `only`) hold one
// class of instructions each -- the matrix instructions, the softmax arithmetic, the operand reads
// from LDS -- and give what each class costs alone; their results are meaningless.
//
// Built by diffulex_amd/build.py into diffulex_amd/build/step_bench; usage: step_bench [steps]
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "attn_pipe_gen.h"
#include "../build/step_only_mfma.h"
#include "../build/step_only_valu.h"
#include "../build/step_only_lds.h"

#define CHECK(x)                                                              \
    do {                                                                      \
        hipError_t e_ = (x);                                                  \
        if (e_ != hipSuccess) {                                               \
            std::printf("%s: %s\n", #x, hipGetErrorString(e_));               \
            std::exit(1);                                                     \
        }                                                                     \
    } while (0)

namespace {

using namespace dfx;

#define STEP_BLOCKS(NAME, NS)                                                                                          \
    struct NAME {                                                                                                      \
        static DFX_D void ab_x(uint32_t k, uint32_t v, float c, float nm, float& l) { NS::pipe_step_ab_x(k, v, c, nm, l); } \
        static DFX_D void ab_y(float c, float nm, float& l, float& mx) { NS::pipe_step_ab_y(c, nm, l, mx); }            \
        static DFX_D void ba_x(uint32_t k, uint32_t v, float c, float nm, float& l) { NS::pipe_step_ba_x(k, v, c, nm, l); } \
        static DFX_D void ba_y(float c, float nm, float& l, float& mx) { NS::pipe_step_ba_y(c, nm, l, mx); }            \
    }
STEP_BLOCKS(Full, dfx);
STEP_BLOCKS(OnlyMfma, dfx_only_mfma);
STEP_BLOCKS(OnlyValu, dfx_only_valu);
STEP_BLOCKS(OnlyLds, dfx_only_lds);

constexpr int kWaves = 8, kStages = 4, kStageBytes = 32768, kMatBytes = 16384;
constexpr int kCachedTiles = 1024;  // 32 MiB: stays in the memory-side cache

DFX_D int swizzle(int row) { return ((row & 3) << 2) | ((row >> 2) & 3); }

template <typename B>
__global__ void __launch_bounds__(64 * kWaves, 1) __attribute__((amdgpu_num_vgpr(32)))
step_kernel(const uint8_t* q, const uint8_t* tiles, long long* out, int steps, int with_loads) {
    extern __shared__ __attribute__((aligned(256))) uint8_t smem[];
    pipe_reserve();
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int col = lane & 31, half = lane >> 5;
    for (int i = threadIdx.x; i < kStages * kStageBytes / 4; i += 64 * kWaves) {
        const uint32_t h = (i * 2654435761u) ^ (blockIdx.x * 40503u);
        reinterpret_cast<uint32_t*>(smem)[i] = (h & 0x807f807fu) | 0x3e803e80u;  // bf16 pairs in (-1, 1)
    }
    __syncthreads();
    // the lane's operand offsets, as TileMath computes them (attn_tile.h)
    const uint32_t base = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(smem));
    const uint32_t k_lane = col * 256 + ((half ^ swizzle(col)) * 16);
    const int g16 = lane >> 4, sl16 = lane & 15;
    const int lrow = (g16 >> 1) * 4 + (sl16 >> 2), chunk = (g16 & 1) * 2 + ((sl16 & 3) >> 1);
    const uint32_t v_lane = lrow * 256 + ((chunk ^ swizzle(lrow)) * 16) + (sl16 & 1) * 8;
    pipe_set_load_offsets((lane >> 4) * 256 + (lane & 15) * 16, ((lane >> 4) + 4) * 256 + (lane & 15) * 16);
    pipe_zero_outputs();
    pipe_issue_queries(q + ((wave * 32 + col) * 256 + half * 16));
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    float l = 0.0f, mx = 0.0f;
    const float c = 0.02f, neg_m = -1.0f;
    pipe_first_scores(base + k_lane, mx);
    asm volatile("" ::"v"(mx));
    __syncthreads();
    const long long c0 = __builtin_readcyclecounter();
    const long long t0 = __builtin_amdgcn_s_memrealtime();
    auto half_step = [&](int r, bool cur_is_a) {
        if (with_loads) asm volatile("s_waitcnt vmcnt(4)" ::: "memory");  // the unit two steps ahead may be on its way
        __builtin_amdgcn_s_barrier();
        if (with_loads) {
            const uint32_t dst = __builtin_amdgcn_readfirstlane(base + ((r + 3) % kStages) * kStageBytes + wave * 2048);
            const uint8_t* p = tiles + static_cast<size_t>((blockIdx.x * 37 + r) % kCachedTiles) * kStageBytes + wave * 2048;
            pipe_issue_band(p, p + kMatBytes, dst);
        }
        const uint32_t k_next = base + ((r + 1) % kStages) * kStageBytes + k_lane;
        const uint32_t v_cur = base + (r % kStages) * kStageBytes + kMatBytes + v_lane;
        if (cur_is_a) {
            B::ab_x(k_next, v_cur, c, neg_m, l);
            B::ab_y(c, neg_m, l, mx);
        } else {
            B::ba_x(k_next, v_cur, c, neg_m, l);
            B::ba_y(c, neg_m, l, mx);
        }
        asm volatile("" ::"v"(mx));
    };
    for (int r = 0; r < steps; r += 2) {
        half_step(r, true);
        half_step(r + 1, false);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    const long long c1 = __builtin_readcyclecounter();
    const long long t1 = __builtin_amdgcn_s_memrealtime();
    pipe_outputs_ready();
    const f32x16 o0 = pipe_get_output(0);
    if (lane == 0) {
        long long* rec = out + (static_cast<size_t>(blockIdx.x) * kWaves + wave) * 4;
        rec[0] = c1 - c0;
        rec[1] = t1 - t0;
        rec[2] = static_cast<long long>(o0[0] + l);  // (keeps the arithmetic alive)
    }
}

template <typename B>
void run(const char* name, int grid, int steps, int with_loads, const uint8_t* q, const uint8_t* tiles, long long* out) {
    CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(step_kernel<B>), hipFuncAttributeMaxDynamicSharedMemorySize,
                              kStages * kStageBytes));
    for (int rep = 0; rep < 3; ++rep) {
        hipLaunchKernelGGL(step_kernel<B>, dim3(grid), dim3(64 * kWaves), kStages * kStageBytes, 0, q, tiles, out, steps, with_loads);
        CHECK(hipDeviceSynchronize());
    }
    std::vector<long long> h(static_cast<size_t>(grid) * kWaves * 4);
    CHECK(hipMemcpy(h.data(), out, h.size() * sizeof(long long), hipMemcpyDeviceToHost));
    std::vector<double> cycles, ns;
    for (size_t i = 0; i < h.size(); i += 4) {
        cycles.push_back(static_cast<double>(h[i]) / steps);
        ns.push_back(static_cast<double>(h[i + 1]) * 10.0 / steps);
    }
    std::sort(cycles.begin(), cycles.end());
    std::sort(ns.begin(), ns.end());
    const double cm = cycles[cycles.size() / 2], nm = ns[ns.size() / 2];
    std::printf("%-28s %4d workgroups  tile loads %-3s  %5.0f cycles/step  %5.0f ns/step  %.2f GHz\n", name, grid,
                with_loads ? "yes" : "no", cm, nm, cm / nm);
}

}  // namespace

int main(int argc, char** argv) {
    const int steps = argc > 1 ? std::max(2, std::atoi(argv[1]) & ~1) : 2000;
    hipDeviceProp_t prop;
    CHECK(hipGetDeviceProperties(&prop, 0));
    const int cus = prop.multiProcessorCount;
    uint8_t *q, *tiles;
    long long* out;
    CHECK(hipMalloc(&q, 1 << 20));
    CHECK(hipMemset(q, 0x3c, 1 << 20));
    CHECK(hipMalloc(&tiles, static_cast<size_t>(kCachedTiles) * kStageBytes));
    CHECK(hipMemset(tiles, 0x3c, static_cast<size_t>(kCachedTiles) * kStageBytes));
    CHECK(hipMalloc(&out, static_cast<size_t>(cus) * kWaves * 4 * sizeof(long long)));
    std::printf("%d steps of one 64-token tile x 256 query rows x head_dim 128 per workgroup (8 waves), %d compute units\n", steps, cus);
    for (int grid : {1, cus}) {
        for (int loads = 0; loads < 2; ++loads) run<Full>("the step", grid, steps, loads, q, tiles, out);
        run<OnlyMfma>("matrix instructions only", grid, steps, 0, q, tiles, out);
        run<OnlyValu>("softmax arithmetic only", grid, steps, 0, q, tiles, out);
        run<OnlyLds>("operand reads only", grid, steps, 0, q, tiles, out);
    }
    return 0;
}
