// Issue-rate probe for the grouped-scale FP8 GEMM (measurement support, no counterpart in the reference).
//
// The chunk loop of group_gemm_fast rebuilt without a GEMM around it: the same block shape (256 threads, 2 x 2
// wavefronts of 2 x 2 sub-tiles, two blocks per CU), the same instruction mix per 64-k chunk and wavefront (16
// v_mfma_f32_32x32x16_fp8_fp8 in pairs over four rotating accumulators, 128 FP32 FMAs folding the previous pair into
// the totals, 8 scale products) and, switched on one by one, the three things a real chunk adds to that math:
//   VIOLA_PROBE_LDS_READS  the 8 ds_read_b128 + 8 ds_read_b32 that fetch the next chunk's operands and scales,
//   VIOLA_PROBE_BARRIER    the one barrier per chunk,
//   VIOLA_PROBE_LOADS      the four 16-byte-per-lane global -> LDS loads of a wavefront, addressed like the tile loader
//                          (128-row tiles of a row-major byte matrix with row stride `lda`, 64 k per chunk).
// Timing a launch of `blocks` blocks over `chunks` chunks gives the time per chunk that this instruction mix needs on
// the machine when nothing else is in the way: what the kernel could reach at best with its tiling, and what each part
// costs. The result values are meaningless (operands are whatever the LDS and `src` hold).
#include "common.hpp"

namespace viola {

typedef float probe_f32x16 __attribute__((ext_vector_type(16)));
typedef int probe_i32x4 __attribute__((ext_vector_type(4)));

constexpr int PROBE_STAGE = 16384, PROBE_RING = 3 * PROBE_STAGE, PROBE_LDS = PROBE_RING + 24576;

__device__ __forceinline__ void probe_load_to_lds(probe_i32x4 rsrc, uint32_t lds_addr, uint32_t voffset, uint32_t soffset) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                 :: "s"(lds_addr), "v"(voffset), "s"(rsrc), "s"(soffset) : "memory");
}

struct ProbeOperands { uint4 a[2][2], b[2][2]; float sa[2][2], sb[2][2]; };

template <int PARTS>
__global__ __launch_bounds__(256, 2) void probe_chunk_loop_kernel(float* out, const uint8_t* src, int chunks, int lda) {
    constexpr bool LDS_READS = PARTS & 1, BARRIER = PARTS & 2, LOADS = PARTS & 4;
    __shared__ __attribute__((aligned(1024))) uint8_t lds[PROBE_LDS];
    const int tid = threadIdx.x, lane = tid % WAVE, wave = __builtin_amdgcn_readfirstlane(tid / WAVE);
    const int wm = wave / 2, wn = wave % 2, l32 = lane % 32, lhi = lane / 32;
    for (int i = tid * 16; i < PROBE_LDS; i += 256 * 16)
        *reinterpret_cast<uint4*>(lds + i) = make_uint4(0x38383838u + i, 0x3c3c3838u, 0x38343834u, 0x30383c38u);
    __syncthreads();
    const uint64_t address = reinterpret_cast<uint64_t>(src);
    const probe_i32x4 resource = {__builtin_amdgcn_readfirstlane((int)(uint32_t)address),
                                  __builtin_amdgcn_readfirstlane((int)(uint32_t)(address >> 32)), 0x7fffffff, 0x00020000};
    const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)lds;
    const int sw = (l32 >> 2) & 3;
    const int rd_a = (wm * 64 + l32) * 64 + ((lhi ^ sw) * 16), rd_b = (wn * 64 + l32) * 64 + ((lhi ^ sw) * 16);
    // the tile loader's plan: instruction `it` of an operand covers 64 rows, four lanes per 64-byte row piece; the a
    // operand has 64 row tiles and the b operand 8 (the 8192 x 1024 x 4096 product), blocks share them as the GEMM's do
    uint32_t offset[4];
    for (int it = 0; it < 4; ++it) {
        const int unit = (it & 1) * 256 + tid, r = unit >> 2, piece = (unit & 3) ^ ((r >> 2) & 3);
        const int tile = it < 2 ? blockIdx.x % 64 : 64 + blockIdx.x % 8;
        offset[it] = (uint32_t)((tile * 128 + r) * lda + piece * 16);
    }
    probe_f32x16 acc[4], total[4];
    const probe_f32x16 zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
    for (int i = 0; i < 4; ++i) { acc[i] = zero; total[i] = zero; }
    auto as_long = [](uint32_t lo, uint32_t hi) -> long { return (long)(((uint64_t)hi << 32) | lo); };
    auto read_operands = [&](int stage, int c, ProbeOperands& o) {
        const uint8_t* tile_a = lds + stage * PROBE_STAGE;
        const uint8_t* tile_b = tile_a + PROBE_STAGE / 2;
        const float* scales = reinterpret_cast<const float*>(lds + PROBE_RING + 8192 + ((c / 4) & 1) * 8192) + (c % 4) * 256;
#pragma unroll
        for (int kg = 0; kg < 2; ++kg) {
#pragma unroll
            for (int j = 0; j < 2; ++j) o.a[kg][j] = *reinterpret_cast<const uint4*>(tile_a + ((rd_a + j * 2048) ^ (kg * 32)));
#pragma unroll
            for (int i = 0; i < 2; ++i) o.b[kg][i] = *reinterpret_cast<const uint4*>(tile_b + ((rd_b + i * 2048) ^ (kg * 32)));
#pragma unroll
            for (int j = 0; j < 2; ++j) o.sa[kg][j] = scales[kg * 128 + wm * 64 + j * 32 + l32];
#pragma unroll
            for (int i = 0; i < 2; ++i) o.sb[kg][i] = scales[1024 + kg * 128 + wn * 64 + i * 32];
        }
    };
    float pending[2] = {0.0f, 0.0f};
    auto compute = [&](const ProbeOperands& o, int c, int fill) {
#pragma unroll
        for (int pair = 0; pair < 4; ++pair) {
            const int base = (pair & 1) * 2, other = base ^ 2;
            int kg[2], ti[2], tj[2];
#pragma unroll
            for (int h = 0; h < 2; ++h) { const int unit = 2 * pair + h; kg[h] = unit / 4; ti[h] = unit / 2 % 2; tj[h] = unit % 2; }
#pragma unroll
            for (int step = 0; step < 4; ++step) {
                const int h = step & 1;
                const uint4 ob = o.b[kg[h]][ti[h]], oa = o.a[kg[h]][tj[h]];
                if (step < 2) acc[base + h] = __builtin_amdgcn_mfma_f32_32x32x16_fp8_fp8(as_long(ob.x, ob.y), as_long(oa.x, oa.y), zero, 0, 0, 0);
                else acc[base + h] = __builtin_amdgcn_mfma_f32_32x32x16_fp8_fp8(as_long(ob.z, ob.w), as_long(oa.z, oa.w), acc[base + h], 0, 0, 0);
                const int folded = other + (step >> 1), half = step & 1, into = (pair + 3) & 3;
#pragma unroll
                for (int r = 8 * half; r < 8 * half + 8; ++r) total[into][r] = fmaf(acc[folded][r], pending[step >> 1], total[into][r]);
                asm volatile("" : "+v"(total[into]));
                __builtin_amdgcn_sched_barrier(0);
                if (LOADS && step == 0)
                    probe_load_to_lds(resource, lds_base + fill * PROBE_STAGE + wave * 1024 + pair * 4096, offset[pair], (uint32_t)(c % (lda / 64)) * 64);
            }
#pragma unroll
            for (int h = 0; h < 2; ++h) pending[h] = o.sa[kg[h]][tj[h]] * o.sb[kg[h]][ti[h]];
        }
    };
    ProbeOperands set0, set1;
    read_operands(0, 0, set0);
    if (!LDS_READS) set1 = set0;
    int stage_now = 0, stage_next = 1;
    auto chunk = [&](int c, const ProbeOperands& now, ProbeOperands& next) {
        __builtin_amdgcn_s_waitcnt(LOADS ? 0x0070 | 4 : 0x0070 | 15);        // as the GEMM: the loads of the chunk after the next may be in flight
        if (BARRIER) __syncthreads();
        if (LDS_READS) read_operands(stage_next, c + 1, next);
        compute(now, c, stage_now);
        stage_now = stage_next;
        stage_next = stage_next == 2 ? 0 : stage_next + 1;
    };
    for (int c = 0; c < chunks; c += 2) { chunk(c, set0, set1); chunk(c + 1, set1, set0); }
    __builtin_amdgcn_s_waitcnt(0x0F70);                                      // no load may land after the LDS allocation is released
    float sum = 0.0f;
    for (int i = 0; i < 16; ++i) sum += total[0][i] + total[1][i] + total[2][i] + total[3][i] + acc[0][i] + acc[1][i] + acc[2][i] + acc[3][i];
    out[(int64_t)blockIdx.x * 256 + tid] = sum;
}

}  // namespace viola

using namespace viola;

extern "C" int viola_probe_chunk_loop(int parts, float* out, const void* src, int64_t src_bytes, int blocks, int chunks, int lda,
                                      viola_stream_t stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    VIOLA_CHECK_ARG(parts >= 0 && parts < 8 && out && blocks > 0 && blocks <= 65535 && chunks > 0 && chunks % 2 == 0);
    VIOLA_CHECK_ARG(lda >= 64 && lda % 64 == 0);
    // 72 row tiles of 128 rows, and the last chunk's 64 bytes of the last row
    VIOLA_CHECK_ARG(!(parts & 4) || (src && reinterpret_cast<uintptr_t>(src) % 16 == 0 && src_bytes >= (int64_t)72 * 128 * lda &&
                                      (int64_t)72 * 128 * lda < (1ll << 31)));
    const uint8_t* bytes = static_cast<const uint8_t*>(src);
    switch (parts) {
        case 0: VIOLA_LAUNCH((probe_chunk_loop_kernel<0>), dim3(blocks), dim3(256), 0, stream, out, bytes, chunks, lda); break;
        case 1: VIOLA_LAUNCH((probe_chunk_loop_kernel<1>), dim3(blocks), dim3(256), 0, stream, out, bytes, chunks, lda); break;
        case 2: VIOLA_LAUNCH((probe_chunk_loop_kernel<2>), dim3(blocks), dim3(256), 0, stream, out, bytes, chunks, lda); break;
        case 3: VIOLA_LAUNCH((probe_chunk_loop_kernel<3>), dim3(blocks), dim3(256), 0, stream, out, bytes, chunks, lda); break;
        case 4: VIOLA_LAUNCH((probe_chunk_loop_kernel<4>), dim3(blocks), dim3(256), 0, stream, out, bytes, chunks, lda); break;
        case 5: VIOLA_LAUNCH((probe_chunk_loop_kernel<5>), dim3(blocks), dim3(256), 0, stream, out, bytes, chunks, lda); break;
        case 6: VIOLA_LAUNCH((probe_chunk_loop_kernel<6>), dim3(blocks), dim3(256), 0, stream, out, bytes, chunks, lda); break;
        default: VIOLA_LAUNCH((probe_chunk_loop_kernel<7>), dim3(blocks), dim3(256), 0, stream, out, bytes, chunks, lda); break;
    }
    return viola_launch_status();
}
