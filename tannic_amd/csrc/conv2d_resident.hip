// conv2d on MFMA with the weights resident in LDS — the fast path for 16-bit
// signals when one output-channel tile's complete weights fit next to an input
// patch.
//
// Persistent blocks: a block of 256 threads first copies the weights of its BCO
// output channels for ALL taps and input channels into LDS, arranged as
// [tap][channel chunk of 32][BCO][32] from a tap-major copy made once per
// call, and then walks over (image, row block) tiles.  For each tile it holds
// the input patch — the (R-1)*stride + KH input rows the R output rows need,
// all channels — in LDS channels-last, as in the chunked patch kernel:
// [channel chunk][row][column + padding][32 channels] with real zeros in the
// padding.  The 16-byte global loads of the NEXT tile's patch are issued before
// the MFMAs of the current tile and transposed (8x8 micro-blocks) into LDS after
// them, so their latency hides behind about 4 K cycles of matrix work.
// The MFMA loop walks (tap, 32-channel chunk) steps with running offsets; the
// operands of step i+1 are requested before the MFMAs of step i.  No range test,
// no global access, no division inside.
#include "conv_common.hpp"

namespace th {

typedef _Float16 half8r __attribute__((ext_vector_type(8)));
typedef __bf16 bfloat8r __attribute__((ext_vector_type(8)));
typedef float float16r __attribute__((ext_vector_type(16)));
typedef unsigned int uint4r __attribute__((ext_vector_type(4)));

template <class T> __device__ inline float16r resident_mfma(uint4r a, uint4r b, float16r c) {
    if constexpr (std::is_same_v<T, f16>) {
        half8r x, y;
        __builtin_memcpy(&x, &a, 16);
        __builtin_memcpy(&y, &b, 16);
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(x, y, c, 0, 0, 0);
    } else {
        bfloat8r x, y;
        __builtin_memcpy(&x, &a, 16);
        __builtin_memcpy(&y, &b, 16);
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(x, y, c, 0, 0, 0);
    }
}

constexpr int kResThreads = 256;
constexpr int kRC = 32;  // channels per LDS record

struct ResidentPlan {
    uint32_t R, IH, IWp, row_blocks, co_tiles, groups, rows_strided;
    uint32_t tiles;        // N * row_blocks
    uint32_t workers;      // blocks per output-channel tile
    uint32_t patch_records;  // IH * IWp
    FastDiv div_cblocks, div_colblocks, div_chunks, div_row_blocks;   // micro-block index -> (channel block, column block, row)
};

__device__ inline uint32_t res_offset(uint32_t rec, uint32_t chunk) { return rec * kRC + ((chunk ^ ((rec >> 2) & 3u)) * 8u); }

// WSPLIT: how many ways the four wavefronts split the output channels (1 or 2);
// the remaining factor splits the pixel groups.  PASSES: micro-blocks per thread.
template <class T, int BCO, int WSPLIT, int PASSES>
__global__ __launch_bounds__(kResThreads) void conv2d_resident_kernel(const T* x, const T* wt, const T* bias, T* y, ConvProblem p, ResidentPlan q) {
    constexpr int TM = BCO / 32 / WSPLIT;
    constexpr int PSPLIT = 4 / WSPLIT;   // wavefronts along pixels
    extern __shared__ __align__(16) unsigned char res_lds[];
    T* wl = reinterpret_cast<T*>(res_lds);
    const uint32_t taps = p.KH * p.KW, chunks = p.C / kRC;
    T* patch = wl + static_cast<size_t>(taps) * chunks * BCO * kRC;

    const uint32_t ct = blockIdx.x % q.co_tiles, worker = blockIdx.x / q.co_tiles;
    const uint32_t co0 = ct * BCO;
    const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
    const int wco = (wave % WSPLIT) * TM * 32;   // first output channel of this wavefront inside the tile
    const int wpx = wave / WSPLIT;               // this wavefront's first pixel group

    // ---- once per block: weights and zeroed patch ------------------------------
    // one [BCO][32] block per (tap, chunk) step; a thread moves the same (row, 16-byte slot) of every block,
    // up to 24 blocks' loads in flight before their LDS writes (no accumulators are live yet)
    {
        const uint32_t steps_total = taps * chunks;
        constexpr int PER_BLOCK = BCO * 4 / kResThreads;   // 16-byte slots per thread and block: 1 (BCO 64) or 2 (BCO 128)
        constexpr int BATCH = 24 / PER_BLOCK;
        for (uint32_t st0 = 0; st0 < steps_total; st0 += BATCH) {
            uint4r v[BATCH][PER_BLOCK];
#pragma unroll
            for (int u = 0; u < BATCH; ++u) {
                const uint32_t st = st0 + u < steps_total ? st0 + u : steps_total - 1;
                const uint32_t tap = q.div_chunks.div(st), chunk = st - tap * chunks;
#pragma unroll
                for (int r = 0; r < PER_BLOCK; ++r) {
                    const uint32_t slot = threadIdx.x + kResThreads * r, ch = slot % 4, row = slot / 4;
                    const uint32_t co = co0 + row < p.O ? co0 + row : p.O - 1;
                    v[u][r] = *reinterpret_cast<const uint4r*>(wt + (static_cast<int64_t>(tap) * p.O + co) * p.C + chunk * kRC + ch * 8);
                }
            }
#pragma unroll
            for (int u = 0; u < BATCH; ++u) {
                if (st0 + u >= steps_total) break;
#pragma unroll
                for (int r = 0; r < PER_BLOCK; ++r) {
                    const uint32_t slot = threadIdx.x + kResThreads * r, ch = slot % 4, row = slot / 4;
                    *reinterpret_cast<uint4r*>(wl + res_offset((st0 + u) * BCO + row, ch)) = v[u][r];
                }
            }
        }
    }
    for (uint32_t i = threadIdx.x; i < chunks * q.patch_records * kRC / 8; i += kResThreads) reinterpret_cast<uint4r*>(patch)[i] = uint4r{0, 0, 0, 0};
    // the lane's pixels inside a tile: groups wpx, wpx + PSPLIT
    const uint32_t npix = q.R * p.WO;
    uint32_t pbase[2], prow_of[2], pcol_of[2];
    bool group_live[2], pixel_live[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const uint32_t g = wpx + PSPLIT * j;
        group_live[j] = g < q.groups;
        const uint32_t qp = g * 32 + lane % 32;
        pixel_live[j] = group_live[j] && qp < npix;
        const uint32_t r = pixel_live[j] ? qp / p.WO : 0, ow = pixel_live[j] ? qp % p.WO : 0;
        prow_of[j] = r;
        pcol_of[j] = ow;
        pbase[j] = (q.rows_strided ? r : r * p.stride_h) * q.IWp + ow * p.stride_w;
    }
    float bias_v[TM][16];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const uint32_t co = co0 + wco + i * 32 + 8 * (v / 4) + 4 * (lane / 32) + v % 4;
            bias_v[i][v] = (p.has_bias && co < p.O) ? static_cast<float>(widen(bias[static_cast<int64_t>(co) * p.bs])) : 0.0f;
        }

    // ---- patch staging: global -> registers (fetch), registers -> LDS (commit) ------------------
    const uint32_t microblocks = (p.C / 8) * (p.W / 8) * q.IH;
    uint4r regs[PASSES][8];
    auto fetch = [&](uint32_t tile) {
        const uint32_t n = q.div_row_blocks.div(tile), oh0 = (tile - n * q.row_blocks) * q.R;
        const T* xn = x + static_cast<int64_t>(n) * p.xs[0];
#pragma unroll
        for (int ps = 0; ps < PASSES; ++ps) {
            const uint32_t mb = threadIdx.x + kResThreads * ps;
            uint32_t t1, cb, prow, colb;
            q.div_cblocks.divmod(mb, t1, cb);
            q.div_colblocks.divmod(t1, prow, colb);
            const int32_t ih = q.rows_strided ? static_cast<int32_t>((oh0 + prow) * p.stride_h) - static_cast<int32_t>(p.pad_h)
                                              : static_cast<int32_t>(oh0 * p.stride_h + prow) - static_cast<int32_t>(p.pad_h);
            const bool live = mb < microblocks && ih >= 0 && ih < static_cast<int32_t>(p.H);
            // rows outside the image are written as zeros: read a valid address, zero at commit
            const T* src = live ? xn + static_cast<int64_t>(cb * 8) * p.xs[1] + static_cast<int64_t>(ih) * p.xs[2] + colb * 8 : x;
            const int64_t cstep = live ? p.xs[1] : 0;
#pragma unroll
            for (int cc = 0; cc < 8; ++cc) regs[ps][cc] = *reinterpret_cast<const uint4r*>(src + cc * cstep);
        }
    };
    auto commit = [&](uint32_t tile) {
        const uint32_t oh0 = (tile - q.div_row_blocks.div(tile) * q.row_blocks) * q.R;
#pragma unroll
        for (int ps = 0; ps < PASSES; ++ps) {
            const uint32_t mb = threadIdx.x + kResThreads * ps;
            if (mb >= microblocks) continue;
            uint32_t t1, cb, prow, colb;
            q.div_cblocks.divmod(mb, t1, cb);
            q.div_colblocks.divmod(t1, prow, colb);
            const int32_t ih = q.rows_strided ? static_cast<int32_t>((oh0 + prow) * p.stride_h) - static_cast<int32_t>(p.pad_h)
                                              : static_cast<int32_t>(oh0 * p.stride_h + prow) - static_cast<int32_t>(p.pad_h);
            const bool live = ih >= 0 && ih < static_cast<int32_t>(p.H);
            uint16_t in[8][8];
#pragma unroll
            for (int cc = 0; cc < 8; ++cc) {
                const uint4r v = live ? regs[ps][cc] : uint4r{0, 0, 0, 0};
                __builtin_memcpy(in[cc], &v, 16);
            }
            // channel block cb = chunk (cb / 4), 16-byte slot (cb % 4) of the 32-channel record
            const uint32_t rec0 = (cb / 4) * q.patch_records + prow * q.IWp + p.pad_w + colb * 8;
#pragma unroll
            for (int px = 0; px < 8; ++px) {
                uint16_t out[8];
#pragma unroll
                for (int cc = 0; cc < 8; ++cc) out[cc] = in[cc][px];
                uint4r v;
                __builtin_memcpy(&v, out, 16);
                *reinterpret_cast<uint4r*>(patch + res_offset(rec0 + px, cb % 4)) = v;
            }
        }
    };

    const uint32_t frag_chunk = lane / 32;
    // weight operand: record (wco + lane % 32) of a step's [BCO][32] block; BCO is a multiple of 16, so the
    // swizzle term is the same for every step
    uint32_t wlane[2];
    {
        const uint32_t rec = wco + lane % 32;
        wlane[0] = rec * kRC + ((frag_chunk ^ ((rec >> 2) & 3u)) * 8u);
        wlane[1] = wlane[0] ^ 16u;
    }
    uint32_t tile = worker;
    if (tile < q.tiles) fetch(tile);
    __syncthreads();   // weights and zero fill are in place
    if (tile < q.tiles) commit(tile);
    __syncthreads();

    for (; tile < q.tiles; tile += q.workers) {
        const uint32_t next = tile + q.workers;
        if (next < q.tiles) fetch(next);

        float16r acc[TM][2];
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                acc[i][0][v] = bias_v[i][v];
                acc[i][1][v] = bias_v[i][v];
            }
        // MFMA loop over (tap, 32-channel chunk); each step is two 16-channel MFMA slices.
        // Offsets: weights  wlane[half] + (tap * chunks + chunk) * BCO * 32 + i * 1024
        //          patch    (xoff[j] ^ (half * 16)) + chunk * patch_records * 32
        // The swizzle term of a patch record does not change with the chunk (patch_records is a
        // multiple of 16), so it is computed once per tap.  The operands of the next step are
        // requested before the MFMAs of the current one.
        uint4r fw[2][2][TM], fx[2][2][2];   // [slot][half][...]
        uint32_t kh = 0, kw = 0, chunk = 0;
        uint32_t xoff[2];
        auto tap_offsets = [&]() {
            const uint32_t tap_rec = (q.rows_strided ? 0 : kh) * q.IWp + kw;
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const uint32_t rec = pbase[j] + tap_rec;
                xoff[j] = rec * kRC + ((frag_chunk ^ ((rec >> 2) & 3u)) * 8u);
            }
        };
        auto load_frags = [&](int slot, uint32_t wstep, uint32_t cstep) {
#pragma unroll
            for (int half = 0; half < 2; ++half) {
#pragma unroll
                for (int i = 0; i < TM; ++i) fw[slot][half][i] = *reinterpret_cast<const uint4r*>(wl + wlane[half] + wstep + i * 32 * kRC);
#pragma unroll
                for (int j = 0; j < 2; ++j) fx[slot][half][j] = *reinterpret_cast<const uint4r*>(patch + (xoff[j] ^ (half * 16u)) + cstep);
            }
        };
        auto advance = [&]() {   // next (tap, chunk), chunk fastest
            if (++chunk == chunks) {
                chunk = 0;
                if (++kw == p.KW) { kw = 0; ++kh; }
                tap_offsets();
            }
        };
        auto mfmas = [&](int slot) {
#pragma unroll
            for (int half = 0; half < 2; ++half)
#pragma unroll
                for (int i = 0; i < TM; ++i) {
                    acc[i][0] = resident_mfma<T>(fw[slot][half][i], fx[slot][half][0], acc[i][0]);
                    if (group_live[1]) acc[i][1] = resident_mfma<T>(fw[slot][half][i], fx[slot][half][1], acc[i][1]);
                }
        };
        const uint32_t steps = taps * chunks;
        const uint32_t wstride = BCO * kRC, cstride = q.patch_records * kRC;
        tap_offsets();
        load_frags(0, 0, 0);
        for (uint32_t st = 0; st < steps; st += 2) {
            if (st + 1 < steps) {
                advance();
                load_frags(1, (st + 1) * wstride, chunk * cstride);
            }
            __builtin_amdgcn_sched_barrier(0);
            mfmas(0);
            if (st + 1 >= steps) break;
            if (st + 2 < steps) {
                advance();
                load_frags(0, (st + 2) * wstride, chunk * cstride);
            }
            __builtin_amdgcn_sched_barrier(0);
            mfmas(1);
        }

        // store this tile: the lane's pixel column, rows = output channels
        const uint32_t n = q.div_row_blocks.div(tile), oh0 = (tile - n * q.row_blocks) * q.R;
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const uint32_t oh = oh0 + prow_of[j];
            if (!pixel_live[j] || oh >= p.HO) continue;
            T* yp = y + static_cast<int64_t>(n) * p.ys[0] + static_cast<int64_t>(oh) * p.ys[2] + static_cast<int64_t>(pcol_of[j]) * p.ys[3];
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const uint32_t co = co0 + wco + i * 32 + 8 * (v / 4) + 4 * (lane / 32) + v % 4;
                    if (co < p.O) yp[static_cast<int64_t>(co) * p.ys[1]] = narrow<T>(acc[i][j][v]);
                }
        }

        __syncthreads();              // every wavefront is done reading the patch
        if (next < q.tiles) commit(next);
        __syncthreads();
    }
}

template <class T, int BCO, int WSPLIT, int PASSES>
int launch_resident(const ConvProblem& p, const ResidentPlan& q, size_t lds, const void* x, const T* wt, const void* bias, void* y, hipStream_t stream) {
    auto kernel = conv2d_resident_kernel<T, BCO, WSPLIT, PASSES>;
    static std::atomic<uint64_t> configured{0};
    if (int rc = raise_lds_limit(reinterpret_cast<const void*>(kernel), 160 * 1024, configured)) return rc;
    hipLaunchKernelGGL(kernel, dim3(q.workers * q.co_tiles), dim3(kResThreads), lds, stream, static_cast<const T*>(x), wt, static_cast<const T*>(bias),
                       static_cast<T*>(y), p, q);
    return launch_status("conv2d_resident_kernel");
}

template <class T> __global__ void conv_weights_tap_major_kernel2(const T* w, T* out, ConvProblem p, uint32_t total) {
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const uint32_t c = i % p.C, o = (i / p.C) % p.O, tap = i / (p.C * p.O);
    out[i] = w[o * p.ws[0] + c * p.ws[1] + (tap / p.KW) * p.ws[2] + (tap % p.KW) * p.ws[3]];
}

template <class T>
int run_resident(const ConvProblem& p, const void* x, const void* w, const void* bias, void* y, hipStream_t stream) {
    if (p.C == 0 || p.C % kRC != 0 || p.W % 8 != 0 || p.xs[3] != 1 || p.xs[2] % 8 != 0 || p.xs[1] % 8 != 0 || p.xs[0] % 8 != 0) return TANNIC_UNSUPPORTED_DTYPE;
    if (reinterpret_cast<uintptr_t>(x) % 16 != 0) return TANNIC_UNSUPPORTED_DTYPE;
    if (p.N == 0 || p.O == 0 || p.HO == 0 || p.WO == 0) return TANNIC_SUCCESS;
    const uint32_t taps = p.KH * p.KW;
    const int BCO = p.O > 64 ? 128 : 64;
    const size_t w_bytes = static_cast<size_t>(taps) * p.C * BCO * sizeof(T);
    const size_t budget = 156 * 1024;
    const size_t table_bytes = 0;
    if (w_bytes + table_bytes >= budget) return TANNIC_UNSUPPORTED_DTYPE;
    ResidentPlan q{};
    q.rows_strided = p.KH == 1 ? 1 : 0;
    q.IWp = p.W + 2 * p.pad_w;
    q.co_tiles = (p.O + BCO - 1) / BCO;
    double best = 0.0;
    size_t best_lds = 0;
    for (uint32_t R = 1; R <= p.HO && R * p.WO <= 256; ++R) {
        const uint32_t IH = q.rows_strided ? R : (R - 1) * p.stride_h + p.KH;
        const size_t patch_bytes = static_cast<size_t>((IH * q.IWp + 15u) & ~15u) * p.C * sizeof(T);
        const size_t lds = w_bytes + patch_bytes + table_bytes;
        const uint64_t microblocks = static_cast<uint64_t>(p.C / 8) * (p.W / 8) * IH;
        if (lds > budget || microblocks > 2 * kResThreads) break;
        const uint32_t groups = (R * p.WO + 31) / 32;
        const uint32_t rounds = groups <= 2 ? 1 : (groups + 3) / 4;   // two-group tiles split channels over wavefronts instead
        const double fill = static_cast<double>(R * p.WO) / (rounds * (groups <= 2 ? 64.0 : 128.0));
        const double rows = static_cast<double>(p.HO) / (((p.HO + R - 1) / R) * R);
        const double score = fill * rows;
        if (score >= best) { best = score; q.R = R; q.IH = IH; q.groups = groups; best_lds = lds; }
    }
    if (best == 0.0) return TANNIC_UNSUPPORTED_DTYPE;
    q.row_blocks = (p.HO + q.R - 1) / q.R;
    q.patch_records = (q.IH * q.IWp + 15u) & ~15u;   // multiple of 16: the swizzle of a record is the same in every chunk
    const uint64_t tiles = static_cast<uint64_t>(p.N) * q.row_blocks;
    if (tiles >= (1ull << 31)) return TANNIC_UNSUPPORTED_DTYPE;
    q.tiles = static_cast<uint32_t>(tiles);
    q.div_cblocks = FastDiv(p.C / 8);
    q.div_colblocks = FastDiv(p.W / 8);
    q.div_chunks = FastDiv(p.C / kRC);
    q.div_row_blocks = FastDiv(q.row_blocks);
    static std::atomic<int> known_cus{0};   // compute units of the device, asked once
    int cus = known_cus.load(std::memory_order_relaxed);
    if (cus == 0) {
        cus = 256;
        hipDeviceProp_t prop;
        int dev = 0;
        if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess && prop.multiProcessorCount > 0) cus = prop.multiProcessorCount;
        known_cus.store(cus, std::memory_order_relaxed);
    }
    uint32_t workers = static_cast<uint32_t>(cus) / q.co_tiles;
    if (workers == 0) workers = 1;
    if (workers > q.tiles) workers = q.tiles;
    // even out the rounds: every worker gets ceil(tiles / workers) tiles at most
    const uint32_t rounds = (q.tiles + workers - 1) / workers;
    q.workers = (q.tiles + rounds - 1) / rounds;
    const uint64_t wcount = static_cast<uint64_t>(taps) * p.O * p.C;
    if (wcount >= (1ull << 31)) return TANNIC_UNSUPPORTED_DTYPE;
    const uint64_t microblocks = static_cast<uint64_t>(p.C / 8) * (p.W / 8) * q.IH;
    T* wt = nullptr;
    if (scratch_acquire(reinterpret_cast<void**>(&wt), wcount * sizeof(T), stream) != TANNIC_SUCCESS) return TANNIC_ERROR;
    hipLaunchKernelGGL((conv_weights_tap_major_kernel2<T>), dim3((wcount + 255) / 256), dim3(256), 0, stream, static_cast<const T*>(w), wt, p,
                       static_cast<uint32_t>(wcount));
    int status = launch_status("conv_weights_tap_major_kernel");
    if (status == TANNIC_SUCCESS) {
        const bool split = q.groups <= 2;      // few pixel groups: two wavefronts share each group and split the channels
        const bool two = microblocks > kResThreads;
        if (BCO == 128) {
            if (split) status = two ? launch_resident<T, 128, 2, 2>(p, q, best_lds, x, wt, bias, y, stream) : launch_resident<T, 128, 2, 1>(p, q, best_lds, x, wt, bias, y, stream);
            else status = two ? launch_resident<T, 128, 1, 2>(p, q, best_lds, x, wt, bias, y, stream) : launch_resident<T, 128, 1, 1>(p, q, best_lds, x, wt, bias, y, stream);
        } else {
            if (split) status = two ? launch_resident<T, 64, 2, 2>(p, q, best_lds, x, wt, bias, y, stream) : launch_resident<T, 64, 2, 1>(p, q, best_lds, x, wt, bias, y, stream);
            else status = two ? launch_resident<T, 64, 1, 2>(p, q, best_lds, x, wt, bias, y, stream) : launch_resident<T, 64, 1, 1>(p, q, best_lds, x, wt, bias, y, stream);
        }
    }
    scratch_release(wt, stream);
    return status;
}

int conv2d_resident(const ConvProblem& p, int dtype, const void* x, const void* w, const void* bias, void* y, hipStream_t stream) {
    if (dtype == TANNIC_FLOAT16) return run_resident<f16>(p, x, w, bias, y, stream);
    if (dtype == TANNIC_BFLOAT16) return run_resident<bf16>(p, x, w, bias, y, stream);
    return TANNIC_UNSUPPORTED_DTYPE;
}

}  // namespace th
