// conv2d for signals with few channels (the first layer of an image network:
// 3 channels, 7x7 kernel, stride 2) on MFMA, 16-bit types.
//
// With so few channels the contraction index is ordered (channel, kernel row,
// kernel column) and every (channel, kernel row) pair is padded to one slot of 8
// columns (KW <= 8, the rest zero weights).  A slot of a pixel is then 8
// CONSECUTIVE signal elements of one input row, so no im2col copy is needed: the
// MFMA operand of a pixel is read straight out of the input rows, which a block
// keeps in LDS as they are in memory (NCHW rows) with zero columns on both sides.
// The slot starts at an even column (the horizontal stride must be even; a kernel
// whose first column falls on an odd one is moved right by one zero weight), so
// every operand is four aligned LDS words.
// A block of 256 threads owns a strip of consecutive output rows of one image
// and 64 output channels.  Per channel it holds a ring of input rows (a power of
// two >= KH); moving down one output row replaces stride_h of them, loaded 16
// bytes at a time while the MFMAs of the current row run.  A tile is one output
// row (WO <= 128): each wavefront multiplies 32 pixels with the weights of the 64
// channels, whose fragments it keeps in registers for the whole strip.  Results
// are rounded into LDS as [channel][pixel] and written as whole rows.  Two
// blocks share a compute unit, so one block's loads and stores overlap the other's MFMAs.
#include "conv_common.hpp"

namespace th {

typedef _Float16 half8s __attribute__((ext_vector_type(8)));
typedef __bf16 bfloat8s __attribute__((ext_vector_type(8)));
typedef float float16s __attribute__((ext_vector_type(16)));
typedef unsigned int uint4s __attribute__((ext_vector_type(4)));

template <class T> __device__ inline float16s stem_mfma(uint4s a, uint4s b, float16s c) {
    if constexpr (std::is_same_v<T, f16>) {
        half8s x, y;
        __builtin_memcpy(&x, &a, 16);
        __builtin_memcpy(&y, &b, 16);
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(x, y, c, 0, 0, 0);
    } else {
        bfloat8s x, y;
        __builtin_memcpy(&x, &a, 16);
        __builtin_memcpy(&y, &b, 16);
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(x, y, c, 0, 0, 0);
    }
}

constexpr int kStemThreads = 256;
constexpr int kStemPixels = 128;   // lanes along a tile: output columns of one row
constexpr int kStemBCO = 64;       // output channels per block
constexpr int kStemOutPitch = kStemPixels + 8;
constexpr int kStemLeft = 8;       // zero columns in front of a row in LDS (keeps the 16-byte row chunks aligned)
constexpr int kStemUnits = 4;      // 16-byte chunks of input rows a thread can hold at a time
constexpr int kStemWeightPieces = 6;   // 16-byte pieces of a block's weights per thread: 64 channels x (22 slots x 8 columns) at most

struct StemPlan {
    uint32_t slots;             // C * KH
    uint32_t ring;              // rows kept per channel, a power of two >= KH
    uint32_t pitch;             // elements per LDS row
    uint32_t delta;             // zero weights in front of a kernel row: makes the slot's first column even
    uint32_t strip;             // output rows per block
    uint32_t strips_per_image, co_tiles;
    uint32_t ring_elems;        // C * ring * pitch
    uint32_t vector_store;
    FastDiv div_kh, div_strips, div_co_tiles, div_chunks, div_c;
};

// NS: 16-wide slices of the contraction = slots / 2 rounded up
template <class T, int NS>
__global__ __launch_bounds__(kStemThreads, 2) void conv2d_stem_kernel(const T* x, const T* w, const T* bias, T* y, ConvProblem p, StemPlan q) {
    extern __shared__ __align__(16) unsigned char stem_lds[];
    T* ring = reinterpret_cast<T*>(stem_lds);
    T* out = ring + q.ring_elems;
    const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;

    uint32_t rest, ct, n, strip;
    q.div_co_tiles.divmod(blockIdx.x, rest, ct);
    q.div_strips.divmod(rest, n, strip);
    const uint32_t co0 = ct * kStemBCO;
    const uint32_t oh_first = strip * q.strip;
    const uint32_t oh_end = oh_first + q.strip < p.HO ? oh_first + q.strip : p.HO;
    const T* ximg = x + static_cast<int64_t>(n) * p.xs[0];

    // ---- input rows: global -> registers -> ring --------------------------------------------------------------
    // a unit is one 16-byte chunk of one row of one channel; rows outside the image are stored as zeros
    const uint32_t chunks = p.W / 8;
    uint4s rows_reg[kStemUnits];
    auto load_rows = [&](int32_t ih_from, uint32_t count) {   // rows ih_from .. ih_from + count - 1 of every channel
        const uint32_t units = p.C * count * chunks;
#pragma unroll
        for (int u = 0; u < kStemUnits; ++u) {
            if (kStemThreads * u >= units) continue;   // the same for the whole block
            const uint32_t idx = threadIdx.x + kStemThreads * u;
            uint32_t t1, chunk, r, c;
            q.div_chunks.divmod(idx, t1, chunk);
            q.div_c.divmod(t1, r, c);
            const int32_t ih = ih_from + static_cast<int32_t>(r);
            const bool live = idx < units && ih >= 0 && ih < static_cast<int32_t>(p.H);
            rows_reg[u] = uint4s{0, 0, 0, 0};
            if (live) rows_reg[u] = *reinterpret_cast<const uint4s*>(ximg + static_cast<int64_t>(c) * p.xs[1] + static_cast<int64_t>(ih) * p.xs[2] + chunk * 8);
        }
    };
    auto store_rows = [&](int32_t ih_from, uint32_t count) {
        const uint32_t units = p.C * count * chunks;
#pragma unroll
        for (int u = 0; u < kStemUnits; ++u) {
            const uint32_t idx = threadIdx.x + kStemThreads * u;
            if (idx >= units) continue;
            uint32_t t1, chunk, r, c;
            q.div_chunks.divmod(idx, t1, chunk);
            q.div_c.divmod(t1, r, c);
            const uint32_t slot = static_cast<uint32_t>(ih_from + static_cast<int32_t>(r) + (1 << 20) * static_cast<int32_t>(q.ring)) & (q.ring - 1);
            *reinterpret_cast<uint4s*>(ring + (c * q.ring + slot) * q.pitch + kStemLeft + chunk * 8) = rows_reg[u];
        }
    };
    // Every global load of the start is issued before the first wait: the block's weights (at most six 16-byte pieces
    // per thread), the input rows of the first output row (as many as the registers hold) and the bias.
    const int32_t top = static_cast<int32_t>(oh_first * p.stride_h) - static_cast<int32_t>(p.pad_h);
    const uint32_t per_step = (kStemUnits * kStemThreads) / (p.C * chunks);   // >= 1 by the plan
    const uint32_t first_count = p.KH < per_step ? p.KH : per_step;

    // ---- weights: this lane's fragments for every slice, kept in registers --------------------------------
    // The block's rows of the OIHW tensor (one contiguous run) are copied to LDS 16 bytes at a time first.
    // fragment (s, i): channel co0 + i * 32 + lane % 32, slot 2 s + lane / 32; element e of a slot is kernel column e - delta
    const uint32_t taps = q.slots * p.KW;   // elements per output channel
    const uint32_t wrows = p.O - co0 < kStemBCO ? p.O - co0 : kStemBCO;
    float bias_v[2];
    {
        T* raw = ring;
        const uint32_t count = wrows * taps;   // the run starts at a multiple of 8 elements (64 * taps is one)
        const T* src = w + static_cast<int64_t>(co0) * taps;
        uint4s wreg[kStemWeightPieces];
#pragma unroll
        for (int j = 0; j < kStemWeightPieces; ++j) {
            const uint32_t i = (threadIdx.x + kStemThreads * j) * 8;
            if (i + 8 <= count) wreg[j] = *reinterpret_cast<const uint4s*>(src + i);
        }
        load_rows(top, first_count);
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const uint32_t co = co0 + i * 32 + lane % 32;
            bias_v[i] = (p.has_bias && co < p.O) ? static_cast<float>(widen(bias[static_cast<int64_t>(co) * p.bs])) : 0.0f;
        }
#pragma unroll
        for (int j = 0; j < kStemWeightPieces; ++j) {
            const uint32_t i = (threadIdx.x + kStemThreads * j) * 8;
            if (i + 8 <= count) *reinterpret_cast<uint4s*>(raw + i) = wreg[j];
            else if (i < count)
                for (uint32_t e = i; e < count; ++e) raw[e] = src[e];
        }
        __syncthreads();
    }
    // Every (slot, channel) pair becomes one 16-byte record [slot][64 channels]: five aligned words around the slot's
    // KW weights, moved by half a word when they start at an odd element, cleared outside the kernel row.
    T* records = ring + ((kStemBCO * taps + 7) / 8) * 8;
    {
        const uint32_t* raw32 = reinterpret_cast<const uint32_t*>(ring);
        const int32_t last_word = static_cast<int32_t>((wrows * taps + 1) / 2) - 1;
        uint32_t keep[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint32_t lo = (2u * j >= q.delta && 2u * j - q.delta < p.KW) ? 0xFFFFu : 0u;
            const uint32_t hi = (2u * j + 1 >= q.delta && 2u * j + 1 - q.delta < p.KW) ? 0xFFFF0000u : 0u;
            keep[j] = lo | hi;
        }
        for (uint32_t u = threadIdx.x; u < 2 * NS * kStemBCO; u += kStemThreads) {
            const uint32_t cl = u % kStemBCO, slot = u / kStemBCO;
            const bool real = cl < wrows && slot < q.slots;
            const int32_t first = static_cast<int32_t>(cl * taps + slot * p.KW) - static_cast<int32_t>(q.delta);   // >= -1
            const int32_t w0 = (first + 2) / 2 - 1;   // floor(first / 2)
            const bool odd = (first & 1) != 0;
            uint32_t word[5];
#pragma unroll
            for (int j = 0; j < 5; ++j) {
                int32_t at = w0 + j;
                at = at < 0 ? 0 : (at > last_word ? last_word : at);
                word[j] = raw32[real ? at : 0];
            }
            uint4s rec;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint32_t v = odd ? (word[j] >> 16) | (word[j + 1] << 16) : word[j];
                rec[j] = real ? v & keep[j] : 0u;
            }
            *reinterpret_cast<uint4s*>(records + u * 8) = rec;
        }
    }
    __syncthreads();
    uint4s afrag[NS][2];
#pragma unroll
    for (int s = 0; s < NS; ++s)
#pragma unroll
        for (int i = 0; i < 2; ++i) afrag[s][i] = *reinterpret_cast<const uint4s*>(records + ((2 * s + lane / 32) * kStemBCO + i * 32 + lane % 32) * 8);
    __syncthreads();   // the copy is consumed: its memory becomes the ring
    // zero everything once: the columns beside the rows are never written again
    for (uint32_t i = threadIdx.x; i < q.ring_elems / 8; i += kStemThreads) reinterpret_cast<uint4s*>(ring)[i] = uint4s{0, 0, 0, 0};
    __syncthreads();

    // the rows of the first tile, in as many steps as the registers need
    store_rows(top, first_count);   // loaded at the very start
    for (uint32_t done = first_count; done < p.KH; done += per_step) {
        const uint32_t count = p.KH - done < per_step ? p.KH - done : per_step;
        load_rows(top + static_cast<int32_t>(done), count);
        store_rows(top + static_cast<int32_t>(done), count);
    }

    // ---- per-lane constants of the operand reads ------------------------------------------------------------------
    // pixel ow = wave * 32 + lane % 32; slot 2 s + lane / 32 -> (channel, kernel row)
    const uint32_t ow = wave * 32 + lane % 32;
    const uint32_t col = kStemLeft + (ow < p.WO ? ow : 0) * p.stride_w - p.pad_w - q.delta;   // even: the plan sees to it
    uint32_t frag_base[NS];   // channel offset + column
    uint32_t frag_kh[NS];
#pragma unroll
    for (int s = 0; s < NS; ++s) {
        const uint32_t slot = 2 * s + lane / 32;
        uint32_t c = 0, kh = 0;
        if (slot < q.slots) q.div_kh.divmod(slot, c, kh);
        frag_base[s] = c * q.ring * q.pitch + col;
        frag_kh[s] = kh;
    }
    // elements of a slot that face a zero weight are cleared, so that no Inf or NaN of the signal can leak through them
    uint4s keep;
    {
        uint16_t k16[8];
#pragma unroll
        for (int k = 0; k < 8; ++k) k16[k] = (static_cast<uint32_t>(k) >= q.delta && static_cast<uint32_t>(k) - q.delta < p.KW) ? 0xFFFFu : 0u;
        __builtin_memcpy(&keep, k16, 16);
    }
    __syncthreads();

    for (uint32_t oh = oh_first; oh < oh_end; ++oh) {
        // rows that the next output row adds
        const int32_t new_from = static_cast<int32_t>(oh * p.stride_h) - static_cast<int32_t>(p.pad_h) + static_cast<int32_t>(p.KH);
        const bool more = oh + 1 < oh_end;
        if (more) load_rows(new_from, p.stride_h);

        float16s acc[2];
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][v] = bias_v[i];
        const uint32_t ih_top = oh * p.stride_h - p.pad_h + (1u << 20) * q.ring;   // kept positive for the ring index
        uint4s bfrag[NS];
#pragma unroll
        for (int s = 0; s < NS; ++s) {
            const uint32_t row = (ih_top + frag_kh[s]) & (q.ring - 1);
            const uint32_t* src = reinterpret_cast<const uint32_t*>(ring + frag_base[s] + row * q.pitch);
            bfrag[s] = uint4s{src[0], src[1], src[2], src[3]} & keep;
        }
#pragma unroll
        for (int s = 0; s < NS; ++s)
#pragma unroll
            for (int i = 0; i < 2; ++i) acc[i] = stem_mfma<T>(bfrag[s], afrag[s][i], acc[i]);
        // accumulator i: lane -> channel i * 32 + lane % 32; value v -> pixel 8 * (v / 4) + 4 * (lane / 32) + v % 4 of the wavefront's 32
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                T r[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) r[e] = narrow_result<T>(acc[i][g * 4 + e]);
                uint2 bits;
                __builtin_memcpy(&bits, r, 8);
                *reinterpret_cast<uint2*>(out + (i * 32 + lane % 32) * kStemOutPitch + wave * 32 + g * 8 + 4 * (lane / 32)) = bits;
            }
        __syncthreads();   // the rows are consumed, the result is complete

        T* yrow = y + static_cast<int64_t>(n) * p.ys[0] + static_cast<int64_t>(oh) * p.ys[2];
        if (q.vector_store) {
            // 16 lanes per channel row, four rows per wavefront instruction
#pragma unroll
            for (int r = 0; r < kStemBCO / 16; ++r) {
                const uint32_t c = wave * 16 + r * 4 + lane / 16, px = (lane % 16) * 8;
                if (co0 + c < p.O && px < p.WO)
                    *reinterpret_cast<uint4s*>(yrow + static_cast<int64_t>(co0 + c) * p.ys[1] + px) = *reinterpret_cast<const uint4s*>(out + c * kStemOutPitch + px);
            }
        } else {
            for (uint32_t c = wave; c < kStemBCO; c += 4) {
                if (co0 + c >= p.O) break;
                for (uint32_t px = lane; px < p.WO; px += 64) yrow[static_cast<int64_t>(co0 + c) * p.ys[1] + static_cast<int64_t>(px) * p.ys[3]] = out[c * kStemOutPitch + px];
            }
        }
        if (more) store_rows(new_from, p.stride_h);
        __syncthreads();
    }
}

template <class T, int NS>
int launch_stem(const ConvProblem& p, const StemPlan& q, uint32_t blocks, size_t lds, const void* x, const void* w, const void* bias, void* y, hipStream_t stream) {
    auto kernel = conv2d_stem_kernel<T, NS>;
    static std::atomic<uint64_t> configured{0};
    if (int rc = raise_lds_limit(reinterpret_cast<const void*>(kernel), 64 * 1024, configured)) return rc;
    hipLaunchKernelGGL(kernel, dim3(blocks), dim3(kStemThreads), lds, stream, static_cast<const T*>(x), static_cast<const T*>(w), static_cast<const T*>(bias),
                       static_cast<T*>(y), p, q);
    return launch_status("conv2d_stem_kernel");
}

template <class T>
int run_stem(const ConvProblem& p, const void* x, const void* w, const void* bias, void* y, hipStream_t stream) {
    const uint32_t slots = p.C * p.KH;
    if (p.C == 0 || p.C > 4 || slots > 22 || p.WO > kStemPixels) return TANNIC_UNSUPPORTED_DTYPE;
    // even horizontal stride: every slot starts at an even column, an aligned LDS word
    if (p.stride_w % 2 != 0 || p.pad_w > kStemLeft - 1) return TANNIC_UNSUPPORTED_DTYPE;
    const uint32_t delta = p.pad_w % 2;
    if (p.KW + delta > 8 || p.stride_h > p.KH) return TANNIC_UNSUPPORTED_DTYPE;
    // 16-byte loads of the input rows
    if (p.W % 8 != 0 || p.xs[3] != 1 || p.xs[2] % 8 != 0 || p.xs[1] % 8 != 0 || p.xs[0] % 8 != 0 || reinterpret_cast<uintptr_t>(x) % 16 != 0) return TANNIC_UNSUPPORTED_DTYPE;
    // the kernel tensor is plain OIHW: its rows are copied as one run
    if (p.ws[3] != 1 || p.ws[2] != static_cast<int64_t>(p.KW) || p.ws[1] != static_cast<int64_t>(p.KH) * p.KW ||
        p.ws[0] != static_cast<int64_t>(p.C) * p.KH * p.KW || reinterpret_cast<uintptr_t>(w) % 16 != 0)
        return TANNIC_UNSUPPORTED_DTYPE;
    if (p.N == 0 || p.O == 0 || p.HO == 0 || p.WO == 0) return TANNIC_SUCCESS;
    StemPlan q{};
    q.slots = slots;
    q.delta = delta;
    q.ring = 1;
    while (q.ring < p.KH) q.ring *= 2;
    // the farthest column an operand touches, and room for a whole number of 16-byte chunks
    const uint32_t reach = kStemLeft + (p.WO - 1) * p.stride_w - p.pad_w - delta + 8;
    const uint32_t need = reach > kStemLeft + p.W ? reach : kStemLeft + p.W;
    q.pitch = (need + 7) / 8 * 8;
    q.ring_elems = p.C * q.ring * q.pitch;
    const uint32_t chunks = p.W / 8;
    // the rows one step adds must fit the staging registers of the block
    if (static_cast<uint64_t>(p.C) * p.stride_h * chunks > kStemUnits * kStemThreads) return TANNIC_UNSUPPORTED_DTYPE;
    // the weights' stay in LDS: the copied rows, then 16-byte records for 2 * NS slots (NS as chosen below)
    const uint32_t ns = (slots + 1) / 2, ns_built = ns <= 3 ? 3 : (ns <= 5 ? 5 : (ns <= 8 ? 8 : 11));
    const size_t raw_bytes = (static_cast<size_t>(kStemBCO) * slots * p.KW + 8 + static_cast<size_t>(2 * ns_built) * kStemBCO * 8) * sizeof(T);
    size_t lds = (static_cast<size_t>(q.ring_elems) + kStemBCO * kStemOutPitch) * sizeof(T);
    if (lds < raw_bytes) lds = raw_bytes;
    if (lds > 64 * 1024) return TANNIC_UNSUPPORTED_DTYPE;
    q.co_tiles = (p.O + kStemBCO - 1) / kStemBCO;
    static std::atomic<int> known_cus{0};   // compute units of the device, asked once
    int cus = known_cus.load(std::memory_order_relaxed);
    if (cus == 0) {
        cus = 256;
        hipDeviceProp_t prop;
        int dev = 0;
        if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess && prop.multiProcessorCount > 0) cus = prop.multiProcessorCount;
        known_cus.store(cus, std::memory_order_relaxed);
    }
    // strips: about two blocks per compute unit, at least KH rows each so that the first tile's rows pay off
    const uint64_t want = static_cast<uint64_t>(2 * cus);
    uint64_t per_image = want / (static_cast<uint64_t>(p.N) * q.co_tiles);
    if (per_image == 0) per_image = 1;
    uint32_t strip = static_cast<uint32_t>((p.HO + per_image - 1) / per_image);
    if (strip < p.KH) strip = p.KH < p.HO ? p.KH : p.HO;
    q.strip = strip;
    q.strips_per_image = (p.HO + strip - 1) / strip;
    const uint64_t blocks = static_cast<uint64_t>(p.N) * q.strips_per_image * q.co_tiles;
    if (blocks >= (1ull << 31)) return TANNIC_UNSUPPORTED_DTYPE;
    q.div_kh = FastDiv(p.KH);
    q.div_strips = FastDiv(q.strips_per_image);
    q.div_co_tiles = FastDiv(q.co_tiles);
    q.div_chunks = FastDiv(chunks);
    q.div_c = FastDiv(p.C);
    q.vector_store = p.ys[3] == 1 && p.ys[2] % 8 == 0 && p.ys[1] % 8 == 0 && p.ys[0] % 8 == 0 && p.WO % 8 == 0 && reinterpret_cast<uintptr_t>(y) % 16 == 0;
    const uint32_t b = static_cast<uint32_t>(blocks);
    if (ns <= 3) return launch_stem<T, 3>(p, q, b, lds, x, w, bias, y, stream);
    if (ns <= 5) return launch_stem<T, 5>(p, q, b, lds, x, w, bias, y, stream);
    if (ns <= 8) return launch_stem<T, 8>(p, q, b, lds, x, w, bias, y, stream);
    return launch_stem<T, 11>(p, q, b, lds, x, w, bias, y, stream);
}

int conv2d_stem(const ConvProblem& p, int dtype, const void* x, const void* w, const void* bias, void* y, hipStream_t stream) {
    if (dtype == TANNIC_FLOAT16) return run_stem<f16>(p, x, w, bias, y, stream);
    if (dtype == TANNIC_BFLOAT16) return run_stem<bf16>(p, x, w, bias, y, stream);
    return TANNIC_UNSUPPORTED_DTYPE;
}

}  // namespace th
