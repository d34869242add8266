// Q4_K weights x a handful of Q8_1 activation rows on the int8 matrix unit: the mid-batch path
// between the mat-vec kernels (whose dot work grows with every activation row) and the tiled
// matmul (which stages weights through LDS and needs hundreds of rows to pay for it).
//
// Replaces loken_dense_q4k_imma_m8_plain of the reference (declared src/inference/moe_cuda/
// mod.rs:456-458, called from dense_q4k_imma_m8_matmul, src/inference/moe_cuda/dense/imma.rs:
// 82-135; kernels cuda/q4k_mmvq_imma.cu, cuda/imma_amd.cu:472-545): plain block_q8_1 rows in,
// `out += dsc * d8 * C - dmm * d8 * S` per sub-block. Here S is the integer sum of the codes,
// as everywhere else in this library, not the rounded `s` field of the Q8_1 block.
//
// Shape of the work. A wave owns 32 weight rows and up to 32 activation rows: one
// v_mfma_i32_32x32x32_i8 is one Q4_K sub-block (32 values) of those rows against those
// activations. Weights never touch LDS: lane l holds row l % 32 and reads, per super-block, its
// 16-byte header and the four 16-byte runs of `qs` at 32 * p + 16 * (l / 32), which are exactly
// its half of the B operand for sub-blocks 2p (low nibbles) and 2p + 1 (high nibbles). The
// activation codes come the same way (lane l: row l % 32, 16 codes at 16 * (l / 32), straight
// from the Q8_1 block), so the only LDS traffic is the table of activation scales, staged once
// per workgroup, from which a lane fetches the 16 scales its accumulator registers stand for.
// The four waves of a workgroup split the super-blocks of the same 32 rows between them and
// add their partial tiles through LDS, which keeps small matrices spread over the chip.
//
// The min term -dmin * m[s] * d8 * S[s] is rank one per sub-block and goes through
// v_mfma_f32_32x32x2_f32 with K = the two halves of the sub-block: A = d8 * (sum of the lane's
// own 16 codes), B = -dmin * m[s] in both halves. No lane exchange is needed for the sum.

#include "lk_common.h"

#include <mutex>
#include <unordered_map>

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));

constexpr int WG = 256, WAVES = 4;
constexpr int TOK = 32;   // activation rows per pass (the matrix instruction's M)

struct Args {
    const uint8_t* w;
    const uint8_t* y;     // Q8_1 rows
    float* dst;
    int nb;               // super-blocks per weight row
    int n;                // weight rows
    int m;                // activation rows in all
    int stride_y;         // Q8_1 blocks between activation rows
    int ldd;              // floats between output rows
};

struct Frag {
    uint4 hdr, q[4];
    v4i a[8];
};

static __device__ __forceinline__ int lds_floats_table(int nb) { return nb * 8 * TOK; }

__global__ __launch_bounds__(WG, 2) void q4k_rows_mfma_kernel(Args p) {
    extern __shared__ __align__(16) uint8_t lds[];
    float* d8_table = (float*)lds;                                   // [nb * 8][TOK]
    float* reduce = d8_table + lds_floats_table(p.nb);               // [WAVES][16][64]

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int l32 = lane & 31, lh = lane >> 5;
    const int m0 = blockIdx.y * TOK;
    const int m_count = min(TOK, p.m - m0);
    const int n_tiles = (p.n + 31) >> 5;
    const size_t row_bytes = (size_t)p.nb * Q4K_BYTES;

    // Activation scales of this pass, zero for the rows the pass does not have. Eight loads are
    // issued before the first is used: one at a time, each would cost a memory latency.
    const uint8_t* y0 = p.y + (size_t)m0 * p.stride_y * Q81_BYTES;
    const int entries = p.nb * 8 * TOK;
    for (int base = threadIdx.x; base < entries; base += WG * 8) {
        uint32_t bits[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int idx = min(base + u * WG, entries - 1);
            const int sub = idx >> 5, tok = min(idx & 31, m_count - 1);
            bits[u] = *(const uint16_t*)(y0 + ((size_t)tok * p.stride_y + sub) * Q81_BYTES);
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int idx = base + u * WG;
            if (idx < entries) d8_table[idx] = (idx & 31) < m_count ? f16_bits_to_f32(bits[u]) : 0.f;
        }
    }

    // The lane's activation row (a row past the end re-reads the last one; its scales are zero).
    const uint8_t* y_lane = y0 + (size_t)min(l32, m_count - 1) * p.stride_y * Q81_BYTES + 4 + 16 * lh;

    auto load = [&](Frag& f, int tile, int kb) {
        const int row = min(tile * 32 + l32, p.n - 1);
        const uint8_t* bp = (const uint8_t*)(to_gbytes(p.w) + row * row_bytes + (size_t)kb * Q4K_BYTES);
        f.hdr = *(const uint4*)bp;
#pragma unroll
        for (int c = 0; c < 4; ++c) f.q[c] = *(const uint4*)(bp + 16 + 32 * c + 16 * lh);
        const uint8_t* ap = y_lane + (size_t)kb * 8 * Q81_BYTES;
#pragma unroll
        for (int s = 0; s < 8; ++s) {
            const uint4 t = *(const uint4_a4*)(ap + s * Q81_BYTES);
            f.a[s] = v4i{(int)t.x, (int)t.y, (int)t.z, (int)t.w};
        }
    };

    // Two accumulators: the scale term is vector arithmetic on `acc`, the min term a chain of
    // matrix instructions on `acc_min`; kept apart, neither waits for the other's latency.
    v16f acc, acc_min;
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[v] = acc_min[v] = 0.f;

    auto compute = [&](const Frag& f, int kb) {
        // the row's eight (scale, min) pairs, six bits each (get_scale_min_k4 of the format)
        const uint32_t w1 = f.hdr.y, w2 = f.hdr.z, w3 = f.hdr.w;
        const uint32_t sc_lo = w1 & 0x3F3F3F3Fu, mn_lo = w2 & 0x3F3F3F3Fu;
        const uint32_t sc_hi = (w3 & 0x0F0F0F0Fu) | ((w1 >> 2) & 0x30303030u);
        const uint32_t mn_hi = ((w3 >> 4) & 0x0F0F0F0Fu) | ((w2 >> 2) & 0x30303030u);
        const float d = f16_bits_to_f32(f.hdr.x & 0xFFFFu), dmin = f16_bits_to_f32(f.hdr.x >> 16);
        float dsc[8], dmm[8];
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            dsc[s] = d * (float)((sc_lo >> (8 * s)) & 0xFFu);
            dsc[s + 4] = d * (float)((sc_hi >> (8 * s)) & 0xFFu);
            dmm[s] = -(dmin * (float)((mn_lo >> (8 * s)) & 0xFFu));
            dmm[s + 4] = -(dmin * (float)((mn_hi >> (8 * s)) & 0xFFu));
        }
        const uint4 ones = make_uint4(0x01010101u, 0x01010101u, 0x01010101u, 0x01010101u);
#pragma unroll
        for (int s = 0; s < 8; ++s) {
            const uint4 q = f.q[s >> 1];
            v4i b;
            if (s & 1) {
                b = v4i{(int)((q.x >> 4) & 0x0F0F0F0Fu), (int)((q.y >> 4) & 0x0F0F0F0Fu),
                        (int)((q.z >> 4) & 0x0F0F0F0Fu), (int)((q.w >> 4) & 0x0F0F0F0Fu)};
            } else {
                b = v4i{(int)(q.x & 0x0F0F0F0Fu), (int)(q.y & 0x0F0F0F0Fu), (int)(q.z & 0x0F0F0F0Fu),
                        (int)(q.w & 0x0F0F0F0Fu)};
            }
            // The int32 accumulators start at the bit pattern of 1.5 * 2^23: adding an integer of
            // magnitude below 2^22 to that pattern yields the float 1.5 * 2^23 + integer, so the
            // dots leave the matrix unit as floats and no conversion is spent on them. The offset
            // goes in the first fused multiply-add, exactly: d * sc is an f16 times a six-bit
            // integer (17 significant bits), MAGIC * d * sc has 19, so neither product rounds and
            // the fma rounds dot * d * sc once, as convert-then-multiply would.
            constexpr int MAGIC_BITS = 0x4B400000;
            constexpr float MAGIC = 12582912.0f;
            v16i c;
#pragma unroll
            for (int v = 0; v < 16; ++v) c[v] = MAGIC_BITS;
            c = __builtin_amdgcn_mfma_i32_32x32x32_i8(f.a[s], b, c, 0, 0, 0);
            const float* d8_sub = d8_table + (kb * 8 + s) * TOK;
            // min term: this lane's activation row and half of the sub-block
            const uint4 au = make_uint4((uint32_t)f.a[s][0], (uint32_t)f.a[s][1], (uint32_t)f.a[s][2], (uint32_t)f.a[s][3]);
            const float half_sum = d8_sub[l32] * (float)dot16(ones, au, 0);
            acc_min = __builtin_amdgcn_mfma_f32_32x32x2f32(half_sum, dmm[s], acc_min, 0, 0, 0);
            // scale term: register v stands for activation row (v / 4) * 8 + lh * 4 + v % 4
            const float off = -MAGIC * dsc[s];
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const float4 t = *(const float4*)(d8_sub + 8 * g + 4 * lh);
                acc[4 * g + 0] = fmaf(fmaf(__int_as_float(c[4 * g + 0]), dsc[s], off), t.x, acc[4 * g + 0]);
                acc[4 * g + 1] = fmaf(fmaf(__int_as_float(c[4 * g + 1]), dsc[s], off), t.y, acc[4 * g + 1]);
                acc[4 * g + 2] = fmaf(fmaf(__int_as_float(c[4 * g + 2]), dsc[s], off), t.z, acc[4 * g + 2]);
                acc[4 * g + 3] = fmaf(fmaf(__int_as_float(c[4 * g + 3]), dsc[s], off), t.w, acc[4 * g + 3]);
            }
        }
    };

    // Steps are (row tile, super-block) pairs: wave w takes super-blocks w, w + 4, ... of every
    // tile of this workgroup; the loads of the next step fly under the arithmetic of this one.
    const int my_blocks = (p.nb - wave + WAVES - 1) / WAVES;   // may be zero for short rows
    int tile = blockIdx.x, kb = wave;
    Frag fa, fb;
    if (tile < n_tiles && my_blocks > 0) load(fa, tile, kb);
    __syncthreads();   // the scale table is complete

    auto finish_tile = [&](int t) {
        // add the four partial tiles and write the activation rows this pass has
        float* mine = reduce + wave * (16 * 64);
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            mine[v * 64 + lane] = acc[v] + acc_min[v];
            acc[v] = acc_min[v] = 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int v = wave * 4 + r;
            const float sum = (reduce[v * 64 + lane] + reduce[(16 + v) * 64 + lane]) +
                              (reduce[(32 + v) * 64 + lane] + reduce[(48 + v) * 64 + lane]);
            const int tok = (v >> 2) * 8 + lh * 4 + (v & 3), row = t * 32 + l32;
            if (tok < m_count && row < p.n) p.dst[(size_t)(m0 + tok) * p.ldd + row] = sum;
        }
        __syncthreads();   // the partial tiles may be overwritten
    };

    while (tile < n_tiles) {
        if (my_blocks > 0) {
            for (;;) {
                int nt = tile, nk = kb + WAVES;
                const bool last = nk >= p.nb;
                if (last) { nk = wave; nt += gridDim.x; }
                if (nt < n_tiles) load(fb, nt, nk);
                compute(fa, kb);
                if (last) { finish_tile(tile); tile = nt; kb = nk; if (tile >= n_tiles) return; }
                else kb = nk;
                // second half of the ping-pong
                nt = tile; nk = kb + WAVES;
                const bool last2 = nk >= p.nb;
                if (last2) { nk = wave; nt += gridDim.x; }
                if (nt < n_tiles) load(fa, nt, nk);
                compute(fb, kb);
                if (last2) { finish_tile(tile); tile = nt; kb = nk; if (tile >= n_tiles) return; }
                else kb = nk;
            }
        } else {
            finish_tile(tile);   // nothing of its own to add, but the barriers are the workgroup's
            tile += gridDim.x;
        }
    }
}

int resident_cap(int lds_bytes) {
    static std::mutex mu;
    static std::unordered_map<int, int> by_lds;
    std::lock_guard<std::mutex> lock(mu);
    auto it = by_lds.find(lds_bytes);
    if (it != by_lds.end()) return it->second;
    int r = 0;
    if (lds_bytes > lk_device().lds_bytes) {
        r = 0;
    } else if (lds_bytes > 48 * 1024 &&
               hipFuncSetAttribute((const void*)q4k_rows_mfma_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                                   lds_bytes) != hipSuccess) {
        (void)hipGetLastError();
        r = 0;
    } else if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&r, (const void*)q4k_rows_mfma_kernel, WG,
                                                            (size_t)lds_bytes) != hipSuccess || r < 1) {
        (void)hipGetLastError();
        r = 1;
    }
    by_lds.emplace(lds_bytes, r);
    return r;
}

}  // namespace

// Returns LK_OK, or the reason nothing was launched.
int lk_q4k_rows_mfma(const void* w, const void* q8_1, float* output, int size_m, int size_n, int size_k,
                     int stride_y, int ldd, hipStream_t stream) {
    if (size_m == 0 || size_n == 0) return LK_OK;
    if (!w || !q8_1 || !output || size_m < 0 || size_n < 0 || size_k <= 0 || size_k % 256 != 0) return LK_ERR_ARG;
    if (stride_y < size_k / 32 || ldd < size_n) return LK_ERR_ARG;
    if ((((uintptr_t)w) & 15) != 0 || (((uintptr_t)q8_1) & 3) != 0) return LK_ERR_ARG;
    const int nb = size_k / 256;
    const int lds_bytes = (nb * 8 * TOK + WAVES * 16 * 64) * (int)sizeof(float);
    const int per_cu = resident_cap(lds_bytes);
    if (per_cu == 0) return LK_ERR_ARG;   // rows too long for the scale table
    const int n_tiles = (size_n + 31) / 32, groups = (size_m + TOK - 1) / TOK;
    if (groups > 65535) return LK_ERR_ARG;
    int cap = lk_device().cus * per_cu / groups;
    if (cap < 1) cap = 1;
    Args a{(const uint8_t*)w, (const uint8_t*)q8_1, output, nb, size_n, size_m, stride_y, ldd};
    hipLaunchKernelGGL(q4k_rows_mfma_kernel, dim3(n_tiles < cap ? n_tiles : cap, groups), dim3(WG), lds_bytes, stream, a);
    return lk_launch_status();
}

extern "C" void loken_dense_q4k_imma_m8_plain(const void* w, const void* q8_1, float* output, int size_m, int size_n,
                                              int size_k, void* stream) {
    (void)lk_q4k_rows_mfma(w, q8_1, output, size_m, size_n, size_k, size_k / 32, size_n, (hipStream_t)stream);
}
