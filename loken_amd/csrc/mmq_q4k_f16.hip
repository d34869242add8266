// Q4_K weight rows against 33 or more Q8_1 token rows (65 or more where they are an expert's run): the sub-block dots on the f16 matrix unit.
//
//   out[token, n] = sum over 256-value blocks of
//        d[n] * sum_s d8_s[token] * D_s[n, token]  -  dmin[n] * sum_s m_s[n] * (d8_s * S_s)[token]
//   D_s[n, token] = sum over the 32 values of sub-block s of (sc_s[n] * q[n, k]) * a[token, k]
//
// The same integers as the int8 tile kernel forms (sc * dot of 4-bit codes and int8 codes: loken's
// BlockQ4K::dot_scalar, src/tensor/quant_cpu/format/q4_k.rs:138-153, combined as cuda/moe/gguf.cuh:
// 664-713 combines them), reached another way. An int8 MFMA leaves dot_s, which still has to meet
// two factors per output element, sc_s[n] and d8_s[token]: a convert and two multiplies on the
// vector unit per element and sub-block, four to six times the cycles of the MFMA that fed them.
// Here the 6-bit scale rides into the matrix unit with the weight: sc * q <= 63 * 15 is exact in
// f16, so is an int8 code, their products and the 32-term sums are exact in the f32 accumulator
// (< 2^24). D_s leaves the unit as a float that already carries the weight scale, and one fma by
// the lane's d8 finishes it. Half the matrix rate of int8, a third of the vector work.
//
// Shape: a workgroup of eight waves takes 256 weight rows x 64 tokens; a wave owns 32 of the rows
// and both token tiles of 32; registers <-> weight rows, lanes <-> tokens (v_mfma_f32_32x32x16_f16
// called as weights x tokens). Per 256-value step the workgroup copies its 256 weight blocks into
// LDS as they lie in memory (consecutive lanes read consecutive 16-byte pieces of a row's block:
// loading them lane-per-row instead touches 64 cache lines per instruction and was a fifth of
// the kernel's time), and each lane then picks its row's nibbles out of LDS in operand order and
// expands them in registers. Token codes are expanded to f16 once per step into LDS. Both tiles
// are two stages deep, filled for step k + 1 while step k is multiplied, one barrier per step.
// The min term is a rank-8 update per block on the bf16 matrix unit, with d8 * S split into
// three bf16 pieces (24 bits, nothing lost).
//
// K order inside a sub-block: lane half h (lane / 32) of MFMA hf holds values 16 h + 8 hf + i,
// i in the order 0 2 1 3 4 6 5 7 (what masking a dword's even and odd bytes yields); weights and
// tokens use the same order, which is all a dot product asks.

#include "mmq_problem.h"

namespace {

typedef _Float16 h2 __attribute__((ext_vector_type(2)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));

static __device__ __forceinline__ h2 as_h2(uint32_t bits) { return __builtin_bit_cast(h2, bits); }
static __device__ __forceinline__ uint32_t h2_bits(h2 v) { return __builtin_bit_cast(uint32_t, v); }

constexpr uint32_t H1024 = 0x64006400u;   // two f16 1024.0: OR-ing an 8-bit integer into the mantissa adds it

struct Wide {
    static constexpr int WAVES = 8;                   // along the weight rows
    static constexpr int THREADS = 64 * WAVES;
    static constexpr int TT = 2;                      // token tiles of 32 per wave
    static constexpr int TM = 32 * TT;                // tokens per workgroup tile
    static constexpr int TN = 32 * WAVES;             // weight rows per workgroup tile
    static constexpr int CCH = TM * 16 / THREADS;     // 16-code chunks per thread per step
    static constexpr int PARTS = THREADS / TM;        // threads sharing one token's scales
    static_assert(TM * 16 % THREADS == 0 && PARTS == 8, "one sub-block's scale per thread");
    static constexpr int WCH = (TN * 9 + THREADS - 1) / THREADS;   // 16-byte weight chunks per thread per step
    // one token stage: f16 codes [plane = (s, hf, h)][token ^ swizzle][8 halves], d8 [s][token] f32,
    // pieces [hi, mid, lo, zero][token][8 bf16]; one weight stage: TN blocks of 144 bytes
    static constexpr int CODES = TM * 512, D8 = TM * 32, PIECES = 4 * TM * 16;
    static constexpr int STAGE = CODES + D8 + PIECES;
    static constexpr int WSTAGE = TN * Q4K_BYTES;
    static constexpr int LDS = 2 * STAGE + 2 * WSTAGE + WAVES * 256;   // + per wave: d and -dmin of its 32 rows
};

// The workgroup's copy of one step's weight blocks: chunk q = tid + i * THREADS is 16-byte piece
// q % 9 of row q / 9's block, and lands at byte 16 q of the stage.
struct WeightCopy {
    using C = Wide;
    const uint8_t* from[C::WCH];   // the chunk's address in step 0 (rows past the end re-read the last row)
    uint4 data[C::WCH];

    __device__ __forceinline__ void place(const uint8_t* w, int64_t row_bytes, int n0, int n) {
#pragma unroll
        for (int i = 0; i < C::WCH; ++i) {
            const int q = min((int)threadIdx.x + i * C::THREADS, C::TN * 9 - 1);
            from[i] = w + (int64_t)min(n0 + q / 9, n - 1) * row_bytes + 16 * (q % 9);
        }
    }
    // The last round has chunks for half the threads only; the others repeat the stage's last
    // chunk (same bytes to the same place), which keeps the step free of branches.
    __device__ __forceinline__ void fetch_part(int64_t step_bytes, int i) { data[i] = *(const uint4*)(from[i] + step_bytes); }
    __device__ __forceinline__ void commit_part(uint8_t* wstage, int i) const {
        *(uint4*)(wstage + min((int)threadIdx.x + i * C::THREADS, C::TN * 9 - 1) * 16) = data[i];
    }
    __device__ __forceinline__ void commit(uint8_t* wstage) const {
#pragma unroll
        for (int i = 0; i < C::WCH; ++i) commit_part(wstage, i);
    }
};

struct TokenFrag16 {
    using C = Wide;
    uint4 codes[C::CCH];
    uint16_t d8, sum;   // of sub-block tid / TM of token tid % TM

    // Byte offsets of this thread's loads inside one K step's slab of records (rows past the end
    // re-read the last row: their results are never stored).
    uint32_t code_at[C::CCH], scale_at;
    __device__ __forceinline__ void place(int m0, int m_end) {
        const int tid = threadIdx.x;
#pragma unroll
        for (int i = 0; i < C::CCH; ++i) {
            const int idx = tid + i * C::THREADS, r = idx >> 4, c = idx & 15;
            code_at[i] = (uint32_t)min(m0 + r, m_end - 1) * MMQ_REC_BYTES + 16 * c;
        }
        const int r = tid % C::TM, part = tid / C::TM;
        scale_at = (uint32_t)min(m0 + r, m_end - 1) * MMQ_REC_BYTES + 256 + 2 * part;
    }
    // Part i < CCH: a chunk of codes; part CCH: the scales and sums.
    static constexpr int FETCH_PARTS = C::CCH + 1;
    __device__ __forceinline__ void fetch_part(const uint8_t* __restrict__ slab, int i) {
        if (i < C::CCH) {
            codes[i] = *(const uint4*)(slab + code_at[i]);
        } else {
            d8 = *(const uint16_t*)(slab + scale_at);
            sum = *(const uint16_t*)(slab + scale_at + 16);
        }
    }
    __device__ __forceinline__ void fetch(const uint8_t* __restrict__ slab) {
#pragma unroll
        for (int i = 0; i < FETCH_PARTS; ++i) fetch_part(slab, i);
    }

    // four int8 codes -> f16, as the pairs (0, 2) and (1, 3)
    static __device__ __forceinline__ void expand(uint32_t u, uint32_t& even, uint32_t& odd) {
        // byte ^ 0x80 = code + 128 in 0..255; OR-ed into the mantissa of 1024.0 (one XOR does both:
        // the constants' bits do not overlap), then 1024 + 128 comes off
        const h2 bias = {(_Float16)1152.0f, (_Float16)1152.0f};
        even = h2_bits(as_h2((u & 0x00FF00FFu) ^ 0x64806480u) - bias);
        odd = h2_bits(as_h2(((u >> 8) & 0x00FF00FFu) ^ 0x64806480u) - bias);
    }

    // Part i of the registers into a stage (the parts of fetch_part).
    __device__ __forceinline__ void commit(uint8_t* stage) const {
#pragma unroll
        for (int i = 0; i < FETCH_PARTS; ++i) commit_part(stage, i);
    }
    __device__ __forceinline__ void commit_part(uint8_t* stage, int i) const {
        const int tid = threadIdx.x;
        if (i < C::CCH) {
            const int idx = tid + i * C::THREADS, r = idx >> 4, c = idx & 15;
            const int s = c >> 1, h = c & 1;
            const uint32_t u[4] = {codes[i].x, codes[i].y, codes[i].z, codes[i].w};
#pragma unroll
            for (int hf = 0; hf < 2; ++hf) {
                uint4 out;
                expand(u[2 * hf], out.x, out.y);
                expand(u[2 * hf + 1], out.z, out.w);
                const int plane = (s * 2 + hf) * 2 + h;
                // the 16 lanes that share a token write 16 planes: the token index is XOR-ed with
                // the plane's (s, h) so that they land in 16 different bank groups
                *(uint4*)(stage + (plane * C::TM + (r ^ c)) * 16) = out;
            }
            return;
        }
        float* ad8 = (float*)(stage + C::CODES);
        uint8_t* ap = stage + C::CODES + C::D8;
        const int r = tid % C::TM, s = tid / C::TM;
        const float d = f16_bits_to_f32(d8);
        ad8[s * C::TM + r] = d;
        // d8 * S as three bf16 (truncations of the running remainder: 8 bits each, exact)
        const float p0 = d * (float)(int)(int16_t)sum;
        const uint32_t b0 = __float_as_uint(p0) & 0xFFFF0000u;
        const float p1 = p0 - __uint_as_float(b0);
        const uint32_t b1 = __float_as_uint(p1) & 0xFFFF0000u;
        const float p2 = p1 - __uint_as_float(b1);
        const uint32_t b2 = __float_as_uint(p2) & 0xFFFF0000u;
        const int at = r * 16 + s * 2;
        *(uint16_t*)(ap + 0 * C::TM * 16 + at) = (uint16_t)(b0 >> 16);
        *(uint16_t*)(ap + 1 * C::TM * 16 + at) = (uint16_t)(b1 >> 16);
        *(uint16_t*)(ap + 2 * C::TM * 16 + at) = (uint16_t)(b2 >> 16);
    }
};

// The 6-bit scales and mins of a Q4_K block header (get_scale_min_k4 of the format).
static __device__ __forceinline__ void unpack_scales(const uint4& hdr, uint32_t sc[8], uint32_t mn[8]) {
    const uint32_t w1 = hdr.y, w2 = hdr.z, w3 = hdr.w;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        sc[j] = (w1 >> (8 * j)) & 63u;
        mn[j] = (w2 >> (8 * j)) & 63u;
        sc[j + 4] = ((w3 >> (8 * j)) & 0xFu) | ((((w1 >> (8 * j)) >> 6) & 3u) << 4);
        mn[j + 4] = ((w3 >> (8 * j + 4)) & 0xFu) | ((((w2 >> (8 * j)) >> 6) & 3u) << 4);
    }
}

// The two A operands of sub-block s from the lane's 16 bytes of its 64-value pair:
// (1024 + q) * sc - 1024 * sc for the low nibbles; the high nibbles sit four bits up,
// (1024 + 16 q) * (sc / 16) - 64 * sc. Both exact in f16 (sc <= 63).
static __device__ __forceinline__ void weight_operands(const uint4& q, bool high, uint32_t sc, uint32_t h1024, v8h a[2]) {
    const _Float16 scale = (_Float16)((float)sc * (high ? 0.0625f : 1.0f));
    const _Float16 offset = (_Float16)((float)sc * (high ? -64.0f : -1024.0f));
    const h2 scale2 = {scale, scale}, offset2 = {offset, offset};
    const uint32_t mask = high ? 0x00F000F0u : 0x000F000Fu;
    const uint32_t u[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
    for (int hf = 0; hf < 2; ++hf) {
        uint32_t ab[4];
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            const uint32_t x = u[2 * hf + e];
            ab[2 * e] = h2_bits(__builtin_elementwise_fma(as_h2((x & mask) | h1024), scale2, offset2));
            ab[2 * e + 1] = h2_bits(__builtin_elementwise_fma(as_h2(((x >> 8) & mask) | h1024), scale2, offset2));
        }
        a[hf] = __builtin_bit_cast(v8h, make_uint4(ab[0], ab[1], ab[2], ab[3]));
    }
}

// The B operands and the token scale of item (s, tt). `ad8` already points at the lane's token.
static __device__ __forceinline__ void load_item(const uint8_t* stage, const uint8_t* ad8, int s, int tt, int token0,
                                                 int h, v8h b[2], float& d8) {
    // token0 ^ (2 s + h) only changes the low four bits, so the tile offset 32 tt adds on top
    using C = Wide;
    const uint8_t* at = stage + (token0 ^ (2 * s + h)) * 16 + h * C::TM * 16 + tt * 512;
    b[0] = *(const v8h*)(at + (s * 4 + 0) * C::TM * 16);
    b[1] = *(const v8h*)(at + (s * 4 + 2) * C::TM * 16);
    d8 = *(const float*)(ad8 + (s * C::TM + 32 * tt) * 4);
}

// Half `HALF` of item `it`'s 16 results into the block's partial sums.
template <int TT, int HALF>
static __device__ __forceinline__ void scale_item(int it, const v16f& dot, float d8, v16f part[TT]) {
    const int s = it / TT, tt = it % TT;
#pragma unroll
    for (int v = 8 * HALF; v < 8 * HALF + 8; ++v) part[tt][v] = s == 0 ? dot[v] * d8 : fmaf(dot[v], d8, part[tt][v]);
}

static __device__ __forceinline__ void q4k_f16_tile(const MmqProblem& pb, int n0, int m0, uint8_t* lds) {
    using C = Wide;
    constexpr int TM = C::TM, TT = C::TT;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int j = lane & 31, h = lane >> 5;
    uint8_t* wstages = lds + 2 * C::STAGE;
    float* wd = (float*)(wstages + 2 * C::WSTAGE) + wave * 64;   // [0, 32) d, [32, 64) -dmin of the wave's rows
    const int last = (int)pb.nb - 1;

    v16f acc[TT];
#pragma unroll
    for (int tt = 0; tt < TT; ++tt)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[tt][v] = 0.f;

    // the zero piece of both stages (the second bf16 MFMA of the min term has 8 spare K slots)
    for (int i = tid; i < 2 * TM; i += C::THREADS) {
        uint8_t* stage = lds + (i / TM) * C::STAGE;
        *(uint4*)(stage + C::CODES + C::D8 + (3 * TM + i % TM) * 16) = make_uint4(0, 0, 0, 0);
    }

    WeightCopy wc;
    TokenFrag16 tf;
    const int64_t slab_bytes = pb.rows_total * MMQ_REC_BYTES;
    tf.place(m0, pb.m_end);
    wc.place(pb.w, pb.row_blocks * Q4K_BYTES, n0, pb.n);
    tf.fetch(pb.y);
#pragma unroll
    for (int i = 0; i < C::WCH; ++i) wc.fetch_part(0, i);
    tf.commit(lds);
    wc.commit(wstages);
    tf.fetch(pb.y + min(1, last) * slab_bytes);
#pragma unroll
    for (int i = 0; i < C::WCH; ++i) wc.fetch_part((int64_t)min(1, last) * Q4K_BYTES, i);
    __syncthreads();

    // 1024.0 | 1024.0 in a vector register: with the mask as the instruction's one literal,
    // (x & mask) | h1024 is a single v_and_or_b32
    uint32_t h1024 = H1024;
    asm volatile("" : "+v"(h1024));
    const int token0 = j;   // the lane's token in the first token tile

    for (int kb = 0; kb <= last; ++kb) {
        const uint8_t* stage = lds + (kb & 1) * C::STAGE;
        const uint8_t* ad8 = stage + C::CODES + token0 * 4;
        const uint8_t* ap = stage + C::CODES + C::D8 + token0 * 16;
        // the lane's row in the weight stage; its half of pair p's nibbles at +16 + 32 p + 16 h
        const uint8_t* wblock = wstages + (kb & 1) * C::WSTAGE + (32 * wave + j) * Q4K_BYTES;
        const uint8_t* next_slab = pb.y + min(kb + 2, last) * slab_bytes;
        const int64_t next_step = (int64_t)min(kb + 2, last) * Q4K_BYTES;

        const uint4 hdr = *(const uint4*)wblock;
        uint4 nib = *(const uint4*)(wblock + 16 + 16 * h);
        uint32_t sc[8], mn[8];
        unpack_scales(hdr, sc, mn);
        if (h == 0) {
            wd[j] = f16_bits_to_f32(hdr.x & 0xFFFFu);
            wd[32 + j] = -f16_bits_to_f32(hdr.x >> 16);
        }

        // Items (s, tt) run through a three-deep pipeline written out by hand: the LDS reads of
        // item i + 1, the two MFMAs of item i, the 16 fmas of item i - 1. Left to itself the
        // scheduler keeps one item in flight (read, wait, multiply, wait, scale).
        constexpr int NI = 8 * TT;
        v8h a[2][2], b[2][2];
        float d8v[3];   // read at item i + 1's loads, used at item i - 1's fmas: three alive
        v16f dot[2], part[TT];
        weight_operands(nib, false, sc[0], h1024, a[0]);
        load_item(stage, ad8, 0, 0, token0, h, b[0], d8v[0]);
#pragma unroll
        for (int it = 0; it < NI; ++it) {
            const int s = it / TT;
            if (it + 1 < NI) load_item(stage, ad8, (it + 1) / TT, (it + 1) % TT, token0, h, b[(it + 1) & 1], d8v[(it + 1) % 3]);
            // the nibbles of the pair after this one (read one sub-block before they are expanded)
            uint4 nib_next = nib;
            if (it % TT == 0 && (s & 1) == 0 && s + 2 < 8) nib_next = *(const uint4*)(wblock + 16 + 32 * ((s + 2) >> 1) + 16 * h);
            // The second MFMA takes the first one's result as its accumulator and cannot issue
            // before that is written, and a wave's own vector instructions do not issue past a
            // waiting one: whatever should run meanwhile has to sit between the two.
            {
                v16f zero = {0.f};
                dot[it & 1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[s & 1][0], b[it & 1][0], zero, 0, 0, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
            if (it >= 1) scale_item<TT, 0>(it - 1, dot[(it - 1) & 1], d8v[(it - 1) % 3], part);
            __builtin_amdgcn_sched_barrier(0);
            dot[it & 1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[s & 1][1], b[it & 1][1], dot[it & 1], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
            if (it >= 1) scale_item<TT, 1>(it - 1, dot[(it - 1) & 1], d8v[(it - 1) % 3], part);
            if (it % TT == 0 && s + 1 < 8) {
                // sub-block s + 1: the high nibbles of the current pair, or the low ones of the next
                if ((s + 1) & 1) {
                    weight_operands(nib, true, sc[s + 1], h1024, a[(s + 1) & 1]);
                    nib = nib_next;
                } else {
                    weight_operands(nib, false, sc[s + 1], h1024, a[(s + 1) & 1]);
                }
            }
            // The next step's tokens and weights leave their registers for the other stages (whose
            // last readers left at the barrier that ended the previous step) one part per item, so
            // that eight waves' LDS writes do not arrive in one burst; each part's registers take
            // the load of the step after next one item later.
            constexpr int PARTS = TokenFrag16::FETCH_PARTS + C::WCH;
            constexpr int FIRST = NI - 1 - PARTS;
            static_assert(FIRST >= 0, "more parts than items to spread them over");
            {
                const int c = it - FIRST, f = it - FIRST - 1;   // the part committed / fetched at this item
                uint8_t* to = lds + ((kb + 1) & 1) * C::STAGE;
                uint8_t* wto = wstages + ((kb + 1) & 1) * C::WSTAGE;
                if (c >= 0 && c < C::WCH) wc.commit_part(wto, c);
                if (c >= C::WCH && c < PARTS) tf.commit_part(to, c - C::WCH);
                if (f >= 0 && f < C::WCH) wc.fetch_part(next_step, f);
                if (f >= C::WCH && f < PARTS) tf.fetch_part(next_slab, f - C::WCH);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        scale_item<TT, 0>(NI - 1, dot[(NI - 1) & 1], d8v[(NI - 1) % 3], part);
        scale_item<TT, 1>(NI - 1, dot[(NI - 1) & 1], d8v[(NI - 1) % 3], part);

        // the block's two per-row factors, for the 16 rows this lane's registers stand for
        __builtin_amdgcn_wave_barrier();
        float dv[16], ndm[16];
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const float4 t = *(const float4*)(wd + 8 * g + 4 * h);
            const float4 u = *(const float4*)(wd + 32 + 8 * g + 4 * h);
            dv[4 * g + 0] = t.x; dv[4 * g + 1] = t.y; dv[4 * g + 2] = t.z; dv[4 * g + 3] = t.w;
            ndm[4 * g + 0] = u.x; ndm[4 * g + 1] = u.y; ndm[4 * g + 2] = u.z; ndm[4 * g + 3] = u.w;
        }
        __builtin_amdgcn_wave_barrier();
        // small integers as bf16: the top half of their f32
        uint32_t mb[4];
#pragma unroll
        for (int q = 0; q < 4; ++q)
            mb[q] = (__float_as_uint((float)mn[2 * q]) >> 16) | (__float_as_uint((float)mn[2 * q + 1]) & 0xFFFF0000u);
        const v8bf m_op = __builtin_bit_cast(v8bf, make_uint4(mb[0], mb[1], mb[2], mb[3]));
#pragma unroll
        for (int tt = 0; tt < TT; ++tt) {
            const v8bf p0 = *(const v8bf*)(ap + (h * TM + 32 * tt) * 16);          // hi | mid
            const v8bf p1 = *(const v8bf*)(ap + ((2 + h) * TM + 32 * tt) * 16);    // lo | zero
            v16f mins = {0.f};
            mins = __builtin_amdgcn_mfma_f32_32x32x16_bf16(m_op, p0, mins, 0, 0, 0);
            mins = __builtin_amdgcn_mfma_f32_32x32x16_bf16(m_op, p1, mins, 0, 0, 0);
#pragma unroll
            for (int v = 0; v < 16; ++v)
                acc[tt][v] = fmaf(ndm[v], mins[v], fmaf(dv[v], part[tt][v], acc[tt][v]));
        }
        __syncthreads();
    }

    const bool vec_ok = ((uintptr_t)pb.dst % 16 == 0) && (pb.ldd % 4 == 0);
#pragma unroll
    for (int tt = 0; tt < TT; ++tt) {
        const int col = m0 + 32 * tt + j;
        if (col >= pb.m_end) continue;
        const int64_t drow = pb.ids_dst ? pb.ids_dst[col] : col;
        float* out = pb.dst + drow * pb.ldd;
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const int gn0 = n0 + 32 * wave + 8 * g + 4 * h;
            if (vec_ok && gn0 + 3 < pb.n) {
                *(float4*)(out + gn0) = make_float4(acc[tt][4 * g], acc[tt][4 * g + 1], acc[tt][4 * g + 2], acc[tt][4 * g + 3]);
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (gn0 + e < pb.n) out[gn0 + e] = acc[tt][4 * g + e];
            }
        }
    }
}

// Workgroup id -> (n tile, m tile): the m tiles of one n tile re-read the same weight rows, so
// they are issued back to back on one XCD (ids are dealt round robin over the 8 XCDs).
__global__ __launch_bounds__(Wide::THREADS, 1) void q4k_f16_dense_kernel(MmqProblem pb, int n_tiles, int m_tiles) {
    extern __shared__ __align__(16) uint8_t lds[];
    const int id = blockIdx.x;
    const int xcd = id & 7, seq = id >> 3;
    const int m_tile = seq % m_tiles;
    const int n_tile = (seq / m_tiles) * 8 + xcd;
    if (n_tile >= n_tiles) return;
    q4k_f16_tile(pb, n_tile * Wide::TN, pb.m_begin + m_tile * Wide::TM, lds);
}

// The same tiles over one of `splits` ranges of K each, the partial tile to part[range].
__global__ __launch_bounds__(Wide::THREADS, 1) void q4k_f16_dense_split_kernel(MmqProblem pb, int n_tiles, int m_tiles,
                                                                              int splits, float* part, int64_t part_stride) {
    extern __shared__ __align__(16) uint8_t lds[];
    const int id = blockIdx.x;
    const int xcd = id & 7;
    int seq = id >> 3;
    const int m_tile = seq % m_tiles;
    seq /= m_tiles;
    const int split = seq % splits;
    const int n_tile = (seq / splits) * 8 + xcd;
    if (n_tile >= n_tiles) return;
    const int64_t kb0 = pb.nb * split / splits, kb1 = pb.nb * (split + 1) / splits;
    pb.w += kb0 * Q4K_BYTES;
    pb.y += kb0 * pb.rows_total * MMQ_REC_BYTES;
    pb.nb = kb1 - kb0;
    pb.dst = part + split * part_stride;
    pb.ldd = pb.n;
    q4k_f16_tile(pb, n_tile * Wide::TN, pb.m_begin + m_tile * Wide::TM, lds);
}

// Expert-batched: expert e's slab against the sorted rows [bounds[e], bounds[e+1]).
__global__ __launch_bounds__(Wide::THREADS, 1) void q4k_f16_moe_kernel(MmqProblem pb, const uint8_t* w_second,
                                                                      int64_t dst_second,
                                                                      const int32_t* __restrict__ bounds,
                                                                      int64_t stride_expert, int n_experts) {
    extern __shared__ __align__(16) uint8_t lds[];
    const int stack = blockIdx.z / n_experts, e = blockIdx.z % n_experts;
    pb.m_begin = bounds[e];
    pb.m_end = bounds[e + 1];
    if (pb.m_end <= pb.m_begin) return;
    pb.w = (stack ? w_second : pb.w) + (int64_t)e * stride_expert;
    if (stack) pb.dst += dst_second;
    for (int m0 = pb.m_begin + blockIdx.y * Wide::TM; m0 < pb.m_end; m0 += gridDim.y * Wide::TM) {
        q4k_f16_tile(pb, blockIdx.x * Wide::TN, m0, lds);
        __syncthreads();   // the next tile's prologue rewrites the first stages
    }
}

}  // namespace

int lk_mmq_q4k_f16_dense(const MmqProblem& pb, hipStream_t s, void* fixup) {
    using C = Wide;
    if (((uintptr_t)pb.w | (uintptr_t)pb.y) % 16 != 0 || pb.rows_total > (1 << 23)) return -1;
    const int n_tiles = (pb.n + C::TN - 1) / C::TN;
    const int m_tiles = (pb.m_end - pb.m_begin + C::TM - 1) / C::TM;
    const int splits = mmq_splits(pb, (int64_t)n_tiles * m_tiles, lk_device().cus, fixup);   // one workgroup a CU
    if (splits > 1) {
        if (mmq_prepare_kernel(q4k_f16_dense_split_kernel, C::LDS) != LK_OK) return 0;
        hipLaunchKernelGGL(q4k_f16_dense_split_kernel, dim3((n_tiles + 7) / 8 * 8 * m_tiles * splits), dim3(C::THREADS), C::LDS,
                           s, pb, n_tiles, m_tiles, splits, (float*)fixup, (int64_t)pb.m_end * pb.n);
        return lk_mmq_split_sum((const float*)fixup, splits, pb, s) == LK_OK ? C::TM : 0;
    }
    if (mmq_prepare_kernel(q4k_f16_dense_kernel, C::LDS) != LK_OK) return 0;
    const int grid = (n_tiles + 7) / 8 * 8 * m_tiles;
    hipLaunchKernelGGL(q4k_f16_dense_kernel, dim3(grid), dim3(C::THREADS), C::LDS, s, pb, n_tiles, m_tiles);
    return hipGetLastError() == hipSuccess ? C::TM : 0;
}

int lk_mmq_q4k_f16_moe(const MmqProblem& pb, const uint8_t* w_second, int64_t dst_second, const int32_t* bounds,
                       int64_t stride_expert, int n_experts, int64_t ncols_max, hipStream_t s) {
    using C = Wide;
    if (((uintptr_t)pb.w | (uintptr_t)pb.y | (uintptr_t)w_second) % 16 != 0 || stride_expert % 16 != 0 ||
        pb.rows_total > (1 << 23))
        return -1;
    if (mmq_prepare_kernel(q4k_f16_moe_kernel, C::LDS) != LK_OK) return 0;
    const int64_t col_tiles = (ncols_max + C::TM - 1) / C::TM;
    const dim3 grid((pb.n + C::TN - 1) / C::TN, (unsigned)(col_tiles < 1 ? 1 : (col_tiles > 65535 ? 65535 : col_tiles)),
                    (unsigned)((w_second ? 2 : 1) * n_experts));
    hipLaunchKernelGGL(q4k_f16_moe_kernel, grid, dim3(C::THREADS), C::LDS, s, pb, w_second, dst_second, bounds,
                       stride_expert, n_experts);
    return hipGetLastError() == hipSuccess ? C::TM : 0;
}
