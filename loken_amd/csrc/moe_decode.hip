// MoE decode: one mat-vec per routed (token, expert) pair, for batches too small to fill the
// expert-batched tiles. Entry points, argument lists and row conventions are loken's
// (src/inference/moe_cuda/mod.rs:235-262, 415-442, 473-483; cuda/moe/moe_gguf.cu:403-511,
// 528-608, 755-860, 896-1060):
//   sorted_token_ids[i] is the flattened (token * topk + choice) slot of routed pair i and
//   expert_ids[i] its expert; gate/up read activation row slot / topk and write row slot; down
//   reads row slot, scales by topk_weights[slot] and writes row slot of a scratch that a fold
//   then sums per token IN SLOT ORDER (no atomics, the same sum on every run).
// The launchers quantize the activation themselves into a per-(device, stream) grow-only
// scratch, as the reference's do; loken_stream_scratch_release frees it.
//
// Kernels: grid (row tiles, pairs); each workgroup stages its pair's Q8_1 row into LDS and runs
// the shared mat-vec row engine on the pair's expert slab. SiLU uses the accurate expf, as the
// host path does (src/inference/moe_cuda_cpu/mod.rs:598).

#include "mmvq_core.h"

#include <mutex>
#include <unordered_map>
#include <vector>

using namespace mmvq;

extern "C" int lk_quantize_q8_1(const void* x, int x_type, void* vy, int kx, int kx_padded, int rows, void* stream);
// moe_down_fold.hip: down + fold of short-row Q4_K / Q5_K / Q6_K experts in one launch; -1: not served
int lk_moe_down_fold(int quant_type, const float* inputs, const void* weights, const int32_t* sorted_token_ids,
                     const int32_t* expert_ids, const float* topk_weights, float* outputs, int num_experts, int topk,
                     int size_m, int size_n, int size_k, const float* down_bias, const float* add_after,
                     hipStream_t stream);

namespace {

// ---------------------------------------------------------------- stream scratch
struct ScratchSlot {
    int device;
    hipStream_t stream;
    void* ptr = nullptr;
    size_t size = 0;
    std::vector<void*> kept;  // outgrown buffers: queued kernels may still read them
};
std::mutex g_scratch_mu;
std::vector<ScratchSlot> g_scratch;

// Caller holds g_scratch_mu from the reservation until its launches are on the stream: the
// buffer belongs to the stream, and another thread's quantize landing between a launcher's
// two kernels is what the second would then read.
void* reserve_scratch(size_t bytes, hipStream_t stream) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return nullptr;
    ScratchSlot* slot = nullptr;
    for (auto& s : g_scratch)
        if (s.device == dev && s.stream == stream) slot = &s;
    if (!slot) {
        g_scratch.push_back(ScratchSlot{dev, stream});
        slot = &g_scratch.back();
    }
    if (slot->size >= bytes) return slot->ptr;
    // growing allocates, which a stream under capture may not do
    hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &cs) == hipSuccess && cs != hipStreamCaptureStatusNone) return nullptr;
    (void)hipGetLastError();
    size_t want = bytes + bytes / 4;
    want = (want + 255) & ~(size_t)255;
    void* fresh = nullptr;
    if (hipMalloc(&fresh, want) != hipSuccess) {
        (void)hipGetLastError();
        return nullptr;
    }
    if (slot->ptr) slot->kept.push_back(slot->ptr);
    slot->ptr = fresh;
    slot->size = want;
    return fresh;
}

// ---------------------------------------------------------------- static scratch
// Scratch of the entry point that allocates nothing (loken_moe_gemm_gguf_down_reduce_static): a
// fixed array in every device's copy of the library image. Each GPU holds its own copy at its own
// address; the name below is only the host's handle for it, so host code asks the runtime for the
// device address once per device and passes that.
constexpr size_t STATIC_SCRATCH_BYTES = LK_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) uint8_t scratch[STATIC_SCRATCH_BYTES];

std::mutex g_static_mu;
std::vector<std::pair<int, uint8_t*>> g_static_ptr;   // (device, address of `scratch` there)

uint8_t* static_scratch() {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return nullptr;
    std::lock_guard<std::mutex> lock(g_static_mu);
    for (const auto& e : g_static_ptr)
        if (e.first == dev) return e.second;
    uint8_t* ptr = nullptr;
    if (hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(scratch)) != hipSuccess || ptr == nullptr) {
        (void)hipGetLastError();
        return nullptr;
    }
    g_static_ptr.emplace_back(dev, ptr);
    return ptr;
}

// ---------------------------------------------------------------- kernels
struct MoeDims {
    int experts, topk, pairs, cols, nb, k32;  // k32: Q8_1 blocks between activation rows
    int64_t slab_bytes;                       // one expert's weights
    int act_f32 = 0;                          // non-zero: `acts` holds f32 rows this many floats apart and
                                              // every workgroup quantizes its pair's row while staging it
    int slab_rows = 0;                        // weight rows per expert when not `cols` (gate and up in one tensor)
    LkGateAct act;                            // MODE_GATED: what becomes of (gate . x, up . x)
    const unsigned int* live = nullptr;       // when given: only the first *live pairs run
    LkMoeAlt alt;                             // the experts from alt.alt_from on live in a second tensor
};

enum { MODE_PLAIN = 0, MODE_GATED = 1, MODE_DOWN = 2 };

template <class E, int R, int MODE>
__global__ __launch_bounds__(WG) void moe_rows_kernel(const uint8_t* __restrict__ w0, const uint8_t* __restrict__ w1,
                                                      const uint8_t* __restrict__ acts,
                                                      const int32_t* __restrict__ sorted_token_ids,
                                                      const int32_t* __restrict__ expert_ids,
                                                      const float* __restrict__ topk_weights,
                                                      const float* __restrict__ down_bias,
                                                      float* __restrict__ out, MoeDims d) {
    extern __shared__ __align__(16) uint8_t lds[];
    const int pair = blockIdx.y;
    // The pair's routing and the live count in ONE round of scalar loads, and the launch's fields in
    // the round before it: asked for where each is first used they arrive in eight dependent rounds.
    const int slot = sorted_token_ids[pair];
    const int e = expert_ids[pair];
    const unsigned int live = d.live != nullptr ? *d.live : 0xFFFFFFFFu;
    asm volatile("" ::"s"(slot), "s"(e), "s"(live), "s"(d.pairs), "s"(d.experts), "s"(d.cols), "s"(d.nb), "s"(d.k32),
                 "s"(d.act_f32), "s"(d.topk), "s"(w0), "s"(w1), "s"(acts), "s"(out), "s"(topk_weights), "s"(d.slab_bytes),
                 "s"(d.alt.alt0), "s"(d.alt.alt_at), "s"(d.alt.alt_from), "s"(d.act.kind));
    if ((unsigned int)pair >= live) return;
    if (slot < 0 || slot >= d.pairs) return;
    float* out_row = out + (size_t)slot * d.cols;
    if (e < 0 || e >= d.experts) {
        // a pair the routing leaves out adds nothing: its row of the fold's input reads zero
        if (MODE == MODE_DOWN)
            for (int r = blockIdx.x * WG + threadIdx.x; r < d.cols; r += gridDim.x * WG) out_row[r] = 0.f;
        return;
    }
    const bool own_row = MODE == MODE_DOWN || (MODE == MODE_PLAIN && topk_weights != nullptr);
    const int act_row = own_row ? slot : slot / d.topk;
    const uint8_t* vy = d.act_f32 ? acts + (size_t)act_row * d.act_f32 * sizeof(float)
                                  : acts + (size_t)act_row * d.k32 * Q81_BYTES;
    const float scale = (MODE != MODE_GATED && topk_weights) ? topk_weights[slot] : 1.0f;
    const uint8_t* slab0 = lk_expert_slab(w0, 0, d.alt, e, d.slab_bytes);
    const int tile_stride = (int)gridDim.x * WAVES, tile_first = (int)blockIdx.x * WAVES;
    if (MODE == MODE_GATED) {
        const uint8_t* slab1 = lk_expert_slab(w1, 1, d.alt, e, d.slab_bytes);
        RowJob<2> job{{to_gbytes(slab0), to_gbytes(slab1)}, vy, d.nb, d.cols, d.k32, tile_stride, tile_first, d.act_f32};
        E::template run<1, R, 2>(job, lds, [&](int row, int, const float* tot) {
            out_row[row] = lk_gated(d.act, tot[0], tot[1], (size_t)e * d.cols + row);
        });
    } else {
        RowJob<1> job{{to_gbytes(slab0)}, vy, d.nb, d.cols, d.k32, tile_stride, tile_first, d.act_f32};
        E::template run<1, R, 1>(job, lds, [&](int row, int, const float* tot) {
            float v = tot[0] * scale;
            if (MODE == MODE_DOWN && down_bias) v += scale * down_bias[(size_t)e * d.cols + row];
            out_row[row] = v;
        });
    }
}

// outputs[t] (+)= sum over k ascending of pairs[t * topk + k]; with `add` the result is written
// as fold + add instead of accumulated (cuda/moe/moe_gguf.cu:591-625).
__global__ void sum_topk_kernel(const float* __restrict__ pairs, const float* __restrict__ add,
                                float* __restrict__ outputs, int tokens, int topk, int cols) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (size_t)tokens * cols) return;
    const size_t token = i / cols, col = i % cols;
    float acc = add ? 0.0f : outputs[i];
    const float* p = pairs + token * topk * cols + col;
    // four rows' loads in flight at a time; the additions stay in k order
    int k = 0;
    for (; k + 4 <= topk; k += 4) {
        const float p0 = p[(size_t)k * cols], p1 = p[(size_t)(k + 1) * cols], p2 = p[(size_t)(k + 2) * cols],
                    p3 = p[(size_t)(k + 3) * cols];
        acc += p0;
        acc += p1;
        acc += p2;
        acc += p3;
    }
    for (; k < topk; ++k) acc += p[(size_t)k * cols];
    outputs[i] = add ? acc + add[i] : acc;
}

template <typename K>
static int prepare(K kernel, int lds_bytes) {
    static std::mutex mu;
    static std::unordered_map<int, int> by_lds;
    std::lock_guard<std::mutex> lock(mu);
    auto it = by_lds.find(lds_bytes);
    if (it != by_lds.end()) return it->second;
    if (lds_bytes > lk_device().lds_bytes) return 0;
    if (lds_bytes > 48 * 1024 &&
        hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes) != hipSuccess) {
        (void)hipGetLastError();
        return 0;
    }
    int r = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&r, (const void*)kernel, WG, (size_t)lds_bytes) != hipSuccess || r < 1) {
        (void)hipGetLastError();
        r = 1;
    }
    r = r > 8 ? 8 : r;
    by_lds.emplace(lds_bytes, r);
    return r;
}

template <class E, int MODE>
static int launch_mode(const uint8_t* w0, const uint8_t* w1, const uint8_t* acts, const int32_t* sti,
                       const int32_t* eid, const float* tw, const float* bias, float* out, const MoeDims& d,
                       hipStream_t s) {
    constexpr int R = MODE == MODE_GATED ? 1 : 2;
    auto kernel = moe_rows_kernel<E, R, MODE>;
    const int lds_bytes = lds_bytes_for<typename E::Fmt>(d.nb, 1);
    const int per_cu = prepare(kernel, lds_bytes);
    if (per_cu == 0) return LK_ERR_ARG;
    const int tile_rows = R * E::rows_per_pass(d.nb);
    const int tiles = (d.cols + tile_rows - 1) / tile_rows;
    const int need = (tiles + WAVES - 1) / WAVES;
    int share = lk_device().cus * per_cu / d.pairs;
    if (share < 1) share = 1;
    const dim3 grid(need < share ? need : share, d.pairs);
    if (grid.y > 65535u) return LK_ERR_ARG;
    hipLaunchKernelGGL(kernel, grid, dim3(WG), lds_bytes, s, w0, w1, acts, sti, eid, tw, bias, out, d);
    return lk_launch_status();
}

template <int MODE>
static int launch_format(int quant_type, const uint8_t* w0, const uint8_t* w1, const uint8_t* acts, const int32_t* sti,
                         const int32_t* eid, const float* tw, const float* bias, float* out, MoeDims d, int size_k,
                         hipStream_t s) {
    const int64_t slab_rows = d.slab_rows ? d.slab_rows : d.cols;
    switch (quant_type) {   // wire ids of the reference's MOE_GGUF_FORMATS table (cuda/moe/gguf.cuh:55-71)
        case 0:
            d.nb = size_k / 32; d.slab_bytes = slab_rows * d.nb * Q80_BYTES;
            return launch_mode<EngQ80, MODE>(w0, w1, acts, sti, eid, tw, bias, out, d, s);
        case 1:
            d.nb = size_k / 256; d.slab_bytes = slab_rows * d.nb * Q4K_BYTES;
            return d.nb <= 8 ? launch_mode<EngQ4KShort, MODE>(w0, w1, acts, sti, eid, tw, bias, out, d, s)
                             : launch_mode<EngQ4K, MODE>(w0, w1, acts, sti, eid, tw, bias, out, d, s);
        case 4:
            d.nb = size_k / 256; d.slab_bytes = slab_rows * d.nb * Q5K_BYTES;
            return d.nb <= 8 ? launch_mode<EngQ5KShort, MODE>(w0, w1, acts, sti, eid, tw, bias, out, d, s)
                             : launch_mode<EngQ5K, MODE>(w0, w1, acts, sti, eid, tw, bias, out, d, s);
        case 5:
            d.nb = size_k / 256; d.slab_bytes = slab_rows * d.nb * Q6K_BYTES;
            return d.nb <= 8 ? launch_mode<EngQ6KShort, MODE>(w0, w1, acts, sti, eid, tw, bias, out, d, s)
                             : launch_mode<EngQ6K, MODE>(w0, w1, acts, sti, eid, tw, bias, out, d, s);
        default:
            // Q2_K, Q3_K, Q5_0, MXFP4, Q5_1, IQ4_NL, IQ4_XS and the codebook formats IQ3_XXS, IQ3_S, IQ2_S, Q2_0,
            // IQ2_XXS: the wave-per-row kernels over Q8_1 rows
            if (d.act_f32) return LK_ERR_ARG;
            return lk_moe_rows_legacy(MODE, quant_type, w0, w1, acts, sti, eid, tw, bias, out, d.experts, d.topk,
                                      d.pairs, d.cols, size_k, d.k32, d.act, (int)slab_rows, d.live, d.alt, s);
    }
}

static int block_len_of_wire(int quant_type) {
    if (quant_type == 0) return 32;
    if (quant_type == 1 || quant_type == 4 || quant_type == 5) return 256;
    return lk_moe_wire_block_len_legacy(quant_type);
}

static bool bad_shape(int quant_type, int num_experts, int topk, int size_m, int size_n, int size_k) {
    const int bl = block_len_of_wire(quant_type);
    return bl == 0 || num_experts <= 0 || topk <= 0 || size_m < 0 || size_n <= 0 || size_k <= 0 ||
           size_k % bl != 0 || size_m % topk != 0;
}

static inline int pad512(int k) { return (k + 511) / 512 * 512; }

// f32 rows a workgroup can quantize while it stages them (what lk_mmvq_fused asks of its input): a
// pair's row is a few KB, so reading it as floats costs less than a quantizer launch ahead of the
// kernel and the scratch round trip between the two.
static inline bool rows_stage_as_f32(const float* inputs, int size_k, int quant_type) {
    if (lk_moe_wire_block_len_legacy(quant_type) != 0) return false;   // those kernels read Q8_1 rows
    return ((uintptr_t)inputs & 15) == 0 && size_k % 4 == 0 && size_k <= 8192;
}

}  // namespace

void lk_mmq_q4k_wide_release(int device);   // mmq_q4k_wide.hip: the token-side operand buffers of the wide Q4_K tiles

extern "C" void loken_stream_scratch_release() {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return;
    (void)hipDeviceSynchronize();   // queued kernels may still read what is freed below
    lk_mmq_q4k_wide_release(dev);
    std::lock_guard<std::mutex> lock(g_scratch_mu);
    for (auto it = g_scratch.begin(); it != g_scratch.end();) {
        if (it->device != dev) { ++it; continue; }
        if (it->ptr) (void)hipFree(it->ptr);
        for (void* p : it->kept) (void)hipFree(p);
        it = g_scratch.erase(it);
    }
}

extern "C" void loken_moe_sum_topk(const float* pairs, float* outputs, int tokens, int topk, int cols, void* stream) {
    if (tokens <= 0 || cols <= 0) return;
    const size_t total = (size_t)tokens * cols;
    hipLaunchKernelGGL(sum_topk_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, (hipStream_t)stream, pairs,
                       (const float*)nullptr, outputs, tokens, topk, cols);
    (void)hipGetLastError();
}

extern "C" int loken_moe_gemm_gguf(const float* inputs, const void* weights, const int32_t* sorted_token_ids,
                                   const int32_t* expert_ids, const float* topk_weights, void* outputs,
                                   int num_experts, int topk, int size_m, int size_n, int size_k, int quant_type,
                                   void* stream) {
    if (block_len_of_wire(quant_type) == 0) return LK_ERR_TYPE;
    if (size_m == 0) return LK_OK;
    if (!inputs || !weights || !sorted_token_ids || !expert_ids || !outputs ||
        bad_shape(quant_type, num_experts, topk, size_m, size_n, size_k)) return LK_ERR_ARG;
    hipStream_t s = (hipStream_t)stream;
    const int kp = pad512(size_k);
    // with routing weights every entry has its own activation row; without, topk entries share one
    const int act_rows = topk_weights ? size_m : size_m / topk;
    if (rows_stage_as_f32(inputs, size_k, quant_type)) {
        MoeDims d{num_experts, topk, size_m, size_n, 0, kp / 32, 0, size_k};
        return launch_format<MODE_PLAIN>(quant_type, (const uint8_t*)weights, nullptr, (const uint8_t*)inputs,
                                         sorted_token_ids, expert_ids, topk_weights, nullptr, (float*)outputs, d, size_k, s);
    }
    std::lock_guard<std::mutex> lock(g_scratch_mu);
    uint8_t* acts = (uint8_t*)reserve_scratch((size_t)act_rows * (kp / 32) * Q81_BYTES, s);
    if (!acts) return LK_ERR_NOMEM;
    if (int rc = lk_quantize_q8_1(inputs, LK_TYPE_F32, acts, size_k, kp, act_rows, stream)) return rc;
    MoeDims d{num_experts, topk, size_m, size_n, 0, kp / 32, 0};
    return launch_format<MODE_PLAIN>(quant_type, (const uint8_t*)weights, nullptr, acts, sorted_token_ids, expert_ids,
                                     topk_weights, nullptr, (float*)outputs, d, size_k, s);
}

// The prefill form of the launch above (declared src/inference/moe_cuda/mod.rs:478-483; called from
// moe_gemm_gguf whenever the card has matrix instructions, src/inference/moe_cuda/gemm.rs:221-258;
// the reference's body for AMD cards: cuda/moe/moe_wmma_amd.cu:311-339): the activation rows arrive
// at the model's own width (input_dtype 0 = f16, 1 = bf16), everything else as loken_moe_gemm_gguf.
// The rows are quantized to Q8_1 from that width (the value an f16 / bf16 holds is exact in f32, so
// the codes are those lk_quantize_q8_1 gives the same values as f32) and run through the same
// per-pair kernels: same integers, same combine, same row conventions. The reference's kernel
// dequantizes the weights to the activation's width instead and multiplies on bf16 fragments; both
// approximate the f32 product of the dequantized operands, this one to the decode path's bound.
extern "C" int loken_moe_gemm_gguf_prefill(const void* inputs, const uint8_t* weights, const int32_t* sorted_token_ids,
                                           const int32_t* expert_ids, const float* topk_weights, void* outputs,
                                           int num_experts, int topk, int size_m, int size_n, int size_k,
                                           int input_dtype, int quant_type, void* stream) {
    if (block_len_of_wire(quant_type) == 0) return LK_ERR_TYPE;
    if (input_dtype != 0 && input_dtype != 1) return LK_ERR_TYPE;
    if (size_m == 0) return LK_OK;
    if (!inputs || !weights || !sorted_token_ids || !expert_ids || !outputs ||
        bad_shape(quant_type, num_experts, topk, size_m, size_n, size_k)) return LK_ERR_ARG;
    hipStream_t s = (hipStream_t)stream;
    const int kp = pad512(size_k);
    const int act_rows = topk_weights ? size_m : size_m / topk;
    std::lock_guard<std::mutex> lock(g_scratch_mu);
    uint8_t* acts = (uint8_t*)reserve_scratch((size_t)act_rows * (kp / 32) * Q81_BYTES, s);
    if (!acts) return LK_ERR_NOMEM;
    if (int rc = lk_quantize_q8_1(inputs, input_dtype == 0 ? LK_TYPE_F16 : LK_TYPE_BF16, acts, size_k, kp, act_rows, stream))
        return rc;
    MoeDims d{num_experts, topk, size_m, size_n, 0, kp / 32, 0};
    return launch_format<MODE_PLAIN>(quant_type, weights, nullptr, acts, sorted_token_ids, expert_ids, topk_weights, nullptr,
                                     (float*)outputs, d, size_k, s);
}

// The gated launch: act(gate . x, up . x) per routed pair. `slab_rows` = weight rows per expert in
// both stacks (size_n, or 2 size_n when `up_weights` points size_n rows into the gate's tensor).
static int gate_up_impl(const float* inputs, const void* gate_weights, const void* up_weights,
                        const int32_t* sorted_token_ids, const int32_t* expert_ids, float* outputs, int num_experts,
                        int topk, int size_m, int size_n, int size_k, int quant_type, const LkGateAct& act,
                        int slab_rows, void* stream, const unsigned int* live = nullptr, const LkMoeAlt& alt = LkMoeAlt{}) {
    if (block_len_of_wire(quant_type) == 0) return LK_ERR_TYPE;
    if (size_m == 0) return LK_OK;
    if (!inputs || !gate_weights || !up_weights || !sorted_token_ids || !expert_ids || !outputs ||
        bad_shape(quant_type, num_experts, topk, size_m, size_n, size_k)) return LK_ERR_ARG;
    hipStream_t s = (hipStream_t)stream;
    const int kp = pad512(size_k), act_rows = size_m / topk;
    // Q4_K rows of at most 16 super-blocks: the engine that keeps the activation's codes in registers
    if (quant_type == 1 && !live && !alt.alt0 && !alt.alt1 && !alt.alt_at && rows_stage_as_f32(inputs, size_k, quant_type)) {
        const int nb = size_k / 256;
        const int rc = lk_q4k_reg_moe_pair((const uint8_t*)gate_weights, (const uint8_t*)up_weights, inputs, sorted_token_ids,
                                           expert_ids, outputs, num_experts, topk, size_m, size_n, nb,
                                           (int64_t)(slab_rows ? slab_rows : size_n) * nb * Q4K_BYTES, act, s);
        if (rc >= 0) return rc;
    }
    if (rows_stage_as_f32(inputs, size_k, quant_type)) {
        MoeDims d{num_experts, topk, size_m, size_n, 0, kp / 32, 0, size_k, slab_rows, act, live, alt};
        return launch_format<MODE_GATED>(quant_type, (const uint8_t*)gate_weights, (const uint8_t*)up_weights,
                                         (const uint8_t*)inputs, sorted_token_ids, expert_ids, nullptr, nullptr, outputs,
                                         d, size_k, s);
    }
    std::lock_guard<std::mutex> lock(g_scratch_mu);
    uint8_t* acts = (uint8_t*)reserve_scratch((size_t)act_rows * (kp / 32) * Q81_BYTES, s);
    if (!acts) return LK_ERR_NOMEM;
    if (int rc = lk_quantize_q8_1(inputs, LK_TYPE_F32, acts, size_k, kp, act_rows, stream)) return rc;
    MoeDims d{num_experts, topk, size_m, size_n, 0, kp / 32, 0, 0, slab_rows, act, live, alt};
    return launch_format<MODE_GATED>(quant_type, (const uint8_t*)gate_weights, (const uint8_t*)up_weights, acts,
                                     sorted_token_ids, expert_ids, nullptr, nullptr, outputs, d, size_k, s);
}

extern "C" int loken_moe_gemm_gguf_gate_up_silu_mul(const float* inputs, const void* gate_weights,
                                                    const void* up_weights, const int32_t* sorted_token_ids,
                                                    const int32_t* expert_ids, float* outputs, int num_experts,
                                                    int topk, int size_m, int size_n, int size_k, int quant_type,
                                                    void* stream) {
    return gate_up_impl(inputs, gate_weights, up_weights, sorted_token_ids, expert_ids, outputs, num_experts, topk,
                        size_m, size_n, size_k, quant_type, LkGateAct{}, 0, stream);
}

extern "C" int loken_moe_gemm_gguf_gate_up_silu_mul_live(const float* inputs, const void* gate_weights,
                                                         const void* up_weights, const int32_t* sorted_token_ids,
                                                         const int32_t* expert_ids, float* outputs, int num_experts,
                                                         int topk, int size_m, int size_n, int size_k, int quant_type,
                                                         const unsigned int* live, void* stream) {
    return gate_up_impl(inputs, gate_weights, up_weights, sorted_token_ids, expert_ids, outputs, num_experts, topk,
                        size_m, size_n, size_k, quant_type, LkGateAct{}, 0, stream, live);
}

extern "C" int loken_moe_gemm_gguf_gate_up_silu_mul_two(const float* inputs, const void* gate_weights,
                                                        const void* up_weights, const void* alt_gate,
                                                        const void* alt_up, int alt_from, const void* const* alt_at,
                                                        const int32_t* sorted_token_ids, const int32_t* expert_ids,
                                                        float* outputs, int num_experts, int topk, int size_m,
                                                        int size_n, int size_k, int quant_type, void* stream) {
    LkMoeAlt alt;
    alt.alt0 = (const uint8_t*)alt_gate; alt.alt1 = (const uint8_t*)alt_up; alt.alt_from = alt_from; alt.alt_at = alt_at;
    return gate_up_impl(inputs, gate_weights, up_weights, sorted_token_ids, expert_ids, outputs, num_experts, topk,
                        size_m, size_n, size_k, quant_type, LkGateAct{}, 0, stream, nullptr, alt);
}

extern "C" int loken_moe_gemm_gguf_gate_up_swiglu_oai(const float* inputs, const void* gate_weights,
                                                      const void* up_weights, const int32_t* sorted_token_ids,
                                                      const int32_t* expert_ids, const float* gate_bias,
                                                      const float* up_bias, float* outputs, int num_experts, int topk,
                                                      int size_m, int size_n, int size_k, int quant_type, float alpha,
                                                      float limit, void* stream) {
    LkGateAct act;
    act.kind = LK_GATE_OAI; act.alpha = alpha; act.limit = limit; act.gate_bias = gate_bias; act.up_bias = up_bias;
    return gate_up_impl(inputs, gate_weights, up_weights, sorted_token_ids, expert_ids, outputs, num_experts, topk,
                        size_m, size_n, size_k, quant_type, act, 0, stream);
}

extern "C" int loken_moe_gemm_gguf_gate_up_swiglu_limited(const float* inputs, const void* gate_weights,
                                                          const void* up_weights, const int32_t* sorted_token_ids,
                                                          const int32_t* expert_ids, float* outputs, int num_experts,
                                                          int topk, int size_m, int size_n, int size_k, int quant_type,
                                                          float limit, void* stream) {
    LkGateAct act;
    act.kind = LK_GATE_LIMITED; act.limit = limit;
    return gate_up_impl(inputs, gate_weights, up_weights, sorted_token_ids, expert_ids, outputs, num_experts, topk,
                        size_m, size_n, size_k, quant_type, act, 0, stream);
}

extern "C" int loken_moe_gemm_gguf_gate_up_gelu_mul_concat(const float* inputs, const void* gate_up_weights,
                                                           const int32_t* sorted_token_ids, const int32_t* expert_ids,
                                                           float* outputs, int num_experts, int topk, int size_m,
                                                           int size_n, int size_k, int quant_type, void* stream) {
    const int bl = block_len_of_wire(quant_type);
    if (bl == 0) return LK_ERR_TYPE;
    if (!gate_up_weights || size_n <= 0 || size_k <= 0 || size_k % bl != 0) return size_m == 0 ? LK_OK : LK_ERR_ARG;
    // an expert's slab holds the gate's size_n rows, then the up's
    // block bytes by wire id: Q8_0, Q4_K, Q2_K, Q3_K, Q5_K, Q6_K, Q5_0, MXFP4, Q5_1, IQ4_NL, IQ4_XS, IQ3_XXS, IQ3_S,
    // IQ2_S, Q2_0, IQ2_XXS
    static const int bytes_of_wire[] = {34, 144, 84, 110, 176, 210, 22, 17, 24, 18, 136, 98, 110, 82, 18, 66};
    const int64_t row_bytes = (int64_t)(size_k / bl) * bytes_of_wire[quant_type];
    const uint8_t* up = (const uint8_t*)gate_up_weights + (int64_t)size_n * row_bytes;
    LkGateAct act;
    act.kind = LK_GATE_GELU;
    return gate_up_impl(inputs, gate_up_weights, up, sorted_token_ids, expert_ids, outputs, num_experts, topk, size_m,
                        size_n, size_k, quant_type, act, 2 * size_n, stream);
}

__global__ void zero_f32_kernel(float* __restrict__ p, size_t n) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0.f;
}

// Down per routed pair, then the fold over a token's pairs; with `pair_rows` the weighted rows go to
// the caller's [size_m, size_n] buffer and the sum is the caller's (cuda/moe/moe_gguf.cu:755-820).
static int down_impl(const float* inputs, const void* weights, const int32_t* sorted_token_ids,
                     const int32_t* expert_ids, const float* topk_weights, float* outputs, int num_experts, int topk,
                     int size_m, int size_n, int size_k, int gguf_dtype, const float* down_bias,
                     const float* add_after, const unsigned int* live, float* pair_rows, void* stream,
                     const LkMoeAlt& alt = LkMoeAlt{}, bool from_static = false) {
    if (block_len_of_wire(gguf_dtype) == 0) return LK_ERR_TYPE;
    if (size_m == 0) return LK_OK;
    if (!inputs || !weights || !sorted_token_ids || !expert_ids || !topk_weights || (!outputs && !pair_rows) ||
        bad_shape(gguf_dtype, num_experts, topk, size_m, size_n, size_k)) return LK_ERR_ARG;
    hipStream_t s = (hipStream_t)stream;
    // a handful of tokens over short K-quant rows: one launch that needs no pair rows at all (the entry
    // point that allocates nothing keeps the two launches over its fixed array)
    if (!from_static && !live && !pair_rows && !alt.alt0 && !alt.alt_at) {
        const int rc = lk_moe_down_fold(gguf_dtype, inputs, weights, sorted_token_ids, expert_ids, topk_weights, outputs,
                                        num_experts, topk, size_m, size_n, size_k, down_bias, add_after, s);
        if (rc >= 0) return rc;
    }
    const int kp = pad512(size_k);
    const bool as_f32 = rows_stage_as_f32(inputs, size_k, gguf_dtype);
    const size_t act_bytes = as_f32 ? 0 : (((size_t)size_m * (kp / 32) * Q81_BYTES) + 255) & ~(size_t)255;
    const size_t pair_bytes = pair_rows ? 0 : (size_t)size_m * size_n * sizeof(float);
    std::lock_guard<std::mutex> lock(g_scratch_mu);
    uint8_t* base = nullptr;
    if (from_static) {
        // nothing is allocated: the device's fixed array, or an error when the call does not fit it
        if (act_bytes + pair_bytes > STATIC_SCRATCH_BYTES) return LK_ERR_SIZE;
        base = static_scratch();
        if (!base) return LK_ERR_LAUNCH;
    } else if (act_bytes + pair_bytes) {
        base = (uint8_t*)reserve_scratch(act_bytes + pair_bytes, s);
        if (!base) return LK_ERR_NOMEM;
    }
    float* pairs = pair_rows ? pair_rows : (float*)(base + act_bytes);
    // (The fixed array keeps the last call's rows. Nothing is cleared: sorted_token_ids names every slot once,
    // as the allocating path and the reference assume (cuda/moe/moe_gguf.cu:785-786), and the kernels write
    // every named slot's row, zeros for a pair whose expert is out of range.)
    if (!as_f32)
        if (int rc = lk_quantize_q8_1(inputs, LK_TYPE_F32, base, size_k, kp, size_m, stream)) return rc;
    if (live) {
        // the pairs past the count leave their rows to the sum: zero (a fill kernel, so that a
        // caller may capture the launch)
        const size_t n = (size_t)size_m * size_n;
        hipLaunchKernelGGL(zero_f32_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, pairs, n);
    }
    MoeDims d{num_experts, topk, size_m, size_n, 0, kp / 32, 0, as_f32 ? size_k : 0, 0, LkGateAct{}, live, alt};
    if (int rc = launch_format<MODE_DOWN>(gguf_dtype, (const uint8_t*)weights, nullptr,
                                          as_f32 ? (const uint8_t*)inputs : base, sorted_token_ids,
                                          expert_ids, topk_weights, down_bias, pairs, d, size_k, s)) return rc;
    if (pair_rows) return lk_launch_status();
    const int tokens = size_m / topk;
    const size_t total = (size_t)tokens * size_n;
    hipLaunchKernelGGL(sum_topk_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, (const float*)pairs,
                       add_after, outputs, tokens, topk, size_n);
    return lk_launch_status();
}

extern "C" int loken_moe_gemm_gguf_down_reduce(const float* inputs, const void* weights,
                                               const int32_t* sorted_token_ids, const int32_t* expert_ids,
                                               const float* topk_weights, float* outputs, int num_experts, int topk,
                                               int size_m, int size_n, int size_k, int gguf_dtype,
                                               const float* down_bias, const float* add_after, void* stream) {
    return down_impl(inputs, weights, sorted_token_ids, expert_ids, topk_weights, outputs, num_experts, topk, size_m,
                     size_n, size_k, gguf_dtype, down_bias, add_after, nullptr, nullptr, stream);
}

extern "C" int loken_moe_gemm_gguf_down_reduce_static(const float* inputs, const void* weights,
                                                      const int32_t* sorted_token_ids, const int32_t* expert_ids,
                                                      const float* topk_weights, float* outputs, int num_experts,
                                                      int topk, int size_m, int size_n, int size_k, int gguf_dtype,
                                                      const float* down_bias, const float* add_after, void* stream) {
    return down_impl(inputs, weights, sorted_token_ids, expert_ids, topk_weights, outputs, num_experts, topk, size_m,
                     size_n, size_k, gguf_dtype, down_bias, add_after, nullptr, nullptr, stream, LkMoeAlt{}, true);
}

extern "C" int loken_moe_gemm_gguf_down_pairs_live(const float* inputs, const void* weights,
                                                   const int32_t* sorted_token_ids, const int32_t* expert_ids,
                                                   const float* topk_weights, float* pair_rows, int num_experts,
                                                   int topk, int size_m, int size_n, int size_k, int quant_type,
                                                   const unsigned int* live, void* stream) {
    if (!pair_rows) return size_m == 0 ? LK_OK : LK_ERR_ARG;
    return down_impl(inputs, weights, sorted_token_ids, expert_ids, topk_weights, nullptr, num_experts, topk, size_m,
                     size_n, size_k, quant_type, nullptr, nullptr, live, pair_rows, stream);
}

extern "C" int loken_moe_gemm_gguf_down_reduce_two(const float* inputs, const void* weights, const void* alt_weights,
                                                   int alt_from, const int32_t* sorted_token_ids,
                                                   const int32_t* expert_ids, const float* topk_weights, float* outputs,
                                                   int num_experts, int topk, int size_m, int size_n, int size_k,
                                                   int quant_type, const float* down_bias, const float* add_after,
                                                   void* stream) {
    LkMoeAlt alt;
    alt.alt0 = (const uint8_t*)alt_weights; alt.alt_from = alt_from;
    return down_impl(inputs, weights, sorted_token_ids, expert_ids, topk_weights, outputs, num_experts, topk, size_m,
                     size_n, size_k, quant_type, down_bias, add_after, nullptr, nullptr, stream, alt);
}

extern "C" int loken_moe_gemm_gguf_down_pairs_two(const float* inputs, const void* weights, const void* alt_weights,
                                                  int alt_from, const void* const* alt_at,
                                                  const int32_t* sorted_token_ids, const int32_t* expert_ids,
                                                  const float* topk_weights, float* pair_rows, int num_experts,
                                                  int topk, int size_m, int size_n, int size_k, int quant_type,
                                                  void* stream) {
    if (!pair_rows) return size_m == 0 ? LK_OK : LK_ERR_ARG;
    LkMoeAlt alt;
    alt.alt0 = (const uint8_t*)alt_weights; alt.alt_from = alt_from; alt.alt_at = alt_at;
    return down_impl(inputs, weights, sorted_token_ids, expert_ids, topk_weights, nullptr, num_experts, topk, size_m,
                     size_n, size_k, quant_type, nullptr, nullptr, nullptr, pair_rows, stream, alt);
}

// ---------------------------------------------------------------- Q4_K expert rows over the caller's Q8_1
// The reference's matrix-unit pair kernels for a handful of rows per expert
// (loken_moe_q4k_imma_m8_gate_up, cuda/moe/moe_q4k_imma_m8.cu:312-335; loken_moe_q4k_imma_m8_down,
// cuda/moe/moe_q4k_imma_m8_down.cu:238-276; declared src/inference/moe_cuda/mod.rs:443-451). Their
// contract differs from the launchers above in three ways: the activation arrives as plain block_q8_1
// rows (size_k / 32 blocks apart, no padding), `expert_ids` holds one expert per routed pair, and the
// gate's rows and the up's share one tensor per expert, closed with the tanh-form GELU. At the loads
// these calls are made for, a pair's rows are a mat-vec: they run on the per-pair kernels above.
// (A tile of eight pairs that spans more than four experts loses rows in the reference; here every
// pair with an expert in range gets its row.)
extern "C" int lk_moe_q4k_rows_gate_up(const void* gate_up_weights, const void* q8_1, const int32_t* sorted_token_ids,
                                       const int32_t* expert_ids, float* output, int num_experts, int topk, int size_m,
                                       int size_n, int size_k, void* stream) {
    if (size_m == 0) return LK_OK;
    if (!gate_up_weights || !q8_1 || !sorted_token_ids || !expert_ids || !output ||
        bad_shape(1, num_experts, topk, size_m, size_n, size_k) || (((uintptr_t)q8_1) & 3) != 0) return LK_ERR_ARG;
    const uint8_t* gate = (const uint8_t*)gate_up_weights;
    const uint8_t* up = gate + (int64_t)size_n * (size_k / 256) * Q4K_BYTES;
    LkGateAct act;
    act.kind = LK_GATE_GELU;
    MoeDims d{num_experts, topk, size_m, size_n, 0, size_k / 32, 0, 0, 2 * size_n, act, nullptr, LkMoeAlt{}};
    return launch_format<MODE_GATED>(1, gate, up, (const uint8_t*)q8_1, sorted_token_ids, expert_ids, nullptr, nullptr,
                                     output, d, size_k, (hipStream_t)stream);
}

extern "C" void loken_moe_q4k_imma_m8_gate_up(const void* gate_up_weights, const void* q8_1,
                                              const int32_t* sorted_token_ids, const int32_t* expert_ids, float* output,
                                              int num_experts, int topk, int size_m, int size_n, int size_k,
                                              void* stream) {
    (void)lk_moe_q4k_rows_gate_up(gate_up_weights, q8_1, sorted_token_ids, expert_ids, output, num_experts, topk, size_m,
                                  size_n, size_k, stream);
}

// One Q8_1 row per routed pair (at the pair's slot); pair rows weighted by topk_weights[slot], then
// added into output[token] in slot order.
extern "C" int loken_moe_q4k_imma_m8_down(const void* weights, const void* q8_1, const int32_t* sorted_token_ids,
                                          const int32_t* expert_ids, const float* topk_weights, float* output,
                                          int num_experts, int topk, int size_m, int hidden, int size_k, void* stream) {
    if (size_m <= 0 || hidden <= 0 || size_k <= 0) return LK_OK;
    if (!weights || !q8_1 || !sorted_token_ids || !expert_ids || !topk_weights || !output ||
        bad_shape(1, num_experts, topk, size_m, hidden, size_k) || (((uintptr_t)q8_1) & 3) != 0) return LK_ERR_ARG;
    hipStream_t s = (hipStream_t)stream;
    std::lock_guard<std::mutex> lock(g_scratch_mu);
    float* pairs = (float*)reserve_scratch((size_t)size_m * hidden * sizeof(float), s);
    if (!pairs) return LK_ERR_NOMEM;
    // a pair whose slot is out of range writes nothing: its row of the sum must read zero
    const size_t n = (size_t)size_m * hidden;
    hipLaunchKernelGGL(zero_f32_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, pairs, n);
    MoeDims d{num_experts, topk, size_m, hidden, 0, size_k / 32, 0, 0, 0, LkGateAct{}, nullptr, LkMoeAlt{}};
    if (int rc = launch_format<MODE_DOWN>(1, (const uint8_t*)weights, nullptr, (const uint8_t*)q8_1, sorted_token_ids,
                                          expert_ids, topk_weights, nullptr, pairs, d, size_k, s)) return rc;
    loken_moe_sum_topk(pairs, output, size_m / topk, topk, hidden, stream);
    return lk_launch_status();
}
