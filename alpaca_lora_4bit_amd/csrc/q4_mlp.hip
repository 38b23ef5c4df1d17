// Decode step of a gated MLP block in ONE launch:   y[M,H] = down( silu(gate(x)) * up(x) ),   1 <= M <= 16,
// gate / up: H -> I, down: I -> H, all three 4-bit layers with sequential groups.  This is what
// QuantLlamaMLP.forward of the reference computes with three (fused: two) products and two elementwise kernels
// (src/alpaca_lora_4bit/model_attn_mlp_patch.py:165-228).
//
// Why one launch.  A weight-streaming product of this size is over in 7-12 us, of which about 1.7 us is the gap
// between two dependent launches and 2-3 us the ramp and the reduction tail, during which HBM idles.  Here the
// workgroups of the down projection are part of the same grid as those of gate and up: they request their packed
// weights as soon as they start -- the weights do not depend on the activations -- and only then wait for the
// part of silu(gate) * up they need, so the stream from HBM never stops between the two products.
//
// Grid (1-D).  Workgroups [0, wgs_phase1) compute gate and up exactly like q4::gemv_seq_kernel (64-column strips,
// K split over `splits_gu` workgroups, 64-bit fixed-point atomics); strip i of gate and strip i of up sit next to
// each other, low strips first.  Workgroups from wgs_phase1 on compute down: workgroup (j, s) takes the rows
// [j*span, (j+1)*span) of the reduction (span = 8 wavefronts x 128) for output strip s, ordered j-major, so the
// first of them need only the first strips of gate and up.
//
// Hand-over.  The workgroup that completes an element of gate or up publishes it as ONE 32-bit word: fp16 bits in
// the low half, the launch's 16-bit tag in the high half (device-scope atomic store).  A consumer loads the words of
// its rows (device-scope atomic loads) and accepts them when every tag equals the launch's tag; otherwise it sleeps
// and reads again.  Value and flag are one atomic object, so no fence or ordering between different addresses is
// needed.  The tag comes from 64-bit tickets in the workspace, 256 of them, 128 bytes apart (one address would
// serialise a few thousand device-scope accesses in one memory channel: measured 140 us per launch).  Workgroup w uses
// ticket w % 256.  Every launch advances every ticket that has a workgroup by exactly 2^20: the first workgroup of
// a class adds 2^20 - (workgroups of the class - 1), every other one adds 1, each when it ends and without waiting
// for the result.  One thread per workgroup reads the ticket; that workgroup's own addition is still outstanding
// then, so less than 2^20 of this launch's share has been added and ticket >> 20 is the number of launches before
// this one, the same for every workgroup.  Words of earlier launches carry older tags, and the words a launch reads
// are all rewritten by that launch, provided the workspace serves one (M, H, I) shape.
//
// Forward progress.  Consumers wait only for producers with lower workgroup ids, which never wait; workgroups are
// started in id order on every XCD.  Every wait is bounded all the same: after `poll_limit` rounds a wavefront
// records the fact in `status` and goes on with what it has, so the grid always drains.
#include "q4_gemv_core.hpp"
#include "q4_gptq.h"

namespace q4 {

constexpr int kTicketShift = 20;
constexpr int kTickets = 256;
constexpr int kTicketStride = 16;          // in 64-bit words: 128 bytes

__device__ __forceinline__ unsigned long long* ticket_of(unsigned long long* base, int wg) {
    return base + (size_t)(wg & (kTickets - 1)) * kTicketStride;
}
__device__ __forceinline__ uint32_t tag_of(unsigned long long ticket) {
    return ((uint32_t)(ticket >> kTicketShift) + 1u) & 0xFFFFu;
}

struct MlpArgs {
    GemvArgs gate, up, down;              // gate.y / up.y may be null (the intermediate is not wanted)
    uint32_t* hand_gate;                  // [M, I] tagged words
    uint32_t* hand_up;
    unsigned long long* ticket;           // kTickets entries, kTicketStride apart
    uint32_t* status;
    int strips_gu, splits_gu;             // I / 64 strips of gate (and of up), K splits of each
    int strips_dn, splits_dn;             // H / 64 strips of down, splits of its reduction over I
    int wgs_phase1;                       // 2 * strips_gu * splits_gu
    int poll_limit;
};

__device__ __forceinline__ uint32_t load_word_agent(const uint32_t* p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// silu(g) * u with the roundings of the unfused modules: act_fn on an fp16 tensor evaluates in fp32 and rounds to
// fp16, the product with up is one more fp16 rounding.
__device__ __forceinline__ uint32_t silu_mul_bits(uint32_t g_word, uint32_t u_word) {
    const float g = (float)__builtin_bit_cast(half_t, (unsigned short)(g_word & 0xFFFFu));
    const float u = (float)__builtin_bit_cast(half_t, (unsigned short)(u_word & 0xFFFFu));
    const half_t h = (half_t)(g / (1.0f + __expf(-g)));
    const half_t r = (half_t)((float)h * u);
    return (uint32_t)__builtin_bit_cast(unsigned short, r);
}

template <int NSTEP, int GSTEPS>
__device__ __forceinline__ void mlp_gate_up_body(const MlpArgs& a, int wg, uint32_t* tag_lds) {
    const int unit = wg / a.splits_gu;                    // uniform
    const int split = wg - unit * a.splits_gu;
    const bool is_up = unit & 1;
    const GemvArgs& l = is_up ? a.up : a.gate;
    uint32_t* hand = is_up ? a.hand_up : a.hand_gate;
    const int n0 = (unit >> 1) * kColsPerWave;

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int nwaves = blockDim.x >> 6;
    const int kk = lane >> 4, c = lane & 15;
    const int k0 = (split * nwaves + wave) * (32 * NSTEP);

    float4_t yacc[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) yacc[j] = float4_t{0.f, 0.f, 0.f, 0.f};

    unsigned long long ticket = 0;
    if (k0 < l.K) {
        SeqChunk<NSTEP, GSTEPS> ch;
        ch.load_x(l.x + (size_t)min(c, l.M - 1) * l.K + k0 + 8 * kk);
        ch.load_weights(l, k0, n0 + 4 * c, kk);
        // behind the weights: it is needed last, and loads return in issue order
        if (threadIdx.x == 0) ticket = __hip_atomic_load(ticket_of(a.ticket, wg), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __builtin_amdgcn_sched_barrier(0);
        ch.multiply(l, yacc, c);
    } else if (threadIdx.x == 0) {
        ticket = __hip_atomic_load(ticket_of(a.ticket, wg), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    if (threadIdx.x == 0) *tag_lds = tag_of(ticket);      // read by everyone behind the barrier of gemv_finish
    gemv_finish(l, yacc, n0, wave, nwaves, kk, c, a.splits_gu, hand, tag_lds);
}

template <int NSTEP, int GSTEPS>
__device__ __forceinline__ void mlp_down_body(const MlpArgs& a, int wg, int wg2, uint32_t* tag_lds) {
    static_assert(NSTEP == 4, "the staging tile of a wavefront is its own [M][64] fp32 part of the reduction buffer");
    extern __shared__ float red[];
    constexpr int CH = 32 * NSTEP;                        // reduction rows per wavefront
    const GemvArgs& d = a.down;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int nwaves = blockDim.x >> 6;
    const int kk = lane >> 4, c = lane & 15;
    const int j = wg2 / a.strips_dn;                      // uniform: which span of the reduction
    const int n0 = (wg2 - j * a.strips_dn) * kColsPerWave;
    const int k0 = (j * nwaves + wave) * CH;
    const bool live = k0 < d.K;                           // wave-uniform; K % CH == 0 (checked on the host)
    const int M = d.M;

    float4_t yacc[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) yacc[i] = float4_t{0.f, 0.f, 0.f, 0.f};

    // the packed weights first: they do not depend on gate and up, so they stream while those are being finished
    SeqChunk<NSTEP, GSTEPS> ch;
    ch.load_weights_branch_free(d, k0, n0 + 4 * c, kk, live);
    // the hand-over words of the first four rows right behind the weights: when they were published long ago (the
    // usual case) the look costs no round trip of its own.  Lane l takes columns k0 + 2l, k0 + 2l + 1 of a row: 512
    // contiguous bytes per wavefront, row and matrix.
    constexpr int RB = 4;                                 // rows per batch of loads (one latency per batch, not per row)
    const int kw = (live ? k0 : 0) + 2 * lane;
    uint32_t hw[RB][4] = {};
    auto load_batch = [&](int m0) {
#pragma unroll
        for (int r = 0; r < RB; ++r) {
            if (m0 + r < M) {                                                     // uniform
                const size_t at = (size_t)(m0 + r) * d.K + kw;
                hw[r][0] = load_word_agent(a.hand_gate + at); hw[r][1] = load_word_agent(a.hand_gate + at + 1);
                hw[r][2] = load_word_agent(a.hand_up + at); hw[r][3] = load_word_agent(a.hand_up + at + 1);
            }
        }
    };
    load_batch(0);
    if (threadIdx.x == 0)
        *tag_lds = tag_of(__hip_atomic_load(ticket_of(a.ticket, wg), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
    __builtin_amdgcn_sched_barrier(0);
    __syncthreads();
    const uint32_t tag = *tag_lds;

    // this wavefront's [M][64] fp32 part of the reduction buffer doubles as its [M][CH] fp16 activation tile
    uint32_t* tile = reinterpret_cast<uint32_t*>(red + ((wave * M) << 6));
    if (live) {
        int polls = 0;
        for (int m0 = 0; m0 < M; m0 += RB) {
            bool have = m0 == 0;
            for (;;) {
                if (!have) load_batch(m0);
                have = false;
                bool stale = false;
#pragma unroll
                for (int r = 0; r < RB; ++r)
                    if (m0 + r < M)
                        stale |= ((hw[r][0] >> 16) != tag) | ((hw[r][1] >> 16) != tag) | ((hw[r][2] >> 16) != tag) | ((hw[r][3] >> 16) != tag);
                if (__builtin_amdgcn_ballot_w64(stale) == 0) break;              // wave-uniform
                if (++polls > a.poll_limit) {
                    if (lane == 0) __hip_atomic_store(a.status, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    break;
                }
                __builtin_amdgcn_s_sleep(4);             // measured: 4 to 16 units and a delayed first look all time the same
            }
#pragma unroll
            for (int r = 0; r < RB; ++r)
                if (m0 + r < M)
                    tile[(m0 + r) * (CH / 2) + lane] = silu_mul_bits(hw[r][0], hw[r][2]) | (silu_mul_bits(hw[r][1], hw[r][3]) << 16);
        }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    if (live) {
        const half_t* row = reinterpret_cast<const half_t*>(tile) + min(c, M - 1) * CH + 8 * kk;
#pragma unroll
        for (int t = 0; t < NSTEP; ++t) ch.xv[t] = *reinterpret_cast<const uint4_t*>(row + 32 * t);
        __builtin_amdgcn_sched_barrier(0);
        ch.multiply(d, yacc, c);
    }
    // the tile reads above precede, in this wavefront's program order, the partial sums it now writes over them
    gemv_finish(d, yacc, n0, wave, nwaves, kk, c, a.splits_dn);
}

template <int NSTEP, int GSTEPS>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(8, 8))) void mlp_decode_kernel(MlpArgs a) {
    __shared__ uint32_t tag_lds;
    const int wg = blockIdx.x;
    if (wg < a.wgs_phase1) mlp_gate_up_body<NSTEP, GSTEPS>(a, wg, &tag_lds);
    else mlp_down_body<NSTEP, GSTEPS>(a, wg, wg - a.wgs_phase1, &tag_lds);
    // the tickets: 2^20 per launch for every class of workgroups, whatever the grid
    if (threadIdx.x == 0) {
        const int in_class = ((int)gridDim.x - (wg & (kTickets - 1)) + kTickets - 1) / kTickets;
        const unsigned long long inc = wg < kTickets ? (1ull << kTicketShift) - (unsigned long long)(in_class - 1) : 1ull;
        __hip_atomic_fetch_add(ticket_of(a.ticket, wg), inc, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

struct MlpLayout {
    size_t acc_gate, acc_up, acc_down, hand_gate, hand_up, ticket, status, total;
};
static MlpLayout mlp_layout(int M, int H, int I) {
    MlpLayout o;
    size_t at = 0;
    o.acc_gate = at; at += (size_t)M * I * 8;
    o.acc_up = at; at += (size_t)M * I * 8;
    o.acc_down = at; at += (size_t)M * H * 8;
    o.hand_gate = at; at += (size_t)M * I * 4;
    o.hand_up = at; at += (size_t)M * I * 4;
    at = (at + 127) & ~(size_t)127;
    o.ticket = at; at += (size_t)kTickets * kTicketStride * 8;
    o.status = at; at += 128;
    o.total = at;
    return o;
}

}  // namespace q4

extern "C" size_t q4_mlp_plan_workspace(int M, int H, int I) { return q4::mlp_layout(M, H, I).total; }

// Shapes the fused kernel takes: chunks of 128 reduction rows inside one quantization group, on both sides.
extern "C" int q4_mlp_applicable(int M, int H, int I, int groupsize) {
    return M >= 1 && M <= 16 && groupsize > 0 && groupsize % 128 == 0 && H % 128 == 0 && I % 128 == 0 && H >= 128 &&
           I >= 128 && (long)(2 * (I / 64) * ((H / 128 + 7) / 8) + (H / 64) * ((I / 128 + 7) / 8)) < (1l << q4::kTicketShift);
}

extern "C" int q4_launch_mlp(const void* x, const int32_t* const* qweight, const int32_t* const* qzeros,
                             const void* const* scales, int groupsize, void* gate_out, void* up_out, void* y, int M, int H,
                             int I, void* workspace, int poll_limit, hipStream_t stream) {
    using namespace q4;
    const MlpLayout lay = mlp_layout(M, H, I);
    char* ws = reinterpret_cast<char*>(workspace);
    MlpArgs a;
    void* outs[3] = {gate_out, up_out, y};
    const size_t accs[3] = {lay.acc_gate, lay.acc_up, lay.acc_down};
    GemvArgs* ls[3] = {&a.gate, &a.up, &a.down};
    for (int i = 0; i < 3; ++i) {
        GemvArgs& l = *ls[i];
        const int K = i < 2 ? H : I, N = i < 2 ? I : H;
        l.x = i < 2 ? reinterpret_cast<const half_t*>(x) : nullptr;
        l.qweight = reinterpret_cast<const uint32_t*>(qweight[i]);
        l.qzeros = reinterpret_cast<const uint32_t*>(qzeros[i]);
        l.scales = reinterpret_cast<const half_t*>(scales[i]);
        l.g_idx = nullptr;
        l.groupsize = groupsize;
        l.y = reinterpret_cast<half_t*>(outs[i]);
        l.accumulate = 0;
        l.M = M; l.K = K; l.N = N; l.G = (K + groupsize - 1) / groupsize;
        l.acc64 = reinterpret_cast<unsigned long long*>(ws + accs[i]);
        l.perm = nullptr;
        l.v1_zeros = nullptr;
    }
    a.hand_gate = reinterpret_cast<uint32_t*>(ws + lay.hand_gate);
    a.hand_up = reinterpret_cast<uint32_t*>(ws + lay.hand_up);
    a.ticket = reinterpret_cast<unsigned long long*>(ws + lay.ticket);
    a.status = reinterpret_cast<uint32_t*>(ws + lay.status);
    constexpr int kWaves = 8;
    a.strips_gu = I / kColsPerWave; a.splits_gu = (H / 128 + kWaves - 1) / kWaves;
    a.strips_dn = H / kColsPerWave; a.splits_dn = (I / 128 + kWaves - 1) / kWaves;
    if (a.splits_gu > 255 || a.splits_dn > 255) return -2;          // 8-bit arrival counter of the accumulators
    a.wgs_phase1 = 2 * a.strips_gu * a.splits_gu;
    a.poll_limit = poll_limit > 0 ? poll_limit : 200000;
    const dim3 grid(a.wgs_phase1 + a.strips_dn * a.splits_dn), block(64 * kWaves);
    const size_t lds = (size_t)kWaves * M * 64 * sizeof(float);
    hipLaunchKernelGGL((mlp_decode_kernel<4, 0>), grid, block, lds, stream, a);
    return hipGetLastError() == hipSuccess ? 0 : -4;
}

// status word of a workspace (device memory): the offset callers copy back to see whether a wait hit its limit
extern "C" size_t q4_mlp_status_offset(int M, int H, int I) { return q4::mlp_layout(M, H, I).status; }
