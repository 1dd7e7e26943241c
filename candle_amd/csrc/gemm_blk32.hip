// Prefill GEMM for the 32-element-block types (Q8_0 and Q4_0 weights, Q8_0 activations) on the int8
// MFMA: y[m, n] = x[m, k] . W[n, k]^T with the arithmetic of the reference's CPU matmul
// (k_quants.rs:1842-1883 with vec_dot :237-254 for Q4_0, :631-649 for Q8_0): per block the integer
// sum of 32 products, times the two block scales.  Replaces the reference's MMQ kernels for these
// types (candle-kernels/src/quantized.cu:436-544, launched from quantized/cuda.rs:298-365).
//
// A 32-element block is exactly one K-slice of v_mfma_i32_32x32x32_i8, so the integer of every
// (activation row, weight row, block) is one MFMA result element, I (Q4_0 nibbles go in as q - 8, so
// no correction term is left).  Its scale d8[row, block] * dw[col, block] is an outer product: a
// second MFMA lays it out in the accumulator layout (v_mfma_f32_32x32x16_bf16 with six non-zero K-slots:
// d8 goes in as three bf16 pieces and dw, an f16, as two, all exact, so the six products are the exact
// product whatever the magnitude of the activations - f16 pieces would lose d8 below 2^-14 - and the result is
// d8 * dw to f32 rounding; the f32 MFMA with one K-slot holds the matrix pipe twice as long), and the VALU
// work per element is one conversion and one fma.
//
// Work split as in the K-quant tile kernel (gemm.hip): a workgroup of eight waves covers 32*MT
// activation rows x 256 weight rows, a wave owns 32 weight rows; per 256-element step of K the
// activations (shared) and the wave's weight bytes go from global memory straight into LDS
// (buffer_load ... lds, 8 rows x 128 B per instruction, 16-byte chunks XOR-swizzled by the row),
// activations double buffered one step ahead.  With few workgroups K is split over blockIdx.z and
// the partial results are added atomically into a zeroed output.
#include "qhip_internal.h"

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef uint32_t v4u __attribute__((ext_vector_type(4)));
typedef void __attribute__((address_space(3))) *lptr_t;

constexpr int kWaves = 8;
constexpr int kThreads = kWaves * 64;

__device__ __forceinline__ __amdgpu_buffer_rsrc_t wave_rsrc(const void *base) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, -1, 0x00020000);
}
// lane l reads 16 bytes at base + off, they land at lds + 16*l (base and lds wave-uniform)
__device__ __forceinline__ void dma16(const void *base, uint32_t off, uint8_t *lds) {
    __builtin_amdgcn_raw_ptr_buffer_load_lds(wave_rsrc(base), (lptr_t)lds, 16, (int)off, 0, 0, 0);
}
// the same marked non-temporal: bytes that the launch reads once
__device__ __forceinline__ void dma16_once(const void *base, uint32_t off, uint8_t *lds) {
    __builtin_amdgcn_raw_ptr_buffer_load_lds(wave_rsrc(base), (lptr_t)lds, 16, (int)off, 0, 0, 2);
}

// LDS: two activation stages, then one weight buffer per wave.
//   act : [MT tiles][2 K-halves][4 row groups][8 rows][8 chunks of 16 B]   chunk c of row r sits at c ^ (r%8)
//   d8  : [32*MT rows][8 blocks] f32
//   wgt : per wave, Q8_0: [2 K-halves][4 row groups][8 rows][8 chunks]; Q4_0: [4 row groups][8 rows][8 chunks]
template <int DT, int MT> struct Tile {
    static constexpr int kAct = MT * 8 * 1024;
    static constexpr int kD8 = MT * 32 * 32;
    static constexpr int oD8 = kAct;
    static constexpr int kStage = kAct + kD8;
    static constexpr int kWgtWave = DT == CQ_DTYPE_Q8_0 ? 8192 : 4096;
    static constexpr int oWgt = 2 * kStage;
    static constexpr int kTotal = oWgt + kWaves * kWgtWave;
};

struct LaneGeo {
    uint32_t row_off;    // copy of 8 rows x 128 B with a row pitch of k bytes: (l/8)*k + ((l%8) ^ (l/8))*16
    uint32_t w4_off;     // the same with the Q4_0 row pitch of k/2 bytes
    uint32_t d8_off;     // copy of 32 rows x 32 B of block scales: (l/2)*(k/32)*4 + (l%2)*16
    uint32_t col[4];     // operand read: byte offset of chunk 2j+h of row l%32 inside a [4][8][8] x 16 B image
    uint32_t col4[8];    // Q4_0: chunk s of row l%32 (the 16 bytes of block s)
};

__device__ __forceinline__ LaneGeo lane_geo(int lane, int64_t k) {
    LaneGeo g;
    const uint32_t r8 = lane >> 3, c8 = lane & 7;
    g.row_off = r8 * (uint32_t)k + ((c8 ^ r8) << 4);
    g.w4_off = r8 * (uint32_t)(k >> 1) + ((c8 ^ r8) << 4);
    g.d8_off = (uint32_t)(lane >> 1) * (uint32_t)(k >> 5) * 4u + (uint32_t)(lane & 1) * 16u;
    const uint32_t r = lane & 31, h = lane >> 5;
#pragma unroll
    for (uint32_t j = 0; j < 4; j++) g.col[j] = (r >> 3) * 1024u + (r & 7) * 128u + (((2 * j + h) ^ (r & 7)) << 4);
#pragma unroll
    for (uint32_t s = 0; s < 8; s++) g.col4[s] = (r >> 3) * 1024u + (r & 7) * 128u + ((s ^ (r & 7)) << 4);
    return g;
}

// This wave's share of the activation copies of K step b into stage `buf`.
template <int DT, int MT>
__device__ __forceinline__ void stage_acts(uint8_t *buf, const cq_act_view &a, const LaneGeo &g, int64_t k, int64_t m0,
                                           int64_t b, int wave) {
    typedef Tile<DT, MT> T;
#pragma unroll
    for (int j = 0; j < MT * 8 / kWaves; j++) {
        const int idx = wave + kWaves * j;           // = (t*2 + kh)*4 + rg
        const int rg = idx & 3, kh = (idx >> 2) & 1, t = idx >> 3;
        dma16(a.qs + (m0 + t * 32 + rg * 8) * k + b * 256 + kh * 128, g.row_off, buf + idx * 1024);
    }
    // block scales: 32 rows x 8 floats per copy, one copy per tile
#pragma unroll
    for (int t = 0; t < MT; t++) {
        if (t + 4 == wave) dma16((const uint8_t *)(a.d + (m0 + t * 32) * (k >> 5) + b * 8), g.d8_off, buf + T::oD8 + t * 1024);
    }
}

// This wave's 32 weight rows of K step b into its own buffer.
template <int DT, bool ONCE>
__device__ __forceinline__ void stage_weights(uint8_t *wl, const cq_weight &w, const LaneGeo &g, int64_t n_tile, int64_t b) {
    const int64_t k = w.k;
    if (DT == CQ_DTYPE_Q8_0) {
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const int rg = i & 3, kh = i >> 2;
            if (ONCE) dma16_once(w.p0 + (n_tile + rg * 8) * k + b * 256 + kh * 128, g.row_off, wl + i * 1024);
            else dma16(w.p0 + (n_tile + rg * 8) * k + b * 256 + kh * 128, g.row_off, wl + i * 1024);
        }
    } else {
#pragma unroll
        for (int rg = 0; rg < 4; rg++) {
            if (ONCE) dma16_once(w.p0 + (n_tile + rg * 8) * (k >> 1) + b * 128, g.w4_off, wl + rg * 1024);
            else dma16(w.p0 + (n_tile + rg * 8) * (k >> 1) + b * 128, g.w4_off, wl + rg * 1024);
        }
    }
}

// DUMP (verification): the block integers are stored through `dump` instead of the result through `y`.
// ONCE: a launch with a single row tile (up to 32 rows), which reads every weight byte once.
template <int DT, int MT, bool DUMP, bool ONCE = false>
__global__ void __launch_bounds__(kThreads) gemm32_kernel(cq_weight w, cq_act_view a, int64_t m, float *__restrict__ y,
                                                          int ksplit, cq_mfma_dump dump) {
    typedef Tile<DT, MT> T;
    extern __shared__ __align__(16) uint8_t smem[];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int h = lane >> 5, col = lane & 31;
    const int64_t k = w.k, ks = k >> 8;                 // K steps of 256 elements
    const int64_t m0 = (int64_t)blockIdx.y * (MT * 32);
    const int64_t n_tile = ((int64_t)blockIdx.x * kWaves + wave) * 32;
    const bool n_ok = n_tile < w.n;                     // wave-uniform; a wave past the last row only helps with the copies
    const int64_t n = n_tile + col;
    const int64_t nc = n_ok ? n : 0;
    const int64_t b0 = ks * blockIdx.z / ksplit, b1 = ks * (blockIdx.z + 1) / ksplit;
    const LaneGeo g = lane_geo(lane, k);
    uint8_t *__restrict__ wl = smem + T::oWgt + wave * T::kWgtWave;
    const uint16_t *dplane = (const uint16_t *)w.p1;    // f16 block scales [n][k/32]

    v16f out[MT];
#pragma unroll
    for (int t = 0; t < MT; t++)
#pragma unroll
        for (int i = 0; i < 16; i++) out[t][i] = 0.0f;

    stage_acts<DT, MT>(smem, a, g, k, m0, b0, wave);
    if (n_ok) stage_weights<DT, ONCE>(wl, w, g, n_tile, b0);
    uint4 dnext = *(const uint4 *)(dplane + nc * (k >> 5) + b0 * 8);
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();

    for (int64_t b = b0; b < b1; b++) {
        const uint8_t *__restrict__ cur = smem + ((b - b0) & 1) * T::kStage;
        uint8_t *__restrict__ nxt = smem + (((b - b0) & 1) ^ 1) * T::kStage;
        const bool more = b + 1 < b1;
        if (more) stage_acts<DT, MT>(nxt, a, g, k, m0, b + 1, wave);
        if (n_ok) {
            // weight operands of the eight blocks into registers, then the buffer is free for the next step
            v4i bw[8];
            if (DT == CQ_DTYPE_Q8_0) {
#pragma unroll
                for (int s = 0; s < 8; s++) bw[s] = *(const v4i *)(wl + (s >> 2) * 4096 + g.col[s & 3]);
            } else {
#pragma unroll
                for (int s = 0; s < 8; s++) {
                    // block s: 16 bytes, low nibbles = elements 0..15 (h = 0), high nibbles = elements 16..31
                    const v4i q = *(const v4i *)(wl + g.col4[s]);
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        const uint32_t x = ((uint32_t)q[i] >> (4 * h)) & 0x0F0F0F0Fu;
                        bw[s][i] = (int)((x + 0x78787878u) ^ 0x80808080u);   // every byte minus 8, no carries between bytes
                    }
                }
            }
            const uint4 dcur = dnext;
            if (more) {
                stage_weights<DT, ONCE>(wl, w, g, n_tile, b + 1);
                dnext = *(const uint4 *)(dplane + nc * (k >> 5) + (b + 1) * 8);
            }
            // scale operand of block s: dw = b1 + b2 (bf16 pieces, exact: an f16 has 11 significant bits); lanes
            // 0..31 carry b1 in K-slots 0..2, lanes 32..63 carry b2 in K-slots 8..10, the other slots zero
            const uint32_t dwords[4] = {dcur.x, dcur.y, dcur.z, dcur.w};
            v8bf dw[8];
#pragma unroll
            for (int s = 0; s < 8; s++) {
                const float f = cq_h2f((uint16_t)((dwords[s >> 1] >> (16 * (s & 1))) & 0xffffu));
                const uint32_t fb = __float_as_uint(f);
                const float b2 = f - __uint_as_float(fb & 0xffff0000u);
                const uint32_t piece = h == 0 ? fb >> 16 : __float_as_uint(b2) >> 16;
                const v4u pk = {piece | (piece << 16), piece, 0u, 0u};
                dw[s] = __builtin_bit_cast(v8bf, pk);
            }

            // steps q = (tile t, block s): the two MFMAs of step q, and in their shadow the scaling of step q-1
            auto afrag = [&](int q) -> v4i {
                const int t = q >> 3, s = q & 7;
                return *(const v4i *)(cur + g.col[s & 3] + (t * 2 + (s >> 2)) * 4096);
            };
            // activation scale of (row l%32 of tile t, block s): read two steps ahead, and only turned into
            // the MFMA operand (three bf16 pieces) in the step that uses it, so that no step
            // waits for the read it has just issued
            auto d8raw = [&](int q) -> float {
                const int t = q >> 3, s = q & 7;
                return *(const float *)(cur + T::oD8 + (t * 32 + col) * 32 + s * 4);
            };
            auto d8frag = [&](float v) -> v8bf {
                // v = a1 + a2 + a3, each the leading eight bits of what the pieces before it leave (exact);
                // K-slots 0..2 of both lane halves
                const uint32_t vb = __float_as_uint(v);
                const float r1 = v - __uint_as_float(vb & 0xffff0000u);
                const uint32_t rb = __float_as_uint(r1);
                const float a3 = r1 - __uint_as_float(rb & 0xffff0000u);
                const v4u pk = {__builtin_amdgcn_perm(rb, vb, 0x07060302u), __float_as_uint(a3) >> 16, 0u, 0u};
                return __builtin_bit_cast(v8bf, pk);
            };
            v16i acc[2];
            v16f sc[2];
            v4i av[3];
            float dv[3];
            av[0] = afrag(0); av[1] = afrag(1);
            dv[0] = d8raw(0); dv[1] = d8raw(1);
            const v16i zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
            const v16f zerof = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int q = 0; q <= MT * 8; q++) {
                if (q + 2 < MT * 8) { av[(q + 2) % 3] = afrag(q + 2); dv[(q + 2) % 3] = d8raw(q + 2); }
                if (q < MT * 8) {
                    acc[q & 1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(av[q % 3], bw[q & 7], zero, 0, 0, 0);
                    sc[q & 1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(d8frag(dv[q % 3]), dw[q & 7], zerof, 0, 0, 0);
                }
                // keeps the MFMAs in front of the scaling below: left alone, the scheduler sinks them to the end
                // of the step, and the next step then starts by waiting for their results
                __builtin_amdgcn_sched_barrier(0);
                if (q > 0) {
                    const int p = (q - 1) & 1, t = (q - 1) >> 3;
#pragma unroll
                    for (int i = 0; i < 16; i++) {
                        if (DUMP) {
                            const int64_t row = m0 + t * 32 + (i >> 2) * 8 + h * 4 + (i & 3);
                            if (row < m) dump.i[(row * w.n + n) * (k >> 5) + b * 8 + ((q - 1) & 7)] = acc[p][i];
                        } else {
                            out[t][i] = __builtin_fmaf((float)acc[p][i], sc[p][i], out[t][i]);
                        }
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        __builtin_amdgcn_s_waitcnt(0);   // the next stage and the wave's next weights have landed in LDS
        __syncthreads();
    }

    if (n_ok && !DUMP) {
#pragma unroll
        for (int t = 0; t < MT; t++) {
#pragma unroll
            for (int i = 0; i < 16; i++) {
                const int64_t row = m0 + t * 32 + (i >> 2) * 8 + h * 4 + (i & 3);
                if (row < m) {
                    if (ksplit == 1) y[row * w.n + n] = out[t][i];
                    else unsafeAtomicAdd(&y[row * w.n + n], out[t][i]);
                }
            }
        }
    }
}

int g_cus = 0;
int num_cus() {
    if (g_cus == 0) {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) == hipSuccess &&
            hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0)
            g_cus = n;
        else
            g_cus = 256;
    }
    return g_cus;
}

// Tile height (MT x 32 activation rows per workgroup) and K split of a launch, from a cost model fitted to
// measurements (Q8_0, 256 CUs; unit 1/16 us): a workgroup spends 10 units per 256-element K step on its
// weights and 23 per 32-row tile on it, 24 on starting and finishing; workgroups run one per CU, in rounds;
// a split launch adds every part to the output atomically, which moves about 1.1 TB/s.
struct Plan {
    int mt, ksplit;
};
Plan pick_plan(const cq_weight *w, int64_t m) {
    const int64_t gx = (w->n + kWaves * 32 - 1) / (kWaves * 32), ks_total = w->k >> 8, cus = num_cus();
    const double atomic_pass = (double)m * (double)w->n * 4.0 / 1.1e6 * 16.0;   // bytes / (1.1e6 bytes per us) in units
    Plan best{1, 1};
    double best_cost = 0.0;
    bool first = true;
    for (int mt = 4; mt >= 1; mt >>= 1) {
        if (mt > 1 && m <= 16 * mt) continue;   // half the height holds all rows
        const int64_t tiles = gx * ((m + mt * 32 - 1) / (mt * 32));
        for (int ks = 1; ks <= 16; ks *= 2) {
            if (ks > 1 && ks_total / ks < 2) break;
            if (ks > 1 && cq_no_split_k()) break;   // CQ_FLAG_DETERMINISTIC
            const int64_t rounds = (tiles * ks + cus - 1) / cus;
            const double cost = (double)rounds * ((double)((ks_total + ks - 1) / ks) * (10.0 + 23.0 * mt) + 24.0) +
                                (ks > 1 ? ks * atomic_pass : 0.0);
            if (first || cost < best_cost) {
                best = Plan{mt, ks};
                best_cost = cost;
                first = false;
            }
        }
    }
    return best;
}

// DUMP: the same launch (tile height, K split) storing the block integers through `d`; y is not touched.
template <int DT, int MT, bool DUMP>
hipError_t launch_mt(const cq_weight *w, cq_act_view a, int64_t m, float *y, int ksplit, bool y_cleared, cq_mfma_dump d,
                     hipStream_t s) {
    const size_t lds = Tile<DT, MT>::kTotal;
    if (hipError_t e = cq_ensure_lds<gemm32_kernel<DT, MT, DUMP>>(w->dev, lds); e != hipSuccess) return e;
    const int64_t gx = (w->n + kWaves * 32 - 1) / (kWaves * 32), gy = (m + MT * 32 - 1) / (MT * 32);
    if (!DUMP && ksplit > 1 && !y_cleared) {
        hipError_t e = cq_launch_fill_zero(y, m * w->n, s);
        if (e != hipSuccess) return e;
    }
    dim3 grid((unsigned)gx, (unsigned)gy, (unsigned)ksplit);
    if constexpr (MT == 1 && !DUMP) {
        // a single row tile over 40 MB of weights and more: the copies marked non-temporal (measured at 17 and 32 rows:
        // 3-7 % faster from there on, 3-5 % slower below)
        const int64_t plane = DT == CQ_DTYPE_Q8_0 ? w->n * w->k : w->n * w->k / 2;
        if (gy == 1 && plane >= 40000000) {
            if (hipError_t e = cq_ensure_lds<gemm32_kernel<DT, 1, false, true>>(w->dev, lds); e != hipSuccess) return e;
            CQ_LAUNCH((gemm32_kernel<DT, 1, false, true>), grid, kThreads, lds, s, *w, a, m, y, ksplit, d);
            return hipGetLastError();
        }
    }
    CQ_LAUNCH((gemm32_kernel<DT, MT, DUMP>), grid, kThreads, lds, s, *w, a, m, y, ksplit, d);
    return hipGetLastError();
}

template <int DT, bool DUMP>
hipError_t launch_dt(const cq_weight *w, cq_act_view a, int64_t m, float *y, bool y_cleared, cq_mfma_dump d, hipStream_t s) {
    const Plan p = pick_plan(w, m);
    if (p.mt == 1) return launch_mt<DT, 1, DUMP>(w, a, m, y, p.ksplit, y_cleared, d, s);
    if (p.mt == 2) return launch_mt<DT, 2, DUMP>(w, a, m, y, p.ksplit, y_cleared, d, s);
    return launch_mt<DT, 4, DUMP>(w, a, m, y, p.ksplit, y_cleared, d, s);
}

}  // namespace

bool cq_gemm32_supported(const cq_weight *w, int act_dtype) {
    // whole 256-element K steps; the copies address 8 rows with 32-bit offsets
    return (w->dtype == CQ_DTYPE_Q8_0 || w->dtype == CQ_DTYPE_Q4_0) && act_dtype == CQ_DTYPE_Q8_0 && w->k >= 256 &&
           w->k % 256 == 0 && w->k <= (1 << 24) && w->n % 32 == 0 && w->n > 0;
}

bool cq_gemm32_splits_k(const cq_weight *w, int64_t m) { return m > 0 && pick_plan(w, m).ksplit > 1; }

hipError_t cq_launch_gemm32(const cq_weight *w, cq_act_view a, int act_dtype, int64_t m, float *y, bool y_cleared,
                            hipStream_t s) {
    if (!cq_gemm32_supported(w, act_dtype)) return hipErrorNotSupported;
    if (m == 0) return hipSuccess;
    if (a.m_stride < (m <= 32 ? 32 : (m + 127) / 128 * 128)) return hipErrorInvalidValue;   // rows the last tile may read
    const cq_mfma_dump none{nullptr, nullptr};
    if (w->dtype == CQ_DTYPE_Q8_0) return launch_dt<CQ_DTYPE_Q8_0, false>(w, a, m, y, y_cleared, none, s);
    return launch_dt<CQ_DTYPE_Q4_0, false>(w, a, m, y, y_cleared, none, s);
}

hipError_t cq_launch_gemm32_dump(const cq_weight *w, cq_act_view a, int act_dtype, int64_t m, cq_mfma_dump d, hipStream_t s) {
    if (!cq_gemm32_supported(w, act_dtype)) return hipErrorNotSupported;
    if (m == 0) return hipSuccess;
    if (a.m_stride < (m <= 32 ? 32 : (m + 127) / 128 * 128)) return hipErrorInvalidValue;
    if (w->dtype == CQ_DTYPE_Q8_0) return launch_dt<CQ_DTYPE_Q8_0, true>(w, a, m, nullptr, true, d, s);
    return launch_dt<CQ_DTYPE_Q4_0, true>(w, a, m, nullptr, true, d, s);
}
