// Transformation-compression kernels for gfx950: LSH projection + sign hash + bucket
// histogram, occupancy scan, id remap, row gathers (mean backward, reconstruct with
// fused bias + ReLU).  The per-cluster sums (mean forward, reconstruct backward) run
// on the member lists through the nnz-schedule SpMM in spmm.hip.
#include <type_traits>

#include "common.h"

namespace cgnn {

int spmm_members(const cgnn_csr *A, int dtype, const void *X, const void *M, void *Y, int64_t F,
                 int mask, void *ws, size_t ws_bytes, hipStream_t stream);

namespace {

// ------------------------------------------------------------------ LSH hash ---
//
// Every projection is the chain h_j = fma(x_k, W[k,j], h_j) for k ascending from 0, which
// fixes its rounding (the CPU oracle uses the same chain).  Tiles of 64 rows of X are
// staged in LDS with coalesced 16-byte loads; the LDS row stride is odd in units of the
// access width, which keeps the 64 strided row reads free of bank conflicts.
//
// Vector-unit kernel (used for double precision): one lane per row, one wave per
// workgroup, KS columns per pass.  W is read with wave-uniform addresses, i.e. through the
// scalar unit, so the inner loop is one LDS read per pack of k and HB vector FMAs per k.
// HB = number of accumulators (bits rounded up); columns >= bits repeat the last real
// column and are ignored when the code is formed.

constexpr int kLshRows = 64;
constexpr int kLshMaxSlab = 32;  // columns staged per pass (floats): 9 KB of LDS per wave

// One correctly rounded fused multiply-add in the operand type (the float overload must
// not go through double: rounding twice is not the same operation).
__device__ __forceinline__ float fused_mul_add(float a, float b, float c) { return __builtin_fmaf(a, b, c); }
__device__ __forceinline__ double fused_mul_add(double a, double b, double c) { return __builtin_fma(a, b, c); }

// Histogram update of one wave.  Feature rows of a graph are far from uniform: a few
// codes can hold most rows, and atomics on one counter serialise in the memory system.
// The wave therefore keeps kHeld (code, count) pairs in wave-uniform registers across its
// calls.  Per call: lanes whose code is held are added to that pair; then, up to kHeld
// times, the first lane still uncounted leads, every lane with its code is counted with
// it, and the pair replaces a held pair that saw no lane in this call (whose count is sent
// with one atomic), or is sent at once if every held pair was used; lanes left over count
// themselves.  A code that keeps turning up stays held until flush(), so a dominant code
// costs one atomic per wave instead of one per row.
constexpr int kHeld = 4;

// Where the (code, count) pairs of a wave go: the global counters.
struct GlobalSink {
    int32_t *bucket_count;
    __device__ __forceinline__ void operator()(int code, int n) const { atomicAdd(bucket_count + code, n); }
};

struct WaveCodeCounter {
    int code_[kHeld] = {-1, -1, -1, -1};
    int count_[kHeld] = {0, 0, 0, 0};
    int next_ = 0;

    template <typename Sink>
    __device__ __forceinline__ void flush(const Sink &sink, int lane) {
#pragma unroll
        for (int k = 0; k < kHeld; ++k) {
            if (count_[k] > 0 && lane == 0) sink(code_[k], count_[k]);
            count_[k] = 0;
        }
    }
    template <typename Sink>
    __device__ __forceinline__ void add(const Sink &sink, int code, bool valid, int lane) {
        unsigned long long todo = __ballot(valid);
        unsigned used = 0;
#pragma unroll
        for (int k = 0; k < kHeld; ++k) {
            const unsigned long long m = __ballot(valid && code == code_[k]);  // codes are >= 0
            count_[k] += __popcll(m);
            todo &= ~m;
            if (m != 0) used |= 1u << k;
        }
        for (int round = 0; round < kHeld && todo != 0; ++round) {
            const int leader = __ffsll(todo) - 1;
            const int lead = __builtin_amdgcn_readlane(code, leader);
            const unsigned long long same = __ballot(valid && code == lead);
            const int n = __popcll(same);
            todo &= ~same;
            int victim = -1;
#pragma unroll
            for (int j = 0; j < kHeld; ++j) {
                const int k = (next_ + j) % kHeld;
                if (victim < 0 && !((used >> k) & 1u)) victim = k;
            }
            if (victim < 0) {
                if (lane == leader) sink(lead, n);
                continue;
            }
#pragma unroll
            for (int k = 0; k < kHeld; ++k)
                if (k == victim) {
                    if (count_[k] > 0 && lane == 0) sink(code_[k], count_[k]);
                    code_[k] = lead;
                    count_[k] = n;
                }
            used |= 1u << victim;
            next_ = (victim + 1) % kHeld;
        }
        if ((todo >> lane) & 1) sink(code, 1);
    }
};

template <typename T>
struct LshArgs {
    const T *__restrict__ X;
    const T *__restrict__ W;
    int32_t *raw_code;
    int32_t *bucket_count;
    int64_t N;
    int32_t F;
    int32_t bits;
    int32_t slab;      // columns per pass, multiple of VEC
    int32_t stride_v;  // LDS row stride in units of VEC elements (odd)
    int32_t wstride;   // matrix-unit kernel, 16-byte rows: LDS stride of a plane in floats
    uint32_t magic;    // floor(2^32 / slab_v) + 1: i / slab_v == mulhi(i, magic) for i < 2^16
};

template <typename T, int VEC>
struct alignas(sizeof(T) * VEC) LPack {
    T v[VEC];
};

template <typename T, int VEC, int HB, bool EXACT>
__global__ __launch_bounds__(kLshRows) void lsh_hash_kernel(LshArgs<T> a) {
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
    LPack<T, VEC> *tile = reinterpret_cast<LPack<T, VEC> *>(lds_raw);
    const int lane = threadIdx.x;
    const int64_t row0 = (int64_t)blockIdx.x * kLshRows;
    const int rows_here = (int)min((int64_t)kLshRows, a.N - row0);
    const int H = a.bits;
    T acc[HB];
#pragma unroll
    for (int j = 0; j < HB; ++j) acc[j] = T(0);

    for (int k0 = 0; k0 < a.F; k0 += a.slab) {
        const int ks = min(a.slab, a.F - k0);  // multiple of VEC
        const int ks_v = ks / VEC;
        // magic division is exact for the full slab; a shorter last slab divides directly
        const bool full = ks == a.slab && a.magic != 0;
        const int total = rows_here * ks_v;
        __syncthreads();
        for (int i = lane; i < total; i += kLshRows) {
            int r = full ? (int)__umulhi((uint32_t)i, a.magic) : i / ks_v;
            int c = i - r * ks_v;
            const T *src = a.X + (row0 + r) * (int64_t)a.F + k0 + c * VEC;
            tile[r * a.stride_v + c] = *reinterpret_cast<const LPack<T, VEC> *>(src);
        }
        __syncthreads();
        if (lane < rows_here) {
            const LPack<T, VEC> *mine = tile + lane * a.stride_v;
            for (int c = 0; c < ks_v; ++c) {
                LPack<T, VEC> x = mine[c];
                // all plane values of these VEC columns first (wave-uniform addresses:
                // scalar loads issued back to back), then the multiply-add chains
                T w[VEC][HB];
#pragma unroll
                for (int i = 0; i < VEC; ++i) {
                    const T *wrow = a.W + (int64_t)(k0 + c * VEC + i) * (EXACT ? HB : H);
#pragma unroll
                    for (int j = 0; j < HB; ++j) w[i][j] = EXACT ? wrow[j] : wrow[min(j, H - 1)];
                }
#pragma unroll
                for (int i = 0; i < VEC; ++i)
#pragma unroll
                    for (int j = 0; j < HB; ++j) acc[j] = fused_mul_add(x.v[i], w[i][j], acc[j]);
            }
        }
    }
    int code = 0;
#pragma unroll
    for (int j = 0; j < HB; ++j)
        if (j < H) code = (code << 1) | (acc[j] > T(0) ? 1 : 0);
    if (lane < rows_here) a.raw_code[row0 + lane] = code;
    if (a.bucket_count == nullptr) return;
    WaveCodeCounter counter;
    const GlobalSink sink{a.bucket_count};
    counter.add(sink, code, lane < rows_here, lane);
    counter.flush(sink, lane);
}

// Single precision runs the same chains on the matrix unit.  v_mfma_f32_16x16x1_4b_f32
// computes, for four independent 16x16 blocks, D[i][j] = fma(A[i], B[j], C[i][j]) with
// one rounding (K = 1, so no sum is formed inside the instruction; results agree bit
// for bit with fmaf, denormals included).  Lane L supplies A = x[row L][k] (block L/16,
// i = L%16) and B = W[k][L%16]; one instruction advances all 64 rows x 16 planes by
// one k at twice the rate of 16 vector FMAs and without touching the scalar unit.
// Accumulator register v of lane L holds plane L%16 of row 16*(v/4) + 4*(L/16) + v%4,
// so ballot(acc[v] > 0) carries four complete 16-bit sign masks, one per 16-lane field.
//
// A pass stages up to 128 columns of the 64 rows, so rows of up to 512 bytes are read
// whole and every cache line of X is fetched once.  That much LDS per wave leaves room for
// only a few waves per compute unit, so the waves are persistent (each walks tiles
// t, t + stride, ... in the general form; in the flat form a workgroup's waves draw from
// its tiles in turn) and keep the next pass in registers, in flight, while they multiply
// the current one out of LDS.  W is staged with zero columns beyond `bits`; NG = 2 covers
// 17..30 planes with two instructions per k.  lsh_hash_mfma_kernel is the general form
// (any F, several passes per tile); lsh_hash_mfma_flat_kernel below is the form for
// 16-byte-aligned rows of at most 128 columns.

typedef float lsh_acc_t __attribute__((ext_vector_type(16)));
typedef float lsh_f4_t __attribute__((ext_vector_type(4)));

// Register / LDS element of the staged X tile: a native vector, so that the prefetch
// array stays in registers.
template <int VEC> struct LshPack;
template <> struct LshPack<4> {
    using type = lsh_f4_t;
    static __device__ __forceinline__ float at(const type &p, int i) { return p[i]; }
};
template <> struct LshPack<1> {
    using type = float;
    static __device__ __forceinline__ float at(const type &p, int) { return p; }
};

constexpr int kLshMfmaSlab = 128;  // columns per pass: rows of up to 512 bytes are staged whole

// Orders a wave's LDS writes before its own later reads of a region no other wave
// touches.  The LDS unit executes the instructions of one wave in order, so only the
// compiler has to be held; unlike a workgroup barrier this does not wait for global loads
// and atomics in flight.
__device__ __forceinline__ void wave_lds_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

template <int VEC, int NG>
__global__ __launch_bounds__(kLshRows) void lsh_hash_mfma_kernel(LshArgs<float> a, int64_t tiles) {
    using Pack = typename LshPack<VEC>::type;
    constexpr int HBP = 16 * NG;
    constexpr int XPER = (VEC == 4 ? kLshMfmaSlab : kLshMaxSlab) / VEC;  // X packs per lane and pass
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
    Pack *tile = reinterpret_cast<Pack *>(lds_raw);
    float *wtile = reinterpret_cast<float *>(lds_raw + (size_t)kLshRows * a.stride_v * sizeof(Pack));
    const int lane = threadIdx.x;
    const int H = a.bits;
    const int slabs = (a.F + a.slab - 1) / a.slab;

    lsh_acc_t acc[NG];
#pragma unroll
    for (int g = 0; g < NG; ++g)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[g][v] = 0.f;

    // columns [k0, k0 + slab) of the 64 rows of tile t: global -> registers, registers -> LDS
    Pack xr[XPER];
    auto fetch = [&](int64_t t, int k0) {
        const int64_t row0 = t * kLshRows;
        const int rows_here = (int)min((int64_t)kLshRows, a.N - row0);
        const float *xbase = a.X + row0 * (int64_t)a.F + k0;
        const int ks_v = min(a.slab, a.F - k0) / VEC;
        const bool full = ks_v * VEC == a.slab && a.magic != 0;
        const int total = rows_here * ks_v;
#pragma unroll
        for (int u = 0; u < XPER; ++u) {
            const int i = lane + u * kLshRows;
            if (i < total) {
                const int r = full ? (int)__umulhi((uint32_t)i, a.magic) : i / ks_v;
                const int c = i - r * ks_v;
                xr[u] = *reinterpret_cast<const Pack *>(xbase + (int64_t)r * a.F + c * VEC);
            }
        }
    };
    auto commit = [&](int64_t t, int k0) {
        const int rows_here = (int)min((int64_t)kLshRows, a.N - t * kLshRows);
        const int ks_v = min(a.slab, a.F - k0) / VEC;
        const bool full = ks_v * VEC == a.slab && a.magic != 0;
        const int total = rows_here * ks_v;
#pragma unroll
        for (int u = 0; u < XPER; ++u) {
            const int i = lane + u * kLshRows;
            if (i < total) {
                const int r = full ? (int)__umulhi((uint32_t)i, a.magic) : i / ks_v;
                const int c = i - r * ks_v;
                tile[r * a.stride_v + c] = xr[u];
            }
        }
    };
    // planes k0 .. k0+slab, zero beyond `bits`: [plane][k] with row stride wstride for
    // 16-byte reads of four consecutive k (VEC == 4), else [k][16*NG]
    auto stage_planes = [&](int k0) {
        const int n = min(a.slab, a.F - k0) * HBP;
        for (int e = lane; e < n; e += kLshRows) {
            const int kk = e / HBP, j = e % HBP;
            const float w = j < H ? a.W[(int64_t)(k0 + kk) * H + j] : 0.f;
            wtile[VEC == 4 ? j * a.wstride + kk : e] = w;
        }
    };

    // The wave walks tiles blockIdx.x, blockIdx.x + gridDim.x, ...; while it multiplies
    // one pass out of LDS, the next pass (of this tile or of the next one) is in flight.
    const int myv = 4 * (lane >> 4) + (lane & 3);
    WaveCodeCounter counter;
    const GlobalSink sink{a.bucket_count};
    if (slabs == 1) stage_planes(0);  // same planes for every tile; ordered before the first pass's reads
    fetch(blockIdx.x, 0);
    for (int64_t t = blockIdx.x; t < tiles; t += gridDim.x) {
        for (int s = 0; s < slabs; ++s) {
            const int k0 = s * a.slab;
            const int ks_v = min(a.slab, a.F - k0) / VEC;
            wave_lds_sync();  // the previous pass has been consumed
            commit(t, k0);
            if (slabs > 1) stage_planes(k0);
            wave_lds_sync();
            if (s + 1 < slabs)
                fetch(t, k0 + a.slab);
            else if (t + gridDim.x < tiles)
                fetch(t + gridDim.x, 0);
            // rows beyond the end of X multiply stale LDS contents; a row of D depends on
            // its own A element only, and those rows are never written out
            const Pack *mine = tile + lane * a.stride_v;
            if constexpr (VEC == 4) {
                const lsh_f4_t *wq = reinterpret_cast<const lsh_f4_t *>(wtile + (lane & 15) * a.wstride);
                const int gstep = 4 * a.wstride;  // 16 planes further, in 16-byte units
#pragma unroll 4
                for (int c = 0; c < ks_v; ++c) {
                    const lsh_f4_t x = mine[c];
                    lsh_f4_t w[NG];
#pragma unroll
                    for (int g = 0; g < NG; ++g) w[g] = wq[g * gstep + c];
#pragma unroll
                    for (int i = 0; i < 4; ++i)
#pragma unroll
                        for (int g = 0; g < NG; ++g)
                            acc[g] = __builtin_amdgcn_mfma_f32_16x16x1f32(x[i], w[g][i], acc[g], 0, 0, 0);
                }
            } else {
                const float *wcol = wtile + (lane & 15);
#pragma unroll 4
                for (int c = 0; c < ks_v; ++c) {
                    const float x = mine[c];
#pragma unroll
                    for (int g = 0; g < NG; ++g)
                        acc[g] = __builtin_amdgcn_mfma_f32_16x16x1f32(x, wcol[c * HBP + g * 16], acc[g], 0, 0, 0);
                }
            }
        }

        unsigned long long sel[NG];
#pragma unroll
        for (int g = 0; g < NG; ++g) {
            sel[g] = 0;
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const unsigned long long b = __ballot(acc[g][v] > 0.f);
                sel[g] = myv == v ? b : sel[g];
                acc[g][v] = 0.f;
            }
        }
        const int64_t row = t * kLshRows + lane;
        const int shift = 16 * ((lane & 15) >> 2);
        uint32_t mask = (uint32_t)(sel[0] >> shift) & 0xffffu;  // bit j = (h_j > 0)
        if (NG == 2) mask |= ((uint32_t)(sel[NG - 1] >> shift) & 0xffffu) << 16;
        const int code = (int)(__brev(mask) >> (32 - H));  // plane 0 is the top bit
        if (row < a.N) a.raw_code[row] = code;
        if (a.bucket_count != nullptr) counter.add(sink, code, row < a.N, lane);
    }
    counter.flush(sink, lane);
}

// Whole rows per pass (F <= 128, 16-byte packs): the 64 rows of a tile are one contiguous
// range of X, so pack p = lane + 64*u of the tile needs no index arithmetic on the way in
// and a lane moves exactly F/4 packs per tile.  XP >= F/4 packs are loaded without any
// branch (offsets clamped to the last pack of the tile, which also covers the partial last
// tile: the rows such loads fill are not written out); only the LDS writes are guarded, by
// a wave-uniform condition.  The code of a tile is stored (and its bucket counted) only
// after the next tile has been committed to LDS, so that no wait for the loads also waits
// for that atomic.
//
// The tiles of a workgroup (those a static deal would give its waves) are handed out by a
// counter in LDS, one at a time: six waves on four SIMDs means two SIMDs carry two waves
// and two carry one, and a wave that has a SIMD to itself gets through its tiles faster.
constexpr int kLshFlatMaxWaves = 8;
constexpr int kLshQueueBytes = 16;  // the counter, padded so that the tiles stay 16-byte aligned

template <int NG, int XP>
__global__ __launch_bounds__(kLshRows *kLshFlatMaxWaves) void lsh_hash_mfma_flat_kernel(LshArgs<float> a,
                                                                                       int64_t tiles) {
    // LDS: the planes, shared by the waves of the workgroup, then one X tile per wave.
    // The waves are independent after the planes have been staged.
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
    const int lane = threadIdx.x & (kLshRows - 1);
    const int wave = threadIdx.x / kLshRows;
    const int waves = blockDim.x / kLshRows;
    float *wtile = reinterpret_cast<float *>(lds_raw);
    const size_t plane_bytes = (size_t)a.wstride * 16 * NG * sizeof(float);
    int *queue = reinterpret_cast<int *>(lds_raw + plane_bytes);
    lsh_f4_t *tile = reinterpret_cast<lsh_f4_t *>(lds_raw + plane_bytes + kLshQueueBytes) +
                     (size_t)wave * kLshRows * a.stride_v;
    const int H = a.bits;
    const int ks_v = a.F / 4;  // packs per row = packs per lane and tile
    const lsh_f4_t *X4 = reinterpret_cast<const lsh_f4_t *>(a.X);
    const int64_t first = (int64_t)blockIdx.x * waves;
    const int64_t step = (int64_t)gridDim.x * waves;
    const GlobalSink sink{a.bucket_count};

    for (int e = threadIdx.x; e < a.F * 16 * NG; e += blockDim.x) {  // planes as [plane][k]
        const int kk = e / (16 * NG), j = e % (16 * NG);
        wtile[j * a.wstride + kk] = j < H ? a.W[(int64_t)kk * H + j] : 0.f;
    }
    if (threadIdx.x == 0) *queue = 0;
    __syncthreads();
    // the j-th tile of this workgroup; grows with j, so a wave that draws one beyond the
    // end is done, and so is every later draw
    auto take = [&]() -> int64_t {
        int j = 0;
        if (lane == 0) j = atomicAdd(queue, 1);
        j = __builtin_amdgcn_readfirstlane(j);
        return (int64_t)(j / waves) * step + first + j % waves;
    };

    lsh_acc_t acc[NG];
#pragma unroll
    for (int g = 0; g < NG; ++g)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[g][v] = 0.f;

    lsh_f4_t xr[XP];
    auto fetch = [&](int64_t t) {
        const int64_t row0 = t * kLshRows;
        const lsh_f4_t *src = X4 + row0 * ks_v;
        const int top = (int)min((int64_t)kLshRows, a.N - row0) * ks_v - 1;
#pragma unroll
        for (int u = 0; u < XP; ++u) xr[u] = __builtin_nontemporal_load(src + min(lane + u * kLshRows, top));
    };
    // slot of pack p: row * stride_v + column pack = p + row * (stride_v - ks_v)
    const bool padded = a.stride_v != ks_v;
    const int myv = 4 * (lane >> 4) + (lane & 3);
    const int shift = 16 * ((lane & 15) >> 2);
    const lsh_f4_t *mine = tile + lane * a.stride_v;
    const lsh_f4_t *wq = reinterpret_cast<const lsh_f4_t *>(wtile + (lane & 15) * a.wstride);
    const int gstep = 4 * a.wstride;  // 16 planes further, in 16-byte units

    auto multiply = [&](int c, auto count) {
        constexpr int n = decltype(count)::value;
        lsh_f4_t x[n], w[NG][n];
#pragma unroll
        for (int i = 0; i < n; ++i) {
            x[i] = mine[c + i];
#pragma unroll
            for (int g = 0; g < NG; ++g) w[g][i] = wq[g * gstep + c + i];
        }
        // left to itself the scheduler sinks every pair of reads to its four matrix
        // instructions, into one set of registers, and pays the LDS latency per pack
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < n; ++i)
#pragma unroll
            for (int k = 0; k < 4; ++k)
#pragma unroll
                for (int g = 0; g < NG; ++g)
                    acc[g] = __builtin_amdgcn_mfma_f32_16x16x1f32(x[i][k], w[g][i][k], acc[g], 0, 0, 0);
    };

    WaveCodeCounter counter;
    int pending_code = 0;
    int64_t pending_row = -1;
    int64_t t = take();
    if (t < tiles) fetch(t);
    while (t < tiles) {
        wave_lds_sync();  // the previous tile has been consumed
#pragma unroll
        for (int u = 0; u < XP; ++u) {
            const int p = lane + u * kLshRows;
            if (u < ks_v) tile[p + (padded ? (int)__umulhi((uint32_t)p, a.magic) : 0)] = xr[u];
        }
        wave_lds_sync();
        if (pending_row >= 0 && pending_row < a.N) a.raw_code[pending_row] = pending_code;
        if (a.bucket_count != nullptr) counter.add(sink, pending_code, pending_row >= 0 && pending_row < a.N, lane);
        const int64_t t_next = take();
        if (t_next < tiles) fetch(t_next);

        // eight column packs at a time: all sixteen LDS reads are issued before the first
        // multiply, so their latency is paid once per 32 matrix instructions
        int c = 0;
        for (; c + 8 <= ks_v; c += 8) multiply(c, std::integral_constant<int, 8>{});
        if (c + 4 <= ks_v) {
            multiply(c, std::integral_constant<int, 4>{});
            c += 4;
        }
        for (; c < ks_v; ++c) multiply(c, std::integral_constant<int, 1>{});

        unsigned long long sel[NG];
#pragma unroll
        for (int g = 0; g < NG; ++g) {
            sel[g] = 0;
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const unsigned long long b = __ballot(acc[g][v] > 0.f);
                sel[g] = myv == v ? b : sel[g];
                acc[g][v] = 0.f;
            }
        }
        uint32_t mask = (uint32_t)(sel[0] >> shift) & 0xffffu;  // bit j = (h_j > 0)
        if (NG == 2) mask |= ((uint32_t)(sel[NG - 1] >> shift) & 0xffffu) << 16;
        pending_code = (int)(__brev(mask) >> (32 - H));  // plane 0 is the top bit
        pending_row = t * kLshRows + lane;
        t = t_next;
    }
    if (pending_row >= 0 && pending_row < a.N) a.raw_code[pending_row] = pending_code;
    if (a.bucket_count != nullptr) counter.add(sink, pending_code, pending_row >= 0 && pending_row < a.N, lane);
    counter.flush(sink, lane);
}

// bits == 0 or F == 0: every projection is empty, code 0.
__global__ void lsh_trivial_kernel(int32_t *raw_code, int32_t *bucket_count, int64_t N) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < N) raw_code[i] = 0;
    if (i == 0 && bucket_count != nullptr) bucket_count[0] = (int32_t)N;
}

__global__ void fill_i32_kernel(int32_t *p, int64_t n, int32_t v) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
         i += (int64_t)gridDim.x * blockDim.x)
        p[i] = v;
}

int fill_i32(int32_t *p, int64_t n, int32_t v, hipStream_t stream) {
    if (n == 0) return CGNN_OK;
    int64_t blocks = ceil_div(n, kBlock);
    if (blocks > 4096) blocks = 4096;
    hipLaunchKernelGGL(fill_i32_kernel, dim3((unsigned)blocks), dim3(kBlock), 0, stream, p, n, v);
    return check_launch("fill");
}

template <typename T, int VEC, int HB, bool EXACT>
int launch_lsh(const LshArgs<T> &a, hipStream_t stream) {
    const size_t lds = (size_t)kLshRows * a.stride_v * VEC * sizeof(T);
    const int64_t blocks = ceil_div(a.N, kLshRows);
    hipLaunchKernelGGL((lsh_hash_kernel<T, VEC, HB, EXACT>), dim3((unsigned)blocks), dim3(kLshRows),
                       lds, stream, a);
    return check_launch("lsh_hash");
}

// Compute units of the current device (looked up once per device).
int compute_units() {
    static int cached[64] = {0};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
    if (cached[dev] == 0) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
            n = 256;
        cached[dev] = n;
    }
    return cached[dev];
}

template <typename Kernel>
int launch_lsh_persistent(Kernel kernel, int waves, size_t lds, const LshArgs<float> &a, hipStream_t stream) {
    const int64_t tiles = ceil_div(a.N, kLshRows);
    // exactly as many workgroups as are resident at once, each wave walking its share of
    // the tiles
    int per_cu = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, kLshRows * waves, lds) != hipSuccess ||
        per_cu < 1)
        per_cu = 1;
    int64_t blocks = (int64_t)per_cu * compute_units();
    if (blocks > ceil_div(tiles, waves)) blocks = ceil_div(tiles, waves);
    hipLaunchKernelGGL(kernel, dim3((unsigned)blocks), dim3(kLshRows * waves), lds, stream, a, tiles);
    return check_launch("lsh_hash");
}

constexpr size_t kLdsPerCu = 160 * 1024;
constexpr size_t kLdsDefaultLimit = 64 * 1024;  // larger workgroups must be allowed per kernel

template <int NG, int XP>
int launch_lsh_flat(const LshArgs<float> &a, hipStream_t stream) {
    const size_t tile_bytes = (size_t)kLshRows * a.stride_v * sizeof(lsh_f4_t);
    const size_t plane_bytes = (size_t)a.wstride * 16 * NG * sizeof(float);
    // as many waves as fit beside one copy of the planes; two per SIMD at most (registers)
    const size_t fixed_bytes = plane_bytes + kLshQueueBytes;
    int waves = (int)((kLdsPerCu - fixed_bytes) / tile_bytes);
    waves = waves < 1 ? 1 : (waves > kLshFlatMaxWaves ? kLshFlatMaxWaves : waves);
    auto kernel = lsh_hash_mfma_flat_kernel<NG, XP>;
    size_t lds = fixed_bytes + waves * tile_bytes;
    if (lds > kLdsDefaultLimit) {
        static bool allowed = false, refused = false;  // per kernel instantiation
        if (!allowed && !refused) {
            if (hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)kLdsPerCu) == hipSuccess)
                allowed = true;
            else {
                refused = true;
                (void)hipGetLastError();
            }
        }
        if (!allowed) {
            waves = (int)((kLdsDefaultLimit - fixed_bytes) / tile_bytes);
            waves = waves < 1 ? 1 : waves;
            lds = fixed_bytes + waves * tile_bytes;
        }
    }
    return launch_lsh_persistent(kernel, waves, lds, a, stream);
}

template <int VEC, int NG>
int launch_lsh_mfma(const LshArgs<float> &a, hipStream_t stream) {
    if (VEC == 4 && a.slab == a.F) {  // whole rows per pass
        const int packs = a.F / 4;
        if (packs <= 4) return launch_lsh_flat<NG, 4>(a, stream);
        if (packs <= 8) return launch_lsh_flat<NG, 8>(a, stream);
        if (packs <= 12) return launch_lsh_flat<NG, 12>(a, stream);
        if (packs <= 16) return launch_lsh_flat<NG, 16>(a, stream);
        if (packs <= 20) return launch_lsh_flat<NG, 20>(a, stream);
        if (packs <= 24) return launch_lsh_flat<NG, 24>(a, stream);
        if (packs == 25) return launch_lsh_flat<NG, 25>(a, stream);
        if (packs <= 28) return launch_lsh_flat<NG, 28>(a, stream);
        return launch_lsh_flat<NG, 32>(a, stream);
    }
    const size_t x_bytes = (size_t)kLshRows * a.stride_v * VEC * sizeof(float);
    return launch_lsh_persistent(lsh_hash_mfma_kernel<VEC, NG>, 1,
                                 x_bytes + (size_t)(VEC == 4 ? a.wstride : a.slab) * 16 * NG * sizeof(float), a,
                                 stream);
}

template <typename T, int VEC>
int dispatch_lsh(const LshArgs<T> &a, hipStream_t stream) {
    const int H = a.bits;
    if constexpr (sizeof(T) == sizeof(float)) {
        if (H <= 16) return launch_lsh_mfma<VEC, 1>(a, stream);
        return launch_lsh_mfma<VEC, 2>(a, stream);
    } else {
        if (H == 8) return launch_lsh<T, VEC, 8, true>(a, stream);
        if (H == 16) return launch_lsh<T, VEC, 16, true>(a, stream);
        if (H < 8) return launch_lsh<T, VEC, 8, false>(a, stream);
        if (H < 16) return launch_lsh<T, VEC, 16, false>(a, stream);
        return launch_lsh<T, VEC, 32, false>(a, stream);
    }
}

template <typename T>
int lsh_hash_typed(int64_t N, int64_t F, int bits, const void *X, const void *W, int32_t *raw_code,
                   int32_t *bucket_count, hipStream_t stream) {
    LshArgs<T> a{};
    a.X = static_cast<const T *>(X);
    a.W = static_cast<const T *>(W);
    a.raw_code = raw_code;
    a.bucket_count = bucket_count;
    a.N = N;
    a.F = (int32_t)F;
    a.bits = bits;
    constexpr int WIDE = 16 / sizeof(T);  // elements per 16-byte access
    const bool wide = (F % WIDE == 0) && (reinterpret_cast<uintptr_t>(X) % 16 == 0);
    const int vec = wide ? WIDE : 1;
    // single precision with 16-byte rows: whole rows of up to 512 bytes per pass
    const int max_slab = sizeof(T) == sizeof(float) ? (wide ? kLshMfmaSlab : kLshMaxSlab) : kLshMaxSlab / 2;
    int slab = (int)(F < max_slab ? F : max_slab);
    slab -= slab % vec;
    a.slab = slab;
    const int slab_v = slab / vec;
    a.stride_v = slab_v | 1;
    a.wstride = ((slab / 4) | 1) * 4;  // odd in 16-byte units: 16 planes read without bank conflicts
    a.magic = slab_v > 1 ? (uint32_t)((1ull << 32) / (uint32_t)slab_v) + 1u : 0u;  // 0: divide directly
    if (wide) return dispatch_lsh<T, WIDE>(a, stream);
    return dispatch_lsh<T, 1>(a, stream);
}

// ---------------------------------------------------------- occupancy scan -----
//
// prefix[b] = #{b' <= b : bucket_count[b'] != 0}.  Three passes over tiles of
// kScanTile buckets: tile totals, an in-place exclusive scan of the totals by one
// workgroup, then the tile scans offset by their totals.

constexpr int kScanItems = 16;
constexpr int kScanTile = kBlock * kScanItems;

__device__ __forceinline__ int wave_inclusive_scan(int v) {
#pragma unroll
    for (int d = 1; d < kWave; d <<= 1) {
        int n = __shfl_up(v, d, kWave);
        if ((int)(threadIdx.x % kWave) >= d) v += n;
    }
    return v;
}

// Inclusive scan of one value per thread over the workgroup; returns the inclusive
// value and the workgroup total.
__device__ __forceinline__ int block_inclusive_scan(int v, int *total) {
    __shared__ int wave_sum[kBlock / kWave];
    const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    int inc = wave_inclusive_scan(v);
    __syncthreads();  // wave_sum may still be read by a previous call
    if (lane == kWave - 1) wave_sum[wave] = inc;
    __syncthreads();
    int offset = 0, sum = 0;
#pragma unroll
    for (int w = 0; w < kBlock / kWave; ++w) {
        if (w < wave) offset += wave_sum[w];
        sum += wave_sum[w];
    }
    *total = sum;
    return inc + offset;
}

__global__ __launch_bounds__(kBlock) void scan_tile_totals_kernel(const int32_t *count, int64_t n,
                                                                 int32_t *totals) {
    const int64_t base = (int64_t)blockIdx.x * kScanTile + (int64_t)threadIdx.x * kScanItems;
    int s = 0;
#pragma unroll
    for (int i = 0; i < kScanItems; ++i)
        if (base + i < n) s += count[base + i] != 0;
    int total;
    block_inclusive_scan(s, &total);
    if (threadIdx.x == 0) totals[blockIdx.x] = total;
}

__global__ __launch_bounds__(kBlock) void scan_totals_kernel(int32_t *totals, int64_t m) {
    int running = 0;
    for (int64_t base = 0; base < m; base += kBlock) {
        int64_t i = base + threadIdx.x;
        int v = i < m ? totals[i] : 0;
        int total;
        int inc = block_inclusive_scan(v, &total);
        if (i < m) totals[i] = running + inc - v;  // exclusive
        running += total;
    }
}

__global__ __launch_bounds__(kBlock) void scan_apply_kernel(const int32_t *count, int64_t n,
                                                           const int32_t *totals, int32_t *prefix) {
    const int64_t base = (int64_t)blockIdx.x * kScanTile + (int64_t)threadIdx.x * kScanItems;
    int flag[kScanItems];
    int s = 0;
#pragma unroll
    for (int i = 0; i < kScanItems; ++i) {
        flag[i] = (base + i < n) ? (count[base + i] != 0) : 0;
        s += flag[i];
    }
    int total;
    int inc = block_inclusive_scan(s, &total);
    int run = totals[blockIdx.x] + inc - s;
#pragma unroll
    for (int i = 0; i < kScanItems; ++i) {
        run += flag[i];
        if (base + i < n) prefix[base + i] = run;
    }
}

__global__ void lsh_finish_kernel(int64_t N, int64_t buckets, const int32_t *raw_code,
                                  const int32_t *bucket_count, const int32_t *prefix, int64_t *ids,
                                  int32_t *counts) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < N || i < buckets;
         i += (int64_t)gridDim.x * blockDim.x) {
        if (i < N) ids[i] = prefix[raw_code[i]];
        if (i < buckets) {
            int c = bucket_count[i];
            if (c) counts[prefix[i]] = c;
        }
    }
}

// ------------------------------------------------------------ row gathers ------
//
// out[i,:] = f(src[ids[i],:]) with LPR lanes per row and VEC features per lane; each
// lane group handles kGatherRows consecutive rows with all loads issued first.

constexpr int kGatherRows = 4;
enum { GATHER_MEAN_GRAD = 0, GATHER_RECONSTRUCT = 1 };

template <typename T>
struct GatherArgs {
    const T *__restrict__ src;       // [groups x F]
    const int64_t *__restrict__ ids; // [N]
    const int32_t *__restrict__ counts;
    const int32_t *__restrict__ perm; // [N] or NULL: order in which the rows are produced
    const T *__restrict__ bias;
    T *__restrict__ out;             // [N x F]
    int32_t *bad_id;                 // set to 1 when an id lies outside [0, groups), or NULL
    uint32_t *signs;                 // reconstruct: bit f % 32 of word [i, f / 32] = !(out[i, f] <= 0), or NULL
    int64_t N, F, groups;
    int32_t relu;
    int32_t sign_words;              // words per row of signs: ceil(F / 32)
};

// Output rows are written once and not read again here: streaming stores.
template <typename T, int VEC>
__device__ __forceinline__ void store_stream(T *p, const LPack<T, VEC> &x) {
    if constexpr (VEC == 1) {
        __builtin_nontemporal_store(x.v[0], p);
    } else {
        typedef T vec_t __attribute__((ext_vector_type(VEC)));
        vec_t v;
#pragma unroll
        for (int i = 0; i < VEC; ++i) v[i] = x.v[i];
        __builtin_nontemporal_store(v, reinterpret_cast<vec_t *>(p));
    }
}

template <typename T, int VEC, int LPR, int OP>
__global__ __launch_bounds__(kBlock) void gather_rows_kernel(GatherArgs<T> a) {
    constexpr int GPB = kBlock / LPR;
    const int lane = threadIdx.x % LPR;
    int64_t first = ((int64_t)blockIdx.x * GPB + threadIdx.x / LPR) * kGatherRows;
    if (first >= a.N) return;
    // With `perm` (rows grouped by cluster) consecutive lane groups read the same row of
    // src, which then comes from cache instead of memory; the result does not depend on
    // the order.
    int64_t g[kGatherRows], row[kGatherRows];
#pragma unroll
    for (int r = 0; r < kGatherRows; ++r) {
        const int64_t p = first + r < a.N ? first + r : a.N - 1;
        row[r] = a.perm ? (int64_t)a.perm[p] : p;
        g[r] = a.ids[row[r]];
        // An id from outside the assignment operators may name no row of src: it is moved to the
        // nearest row that exists, so no access leaves the arrays, and reported through the flag.
        if (g[r] < 0 || g[r] >= a.groups) {
            g[r] = g[r] < 0 ? 0 : a.groups - 1;
            if (a.bad_id) *a.bad_id = 1;  // every writer stores the same value
        }
    }
    T denom[kGatherRows];
    if constexpr (OP == GATHER_MEAN_GRAD) {
#pragma unroll
        for (int r = 0; r < kGatherRows; ++r) denom[r] = (T)max(a.counts[g[r]], 1);
    }
    // the lanes of a row walk the features together (a lane past the end of the row idles), so that
    // lanes can exchange sign bits below
    for (int64_t fb = 0; fb < a.F; fb += (int64_t)LPR * VEC) {
        const int64_t f = fb + (int64_t)lane * VEC;
        const bool on = f < a.F;
        LPack<T, VEC> x[kGatherRows];
        uint32_t bits[kGatherRows];
#pragma unroll
        for (int r = 0; r < kGatherRows; ++r) bits[r] = 0;
        if (on) {
#pragma unroll
            for (int r = 0; r < kGatherRows; ++r)
                x[r] = *reinterpret_cast<const LPack<T, VEC> *>(a.src + g[r] * a.F + f);
            LPack<T, VEC> b;
            if constexpr (OP == GATHER_RECONSTRUCT) {
                if (a.bias) b = *reinterpret_cast<const LPack<T, VEC> *>(a.bias + f);
            }
#pragma unroll
            for (int r = 0; r < kGatherRows; ++r) {
                if (first + r >= a.N) break;
#pragma unroll
                for (int i = 0; i < VEC; ++i) {
                    T v = x[r].v[i];
                    if constexpr (OP == GATHER_MEAN_GRAD) {
                        v = v / denom[r];
                    } else {
                        if (a.bias) v = v + b.v[i];
                        v = (a.relu && v < T(0)) ? T(0) : v;
                        bits[r] |= (v <= T(0) ? 0u : 1u) << i;
                    }
                    x[r].v[i] = v;
                }
                store_stream<T, VEC>(a.out + row[r] * a.F + f, x[r]);
            }
        }
        if constexpr (OP == GATHER_RECONSTRUCT) {
            if (a.signs != nullptr) {
                // VEC divides 32: the lanes whose bits share a word are R neighbours within the row's lanes
                constexpr int R = LPR < 32 / VEC ? LPR : 32 / VEC;
#pragma unroll
                for (int r = 0; r < kGatherRows; ++r) {
                    if (first + r >= a.N) break;  // the same for all lanes of the row
                    uint32_t w = bits[r] << (f & 31);
#pragma unroll
                    for (int d = 1; d < R; d <<= 1) w |= __shfl_xor(w, d);
                    if (on && lane % R == 0) a.signs[row[r] * a.sign_words + (f >> 5)] = w;
                }
            }
        }
    }
}

// Both gathers in natural row order over rows that are not whole cache lines (and, for the
// reconstruct, without sign words): the output is walked as one array of 16-byte packs, so every store instruction of a wave covers 64
// consecutive packs -- whole 128-byte lines -- wherever the rows begin and end.  A workgroup
// takes a multiple of 64 rows (a whole number of lines whatever F is), enough of them for
// every thread to have four packs; pack l of them lies in row l / packs_per_row, by
// multiplication (exact for l < 2^16).
constexpr int kFlatRows = 64;
constexpr int kFlatItems = 4;  // packs of a thread in flight together

template <typename T, int VEC, int OP>
__global__ __launch_bounds__(kBlock) void gather_flat_kernel(GatherArgs<T> a, int ppr, uint32_t magic,
                                                             int rows_per_group) {
    const int64_t row0 = (int64_t)blockIdx.x * rows_per_group;
    const int rows = (int)min((int64_t)rows_per_group, a.N - row0);
    const int packs = rows * ppr;
    const LPack<T, VEC> *src = reinterpret_cast<const LPack<T, VEC> *>(a.src);
    T *out = a.out + row0 * a.F;
    for (int l0 = threadIdx.x; l0 < packs; l0 += kFlatItems * kBlock) {
        int col[kFlatItems];
        int64_t g[kFlatItems];
#pragma unroll
        for (int u = 0; u < kFlatItems; ++u) {
            const int l = min(l0 + u * kBlock, packs - 1);
            const int r = (int)__umulhi((uint32_t)l, magic);
            col[u] = l - r * ppr;
            g[u] = a.ids[row0 + r];
        }
        T denom[kFlatItems];
        LPack<T, VEC> x[kFlatItems];
#pragma unroll
        for (int u = 0; u < kFlatItems; ++u) {
            // an id that names no row of src is moved to the nearest row that exists and reported
            if (g[u] < 0 || g[u] >= a.groups) {
                g[u] = g[u] < 0 ? 0 : a.groups - 1;
                if (a.bad_id) *a.bad_id = 1;  // every writer stores the same value
            }
            if constexpr (OP == GATHER_MEAN_GRAD) denom[u] = (T)max(a.counts[g[u]], 1);
            x[u] = src[g[u] * ppr + col[u]];
        }
#pragma unroll
        for (int u = 0; u < kFlatItems; ++u) {
            const int l = l0 + u * kBlock;
            if (l >= packs) break;
            if constexpr (OP == GATHER_MEAN_GRAD) {
#pragma unroll
                for (int i = 0; i < VEC; ++i) x[u].v[i] = x[u].v[i] / denom[u];
            } else {
                LPack<T, VEC> b;
                if (a.bias) b = reinterpret_cast<const LPack<T, VEC> *>(a.bias)[col[u]];
#pragma unroll
                for (int i = 0; i < VEC; ++i) {
                    T v = x[u].v[i];
                    if (a.bias) v = v + b.v[i];
                    x[u].v[i] = (a.relu && v < T(0)) ? T(0) : v;
                }
            }
            store_stream<T, VEC>(out + (int64_t)l * VEC, x[u]);
        }
    }
}

template <typename T, int VEC, int OP>
int launch_gather_lpr(const GatherArgs<T> &a, hipStream_t stream) {
    const int64_t slots = a.F / VEC;
    int lpr = pow2_ceil(slots);
    lpr = lpr <= 4 ? 4 : (lpr <= 8 ? 8 : (lpr <= 16 ? 16 : (lpr <= 32 ? 32 : 64)));
    const int gpb = kBlock / lpr;
    const int64_t groups_needed = ceil_div(a.N, kGatherRows);
    dim3 grid((unsigned)ceil_div(groups_needed, gpb)), block(kBlock);
    switch (lpr) {
        case 4: hipLaunchKernelGGL((gather_rows_kernel<T, VEC, 4, OP>), grid, block, 0, stream, a); break;
        case 8: hipLaunchKernelGGL((gather_rows_kernel<T, VEC, 8, OP>), grid, block, 0, stream, a); break;
        case 16: hipLaunchKernelGGL((gather_rows_kernel<T, VEC, 16, OP>), grid, block, 0, stream, a); break;
        case 32: hipLaunchKernelGGL((gather_rows_kernel<T, VEC, 32, OP>), grid, block, 0, stream, a); break;
        default: hipLaunchKernelGGL((gather_rows_kernel<T, VEC, 64, OP>), grid, block, 0, stream, a); break;
    }
    return check_launch("gather_rows");
}

template <typename T, int OP>
int launch_gather(const GatherArgs<T> &a, hipStream_t stream) {
    if (a.N == 0 || a.F == 0) return CGNN_OK;
    if (ceil_div(a.N, kGatherRows) >= ((int64_t)1 << 31))
        return fail(CGNN_EUNSUPPORTED, "gather: too many rows");
    constexpr int WIDE = 16 / sizeof(T);
    auto al = [](const void *p) { return p == nullptr || reinterpret_cast<uintptr_t>(p) % 16 == 0; };
    const bool wide = a.F % WIDE == 0 && al(a.src) && al(a.out) && al(a.bias);
    const int64_t ppr = a.F / WIDE;
    if (wide && a.perm == nullptr && a.signs == nullptr && (a.F * (int64_t)sizeof(T)) % 128 != 0 && ppr > 1 &&
        kFlatRows * ppr < (1 << 16) && ceil_div(a.N, kFlatRows) < ((int64_t)1 << 31)) {
        const uint32_t magic = (uint32_t)((1ull << 32) / (uint32_t)ppr) + 1u;
        // 64 rows, or as many times 64 as give the threads their four packs each
        const int rows = kFlatRows * (int)std::max<int64_t>(1, kFlatItems * kBlock / (kFlatRows * ppr));
        hipLaunchKernelGGL((gather_flat_kernel<T, WIDE, OP>), dim3((unsigned)ceil_div(a.N, rows)), dim3(kBlock), 0,
                           stream, a, (int)ppr, magic, rows);
        return check_launch("gather_flat");
    }
    if (wide) return launch_gather_lpr<T, WIDE, OP>(a, stream);
    return launch_gather_lpr<T, 1, OP>(a, stream);
}

// reps[g, :] /= max(counts[g], 1), VEC features per thread (a row holds `slots` such pieces).
template <typename T, int VEC>
__global__ __launch_bounds__(kBlock) void divide_counts_kernel(T *reps, const int32_t *counts, int64_t total_slots,
                                                              uint32_t slots) {
    const bool narrow = total_slots < ((int64_t)1 << 32);  // the row of a piece by a 32-bit division
    for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < total_slots; i += (int64_t)gridDim.x * kBlock) {
        const int64_t g = narrow ? (int64_t)((uint32_t)i / slots) : i / (int64_t)slots;
        const T c = (T)max(counts[g], 1);
        LPack<T, VEC> v = *reinterpret_cast<const LPack<T, VEC> *>(reps + i * VEC);
#pragma unroll
        for (int k = 0; k < VEC; ++k) v.v[k] = v.v[k] / c;
        *reinterpret_cast<LPack<T, VEC> *>(reps + i * VEC) = v;
    }
}

__global__ void copy16_kernel(const uint4 *__restrict__ src, uint4 *__restrict__ dst, size_t n) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
         i += (size_t)gridDim.x * blockDim.x)
        dst[i] = src[i];
}

// Reads n 16-byte words and keeps nothing: the memory system's streaming-read rate.
typedef unsigned int probe_word_t __attribute__((ext_vector_type(4)));

__global__ __launch_bounds__(kBlock) void read16_kernel(const probe_word_t *__restrict__ src, size_t n,
                                                       uint32_t *__restrict__ sink) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    uint32_t acc = 0;
    for (; i + 3 * stride < n; i += 4 * stride) {
        probe_word_t v[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) v[u] = __builtin_nontemporal_load(src + i + u * stride);
#pragma unroll
        for (int u = 0; u < 4; ++u) acc ^= v[u][0] ^ v[u][1] ^ v[u][2] ^ v[u][3];
    }
    for (; i < n; i += stride) {
        const probe_word_t v = src[i];
        acc ^= v[0] ^ v[1] ^ v[2] ^ v[3];
    }
    if (acc == 0x9e3779b9u) *sink = acc;  // keeps the loads alive; practically never taken
}

// Writes n 16-byte words of zeros with streaming stores: the memory system's write rate.
__global__ __launch_bounds__(kBlock) void fill16_kernel(probe_word_t *__restrict__ dst, size_t n) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    const probe_word_t zero = {0u, 0u, 0u, 0u};
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride)
        __builtin_nontemporal_store(zero, dst + i);
}

int check_bits(int bits) {
    if (bits < 0 || bits > 30) return fail(CGNN_EINVAL, "hash bits must be in [0,30]");
    return CGNN_OK;
}

size_t scan_tiles(int bits) { return (size_t)ceil_div((int64_t)1 << bits, kScanTile); }

cgnn_csr members_csr(int64_t N, int64_t groups, const int32_t *offsets, const int32_t *perm,
                     const int32_t *sorted_id, int64_t max_members = 0) {
    cgnn_csr A{};
    A.rows = groups;
    A.cols = N;
    A.nnz = N;
    A.rowptr = offsets;
    A.colidx = perm;
    A.rowidx = sorted_id;
    A.val = nullptr;
    A.max_row_nnz = max_members > 0 && max_members < INT32_MAX ? (int32_t)max_members : 0;
    A.seg_nnz = 0;  // default run length: measured best for both cluster sums
    return A;
}

}  // namespace
// out[i] = #{j <= i : in[j] != 0} over n int32 entries; scratch of occupancy_scan_bytes(n).
size_t occupancy_scan_bytes(int64_t n) { return align_up((size_t)ceil_div(n < 1 ? 1 : n, kScanTile) * sizeof(int32_t), 256); }

int occupancy_scan(const int32_t *in, int64_t n, int32_t *out, void *scratch, hipStream_t stream) {
    if (n <= 0) return CGNN_OK;
    const int64_t tiles = ceil_div(n, kScanTile);
    int32_t *totals = static_cast<int32_t *>(scratch);
    hipLaunchKernelGGL(scan_tile_totals_kernel, dim3((unsigned)tiles), dim3(kBlock), 0, stream, in, n, totals);
    hipLaunchKernelGGL(scan_totals_kernel, dim3(1), dim3(kBlock), 0, stream, totals, tiles);
    hipLaunchKernelGGL(scan_apply_kernel, dim3((unsigned)tiles), dim3(kBlock), 0, stream, in, n, totals, out);
    return check_launch("occupancy_scan");
}

}  // namespace cgnn

using namespace cgnn;

extern "C" int cgnn_lsh_hash(int64_t N, int64_t F, int bits, int dtype, const void *X, const void *W,
                             int32_t *raw_code, int32_t *bucket_count, cgnn_stream_t stream) {
    int rc = check_bits(bits);
    if (rc != CGNN_OK) return rc;
    CGNN_REQUIRE(N >= 0 && F >= 0, "cgnn_lsh_hash: negative size");
    CGNN_REQUIRE(N < INT32_MAX, "cgnn_lsh_hash: row count exceeds the int32 bucket counters");
    CGNN_REQUIRE(F < (1 << 24), "cgnn_lsh_hash: feature width too large");
    CGNN_REQUIRE(N == 0 || raw_code != nullptr, "cgnn_lsh_hash: raw_code is null");
    if (bucket_count != nullptr) rc = fill_i32(bucket_count, (int64_t)1 << bits, 0, stream);
    if (rc != CGNN_OK || N == 0) return rc;
    if (bits == 0 || F == 0) {
        hipLaunchKernelGGL(lsh_trivial_kernel, dim3((unsigned)ceil_div(N, kBlock)), dim3(kBlock), 0,
                           stream, raw_code, bucket_count, N);
        return check_launch("lsh_trivial");
    }
    CGNN_REQUIRE(X != nullptr && W != nullptr, "cgnn_lsh_hash: X or W is null");
    if (dtype == CGNN_F32) return lsh_hash_typed<float>(N, F, bits, X, W, raw_code, bucket_count, stream);
    if (dtype == CGNN_F64) return lsh_hash_typed<double>(N, F, bits, X, W, raw_code, bucket_count, stream);
    return fail(CGNN_EUNSUPPORTED, "cgnn_lsh_hash: dtype must be f32 or f64");
}

extern "C" size_t cgnn_lsh_scan_workspace_bytes(int bits) {
    if (bits < 0 || bits > 30) return 0;
    return align_up(scan_tiles(bits) * sizeof(int32_t), 256);
}

extern "C" int cgnn_lsh_scan(int bits, const int32_t *bucket_count, int32_t *prefix, void *workspace,
                             size_t workspace_bytes, cgnn_stream_t stream) {
    int rc = check_bits(bits);
    if (rc != CGNN_OK) return rc;
    CGNN_REQUIRE(bucket_count != nullptr && prefix != nullptr, "cgnn_lsh_scan: null array");
    if (workspace == nullptr || workspace_bytes < cgnn_lsh_scan_workspace_bytes(bits))
        return fail(CGNN_EWORKSPACE, "cgnn_lsh_scan: workspace too small");
    const int64_t n = (int64_t)1 << bits;
    const int64_t tiles = (int64_t)scan_tiles(bits);
    int32_t *totals = static_cast<int32_t *>(workspace);
    hipLaunchKernelGGL(scan_tile_totals_kernel, dim3((unsigned)tiles), dim3(kBlock), 0, stream,
                       bucket_count, n, totals);
    hipLaunchKernelGGL(scan_totals_kernel, dim3(1), dim3(kBlock), 0, stream, totals, tiles);
    hipLaunchKernelGGL(scan_apply_kernel, dim3((unsigned)tiles), dim3(kBlock), 0, stream, bucket_count,
                       n, totals, prefix);
    return check_launch("lsh_scan");
}

extern "C" int cgnn_lsh_finish(int64_t N, int bits, const int32_t *raw_code,
                               const int32_t *bucket_count, const int32_t *prefix, int64_t *ids,
                               int32_t *counts, cgnn_stream_t stream) {
    int rc = check_bits(bits);
    if (rc != CGNN_OK) return rc;
    CGNN_REQUIRE(N >= 0, "cgnn_lsh_finish: negative size");
    CGNN_REQUIRE(bucket_count && prefix && counts, "cgnn_lsh_finish: null array");
    CGNN_REQUIRE(N == 0 || (raw_code && ids), "cgnn_lsh_finish: null array");
    const int64_t buckets = (int64_t)1 << bits;
    int64_t work = N > buckets ? N : buckets;
    int64_t blocks = ceil_div(work, kBlock);
    if (blocks > 16384) blocks = 16384;
    hipLaunchKernelGGL(lsh_finish_kernel, dim3((unsigned)blocks), dim3(kBlock), 0, stream, N, buckets,
                       raw_code, bucket_count, prefix, ids, counts);
    return check_launch("lsh_finish");
}

extern "C" size_t cgnn_cluster_mean_workspace_bytes(int64_t N, int64_t F, int64_t groups, int dtype) {
    cgnn_csr A = members_csr(N, groups, nullptr, nullptr, nullptr);
    return cgnn_spmm_workspace_bytes(&A, F, dtype, CGNN_SPMM_NNZ);
}

template <typename T>
static int divide_counts(void *reps, const int32_t *counts, int64_t groups, int64_t F,
                         hipStream_t stream) {
    if (groups * F == 0) return CGNN_OK;
    constexpr int WIDE = 16 / sizeof(T);
    const bool wide = F % WIDE == 0 && reinterpret_cast<uintptr_t>(reps) % 16 == 0;
    const int64_t slots = wide ? F / WIDE : F, total = groups * slots;
    if (slots >= ((int64_t)1 << 32)) return fail(CGNN_EUNSUPPORTED, "cluster_mean: rows too wide");
    int64_t blocks = ceil_div(total, kBlock);
    if (blocks > 65536) blocks = 65536;
    if (wide)
        hipLaunchKernelGGL((divide_counts_kernel<T, WIDE>), dim3((unsigned)blocks), dim3(kBlock), 0, stream,
                           static_cast<T *>(reps), counts, total, (uint32_t)slots);
    else
        hipLaunchKernelGGL((divide_counts_kernel<T, 1>), dim3((unsigned)blocks), dim3(kBlock), 0, stream,
                           static_cast<T *>(reps), counts, total, (uint32_t)slots);
    return check_launch("divide_counts");
}

extern "C" int cgnn_cluster_mean(int64_t N, int64_t F, int64_t groups, int64_t max_members, int dtype, const void *X,
                                 const int32_t *offsets, const int32_t *perm,
                                 const int32_t *sorted_id, const int32_t *counts, void *reps,
                                 void *workspace, size_t workspace_bytes, cgnn_stream_t stream) {
    CGNN_REQUIRE(N >= 0 && F >= 0 && groups >= 1, "cgnn_cluster_mean: bad size");
    CGNN_REQUIRE(dtype == CGNN_F32 || dtype == CGNN_F64, "cgnn_cluster_mean: dtype must be f32 or f64");
    if (F == 0) return CGNN_OK;
    CGNN_REQUIRE(offsets && counts && reps, "cgnn_cluster_mean: null array");
    CGNN_REQUIRE(N == 0 || (X && perm && sorted_id), "cgnn_cluster_mean: null array");
    cgnn_csr A = members_csr(N, groups, offsets, perm, sorted_id, max_members);
    int rc = spmm_members(&A, dtype, X, nullptr, reps, F, 0, workspace, workspace_bytes, stream);
    if (rc != CGNN_OK) return rc;
    if (dtype == CGNN_F32) return divide_counts<float>(reps, counts, groups, F, stream);
    return divide_counts<double>(reps, counts, groups, F, stream);
}

template <typename T, int OP>
static int gather_typed(int64_t N, int64_t F, int64_t groups, const void *src, const int64_t *ids,
                        const int32_t *counts, const int32_t *perm, const void *bias, int relu, void *out,
                        int32_t *bad_id, hipStream_t stream, uint32_t *signs = nullptr) {
    GatherArgs<T> a{};
    a.signs = signs;
    a.sign_words = (int32_t)ceil_div(F, 32);
    a.src = static_cast<const T *>(src);
    a.ids = ids;
    a.counts = counts;
    // scattered row writes pay off only when a row is a whole number of 128-byte lines
    a.perm = (F * (int64_t)sizeof(T)) % 128 == 0 ? perm : nullptr;
    a.bias = static_cast<const T *>(bias);
    a.out = static_cast<T *>(out);
    a.bad_id = bad_id;
    a.N = N;
    a.F = F;
    a.groups = groups;
    a.relu = relu ? 1 : 0;
    return launch_gather<T, OP>(a, stream);
}

extern "C" int cgnn_cluster_mean_backward(int64_t N, int64_t F, int64_t groups, int dtype,
                                          const void *grad, const int64_t *ids,
                                          const int32_t *counts, const int32_t *perm, void *dx,
                                          int32_t *bad_id, cgnn_stream_t stream) {
    CGNN_REQUIRE(N >= 0 && F >= 0 && groups >= 1, "cgnn_cluster_mean_backward: bad size");
    if (N == 0 || F == 0) return CGNN_OK;
    CGNN_REQUIRE(grad && ids && counts && dx, "cgnn_cluster_mean_backward: null array");
    if (dtype == CGNN_F32)
        return gather_typed<float, GATHER_MEAN_GRAD>(N, F, groups, grad, ids, counts, perm, nullptr, 0, dx, bad_id, stream);
    if (dtype == CGNN_F64)
        return gather_typed<double, GATHER_MEAN_GRAD>(N, F, groups, grad, ids, counts, perm, nullptr, 0, dx, bad_id, stream);
    return fail(CGNN_EUNSUPPORTED, "cgnn_cluster_mean_backward: dtype must be f32 or f64");
}

extern "C" int cgnn_reconstruct(int64_t N, int64_t F, int64_t groups, int dtype, const void *reps,
                                const int64_t *ids, const int32_t *perm, const void *bias, int relu,
                                void *out, int32_t *bad_id, cgnn_stream_t stream) {
    CGNN_REQUIRE(N >= 0 && F >= 0 && groups >= 0, "cgnn_reconstruct: bad size");
    CGNN_REQUIRE(N == 0 || F == 0 || groups >= 1, "cgnn_reconstruct: rows to reconstruct but no representatives");
    if (N == 0 || F == 0) return CGNN_OK;
    CGNN_REQUIRE(reps && ids && out, "cgnn_reconstruct: null array");
    if (dtype == CGNN_F32)
        return gather_typed<float, GATHER_RECONSTRUCT>(N, F, groups, reps, ids, nullptr, perm, bias, relu, out, bad_id, stream);
    if (dtype == CGNN_F64)
        return gather_typed<double, GATHER_RECONSTRUCT>(N, F, groups, reps, ids, nullptr, perm, bias, relu, out, bad_id, stream);
    return fail(CGNN_EUNSUPPORTED, "cgnn_reconstruct: dtype must be f32 or f64");
}

extern "C" int cgnn_reconstruct_backward(int64_t N, int64_t F, int64_t groups, int64_t max_members, int dtype,
                                         const void *grad, const void *output,
                                         const int32_t *offsets, const int32_t *perm,
                                         const int32_t *sorted_id, int relu, void *reps_grad,
                                         void *workspace, size_t workspace_bytes,
                                         cgnn_stream_t stream) {
    CGNN_REQUIRE(N >= 0 && F >= 0 && groups >= 0, "cgnn_reconstruct_backward: bad size");
    CGNN_REQUIRE(dtype == CGNN_F32 || dtype == CGNN_F64, "cgnn_reconstruct_backward: dtype must be f32 or f64");
    if (F == 0 || groups == 0) return CGNN_OK;
    CGNN_REQUIRE(offsets && reps_grad, "cgnn_reconstruct_backward: null array");
    CGNN_REQUIRE(N == 0 || (grad && perm && sorted_id), "cgnn_reconstruct_backward: null array");
    CGNN_REQUIRE(!relu || N == 0 || output, "cgnn_reconstruct_backward: relu needs the saved output");
    cgnn_csr A = members_csr(N, groups, offsets, perm, sorted_id, max_members);
    return spmm_members(&A, dtype, grad, output, reps_grad, F, relu != 0 ? 1 : 0, workspace, workspace_bytes,
                        stream);
}

extern "C" int64_t cgnn_sign_words(int64_t F) { return F <= 0 ? 0 : (F + 31) / 32; }

extern "C" int cgnn_reconstruct_signs(int64_t N, int64_t F, int64_t groups, int dtype, const void *reps,
                                      const int64_t *ids, const int32_t *perm, const void *bias, void *out,
                                      uint32_t *signs, int32_t *bad_id, cgnn_stream_t stream) {
    CGNN_REQUIRE(N >= 0 && F >= 0 && groups >= 0, "cgnn_reconstruct_signs: bad size");
    CGNN_REQUIRE(N == 0 || F == 0 || groups >= 1, "cgnn_reconstruct_signs: rows to reconstruct but no representatives");
    if (N == 0 || F == 0) return CGNN_OK;
    CGNN_REQUIRE(reps && ids && out && signs, "cgnn_reconstruct_signs: null array");
    if (dtype == CGNN_F32)
        return gather_typed<float, GATHER_RECONSTRUCT>(N, F, groups, reps, ids, nullptr, perm, bias, 1, out, bad_id, stream, signs);
    if (dtype == CGNN_F64)
        return gather_typed<double, GATHER_RECONSTRUCT>(N, F, groups, reps, ids, nullptr, perm, bias, 1, out, bad_id, stream, signs);
    return fail(CGNN_EUNSUPPORTED, "cgnn_reconstruct_signs: dtype must be f32 or f64");
}

extern "C" int cgnn_reconstruct_backward_signs(int64_t N, int64_t F, int64_t groups, int64_t max_members, int dtype,
                                               const void *grad, const uint32_t *signs, const int32_t *offsets,
                                               const int32_t *perm, const int32_t *sorted_id, void *reps_grad,
                                               void *workspace, size_t workspace_bytes, cgnn_stream_t stream) {
    CGNN_REQUIRE(N >= 0 && F >= 0 && groups >= 0, "cgnn_reconstruct_backward_signs: bad size");
    CGNN_REQUIRE(dtype == CGNN_F32 || dtype == CGNN_F64, "cgnn_reconstruct_backward_signs: dtype must be f32 or f64");
    if (F == 0 || groups == 0) return CGNN_OK;
    CGNN_REQUIRE(offsets && reps_grad, "cgnn_reconstruct_backward_signs: null array");
    CGNN_REQUIRE(N == 0 || (grad && perm && sorted_id && signs), "cgnn_reconstruct_backward_signs: null array");
    cgnn_csr A = members_csr(N, groups, offsets, perm, sorted_id, max_members);
    return spmm_members(&A, dtype, grad, signs, reps_grad, F, 2, workspace, workspace_bytes, stream);
}

extern "C" int cgnn_read_bytes(const void *src, size_t n, void *sink, cgnn_stream_t stream) {
    CGNN_REQUIRE(n % 16 == 0, "cgnn_read_bytes: size must be a multiple of 16");
    if (n == 0) return CGNN_OK;
    CGNN_REQUIRE(src && sink, "cgnn_read_bytes: null pointer");
    // two workgroups per compute unit: the shape that read fastest on MI355X
    hipLaunchKernelGGL(read16_kernel, dim3(2u * (unsigned)compute_units()), dim3(kBlock), 0, stream,
                       static_cast<const probe_word_t *>(src), n / 16, static_cast<uint32_t *>(sink));
    return check_launch("read_bytes");
}

extern "C" int cgnn_fill_bytes(void *dst, size_t n, cgnn_stream_t stream) {
    CGNN_REQUIRE(n % 16 == 0, "cgnn_fill_bytes: size must be a multiple of 16");
    if (n == 0) return CGNN_OK;
    CGNN_REQUIRE(dst, "cgnn_fill_bytes: null pointer");
    size_t blocks = (n / 16 + kBlock - 1) / kBlock;
    if (blocks > 8192) blocks = 8192;
    hipLaunchKernelGGL(fill16_kernel, dim3((unsigned)blocks), dim3(kBlock), 0, stream,
                       static_cast<probe_word_t *>(dst), n / 16);
    return check_launch("fill_bytes");
}

extern "C" int cgnn_copy_bytes(const void *src, void *dst, size_t n, cgnn_stream_t stream) {
    CGNN_REQUIRE(n % 16 == 0, "cgnn_copy_bytes: size must be a multiple of 16");
    if (n == 0) return CGNN_OK;
    CGNN_REQUIRE(src && dst, "cgnn_copy_bytes: null pointer");
    size_t blocks = (n / 16 + kBlock - 1) / kBlock;
    if (blocks > 8192) blocks = 8192;
    hipLaunchKernelGGL(copy16_kernel, dim3((unsigned)blocks), dim3(kBlock), 0, stream,
                       static_cast<const uint4 *>(src), static_cast<uint4 *>(dst), n / 16);
    return check_launch("copy_bytes");
}
